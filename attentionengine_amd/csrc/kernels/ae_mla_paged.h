// Shared by the two MLA decode templates when they are built for a paged cache (AE_PAGED 1); included
// after AE_DV, AE_NT, AE_HEADS_PER_WG, AE_NSPLIT and AE_N_ROWSCALES are defined.
//
// Splits of a batch entry that hold keys: ceil(length / kv_per_split).  An entry with at most one writes its
// result itself (split 0: `out` and the row scales, as a launch without splits does) and the merge kernel
// passes it over; the merge of a longer entry reads only the splits that hold keys.  Splits without keys
// write nothing.
//
// ae_mla_write_no_keys: result of an entry of length 0, written by the whole workgroup of its split 0: zero
// output and -inf row scales, the values the kernels' epilogues produce for an empty range.
#pragma once

__device__ __forceinline__ int ae_mla_splits_used(const ae_attn_params& p, int seqlen_b) {
  const int n = (seqlen_b + p.kv_per_split - 1) / p.kv_per_split;
  return n < p.num_splits ? n : p.num_splits;
}

__device__ __forceinline__ void ae_mla_write_no_keys(const ae_attn_params& p, int b, int hk, int ht, int group,
                                                     int tid) {
  for (int i = tid; i < AE_HEADS_PER_WG * (AE_DV / 4); i += AE_NT) {
    const int head_in_group = ht * AE_HEADS_PER_WG + i / (AE_DV / 4);
    const int col = (i % (AE_DV / 4)) * 4;
    if (head_in_group >= group) continue;
    const int hq = hk * group + head_in_group;
    ae_elem* o = (ae_elem*)p.out + (int64_t)b * p.o_stride_b + (int64_t)hq * p.o_stride_h + col;
    *(ae_elem4*)o = (ae_elem4){(ae_elem)0.f, (ae_elem)0.f, (ae_elem)0.f, (ae_elem)0.f};
  }
  for (int i = tid; i < AE_HEADS_PER_WG; i += AE_NT) {
    const int head_in_group = ht * AE_HEADS_PER_WG + i;
    if (head_in_group >= group) continue;
    const int hq = hk * group + head_in_group;
#pragma unroll
    for (int r = 0; r < AE_N_ROWSCALES; r++) {
      if (p.rowscale_out[r]) p.rowscale_out[r][(int64_t)b * p.heads_q + hq] = AE_NEG_INF;
    }
  }
}
