// Shared by the two MLA decode templates when they are built for a paged cache (AE_PAGED 1); included
// after AE_DV, AE_NT, AE_HEADS_PER_WG, AE_NSPLIT and AE_N_ROWSCALES are defined.
//
// Result of a (batch entry, kv head, head tile, split) that holds no key, written by the whole workgroup:
// zero output and -inf row scales, the same values the kernels' epilogues produce for an empty range,
// into `out` (one split) or into the split's partials (which the combine functor then ignores).
#pragma once

__device__ __forceinline__ void ae_mla_write_no_keys(const ae_attn_params& p, int b, int hk, int ht, int split,
                                                     int group, int tid) {
  for (int i = tid; i < AE_HEADS_PER_WG * (AE_DV / 4); i += AE_NT) {
    const int head_in_group = ht * AE_HEADS_PER_WG + i / (AE_DV / 4);
    const int col = (i % (AE_DV / 4)) * 4;
    if (head_in_group >= group) continue;
    const int hq = hk * group + head_in_group;
#if AE_NSPLIT == 1
    ae_elem* o = (ae_elem*)p.out + (int64_t)b * p.o_stride_b + (int64_t)hq * p.o_stride_h + col;
    *(ae_elem4*)o = (ae_elem4){(ae_elem)0.f, (ae_elem)0.f, (ae_elem)0.f, (ae_elem)0.f};
#else
    const int64_t row = ((int64_t)b * p.heads_q + hq) * p.num_splits + split;
    *(ae_f32x4*)(p.partial_o + row * AE_DV + col) = (ae_f32x4){0.f, 0.f, 0.f, 0.f};
#endif
  }
  for (int i = tid; i < AE_HEADS_PER_WG; i += AE_NT) {
    const int head_in_group = ht * AE_HEADS_PER_WG + i;
    if (head_in_group >= group) continue;
    const int hq = hk * group + head_in_group;
#pragma unroll
    for (int r = 0; r < AE_N_ROWSCALES; r++) {
#if AE_NSPLIT == 1
      if (p.rowscale_out[r]) p.rowscale_out[r][(int64_t)b * p.heads_q + hq] = AE_NEG_INF;
#else
      const int64_t row = ((int64_t)b * p.heads_q + hq) * p.num_splits + split;
      p.partial_rs[(int64_t)r * p.batch * p.heads_q * p.num_splits + row] = AE_NEG_INF;
#endif
    }
  }
}
