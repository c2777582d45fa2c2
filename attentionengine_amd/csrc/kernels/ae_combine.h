// Merge kernel of the split-KV decode paths (shared by ae_decode.hip and ae_mla_decode.hip).
// Needs AE_DV, AE_NSPLIT, AE_N_ROWSCALES, AE_COMBINE_THREADS and the generated ae_combine().
#ifndef AE_COMBINE_H
#define AE_COMBINE_H

// Merge of the per-split partials: grid (Hq, B), one workgroup per output row.
// out[b,0,h,:] = sum_k partial_o[b,h,k,:] * o_scale[k], o_scale = combine(final_rowscales[k])
// (attn_gqa_decode_tl.py:224-266; generic form core/template/tl_template/attn/attn_decode_tl.py:184-189).
extern "C" __global__ __launch_bounds__(AE_COMBINE_THREADS)
void ae_decode_combine_kernel(const ae_attn_params p) {
  const int h = blockIdx.x;
  const int b = blockIdx.y;
  const int64_t row = ((int64_t)b * p.heads_q + h) * AE_NSPLIT;
  // Paged cache (per-entry lengths): only the first ceil(length / kv_per_split) splits of an entry hold keys and
  // wrote partial results; an entry with at most one wrote `out` itself.
  int n_used = AE_NSPLIT;
  if (p.seqlens_k != nullptr) {
    int len = p.seqlens_k[b];
    len = len < p.seqlen_kv ? len : p.seqlen_kv;
    const int n = ((len > 0 ? len : 0) + p.kv_per_split - 1) / p.kv_per_split;
    n_used = n < AE_NSPLIT ? n : AE_NSPLIT;
    if (n_used <= 1) return;
  }
  float rs[AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1][AE_NSPLIT];
#pragma unroll
  for (int i = 0; i < AE_N_ROWSCALES; i++)
#pragma unroll
    for (int k = 0; k < AE_NSPLIT; k++)
      rs[i][k] = k < n_used ? p.partial_rs[(int64_t)i * p.batch * p.heads_q * AE_NSPLIT + row + k] : AE_NEG_INF;
  float w[AE_NSPLIT];
  float merged[AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1];
  ae_combine(rs, w, merged);
  ae_elem* optr = (ae_elem*)p.out + (int64_t)b * p.o_stride_b + (int64_t)h * p.o_stride_h;
  for (int dv = threadIdx.x; dv < AE_DV; dv += AE_COMBINE_THREADS) {
    // The partial results are read 16 splits at a time, unconditionally, so that the loads of a group all go
    // out before the first one is waited for (one memory round trip per group instead of one per split: the
    // merge of 32 splits 18 -> 4 us).  Splits that wrote nothing re-read the last one that did, with weight 0.
    float acc = 0.f;
    constexpr int G = AE_NSPLIT < 16 ? AE_NSPLIT : 16;
#pragma unroll
    for (int k0 = 0; k0 < AE_NSPLIT; k0 += G) {
      float val[G];
#pragma unroll
      for (int i = 0; i < G; i++) {
        const int k = k0 + i < AE_NSPLIT ? k0 + i : AE_NSPLIT - 1;
        const int kc = k < n_used ? k : n_used - 1;
        val[i] = p.partial_o[(row + kc) * AE_DV + dv];
      }
#pragma unroll
      for (int i = 0; i < G; i++) {
        const int k = k0 + i;
        acc += val[i] * ((k < AE_NSPLIT && k < n_used) ? w[k < AE_NSPLIT ? k : 0] : 0.f);
      }
    }
    optr[dv] = (ae_elem)acc;
  }
  if (threadIdx.x == 0) {
    // One-token decode: row scales [B, Hq].  Split-KV prefill (p.seqlen_q > 1: its launch hands the (q position,
    // head) pairs over as p.heads_q = Sq * Hq "heads", h = s * Hq + head): row scales [B, Hq, Sq], the layout of
    // the unsplit kernels.
    int64_t at = (int64_t)b * p.heads_q + h;
    if (p.seqlen_q > 1) {
      const int hq = p.heads_q / p.seqlen_q;
      at = ((int64_t)b * hq + h % hq) * p.seqlen_q + h / hq;
    }
#pragma unroll
    for (int i = 0; i < AE_N_ROWSCALES; i++)
      if (p.rowscale_out[i]) p.rowscale_out[i][at] = merged[i];
  }
}

#endif  // AE_COMBINE_H
