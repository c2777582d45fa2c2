// MLA (shared latent KV) split-KV decode for gfx950 / CDNA4.
//
// Takes the place of the reference's TileLang MLA decode template
// (attention_engine/core/template/tl_template/attn/mla_decode_tl.py: flash_attn_split 104-179) and of
// the CuTe/FlashMLA split kernel (core/template/cute_template_kvshared/kernels/splitkv_mla.cu:
// 1061-1393).  K = [latent | rope] (AE_D = AE_D1 + AE_D2 wide), V = the first AE_DV columns of the
// same rows, one kv head shared by all query heads of its group (128 for DeepSeek-V3).
//
// This is a GEMM-shaped problem (arithmetic intensity ~ 2*heads flop per KV byte), so it uses the
// prefill kernel's scheme with the query HEADS in the role of query rows:
//   * S^T[kv,head] = K Q^T and O^T[dv,head] += V^T P^T with v_mfma_f32_32x32x16; a lane owns one
//     head's online row state; Q stays in registers for the whole kernel (AE_D/16 fragments);
//   * a wave owns 32 heads and HALF of the value dimension: the full 32 x 512 fp32 accumulator
//     (256 registers) next to the Q fragments (144) cannot be rescaled in place, a half (128) can.
//     A workgroup is 4 waves = 2 head blocks x 2 value halves = 64 heads of one (batch, kv head,
//     split); the two waves of a head block compute the same scores;
//   * each KV tile is loaded into LDS once per workgroup and serves both products: K rows are read
//     with ds_read_b128, the V operand is read from the SAME LDS rows through ds_read_b64_tr_b16;
//   * the workgroups that share a KV range (the head tiles of one batch entry) get ids 8 apart, so
//     the round-robin dispatch puts them on the same XCD and the second reads the tile from its L2;
//   * one wave per SIMD (512-register budget);
//   * partial (o, rowscales) per split in fp32, merged by ae_decode_combine_kernel.

#include "ae_hip.h"
#include "ae_config.h"
#include "ae_device.h"
#include "ae_functors.h"

#define AE_D (AE_D1 + AE_D2)
#define AE_NT (AE_NWAVES * 64)
#define AE_HEADS_PER_WG ((AE_NWAVES / 2) * 32)
#define AE_NB (AE_BN / 32)
#define AE_NS (AE_NB * 16)
#define AE_NDB (AE_DV / 64)              // 32-wide dv blocks of this wave's half of DV
#define AE_NO (AE_NDB * 16)
#define AE_KSTR (AE_D * 2 + AE_K_PAD)
#define AE_STAGE_BYTES (AE_BN * AE_KSTR)
#define AE_CPR (AE_D / 8)                // 16-byte chunks per K row
#define AE_CPR1 (AE_D1 / 8)              // chunks that come from the latent tensor
#define AE_LOADS ((AE_BN * AE_CPR + AE_NT - 1) / AE_NT)

static_assert(AE_D1 % 16 == 0 && AE_D2 % 16 == 0, "latent / rope dims must be multiples of 16");
static_assert(AE_DV % 64 == 0 && AE_DV <= AE_D1, "V must be a prefix of the latent part");
static_assert(AE_NWAVES % 2 == 0, "waves come in (head block, value half) pairs");
static_assert(AE_BN % 32 == 0, "kv tile must be a multiple of 32");

typedef __attribute__((address_space(3))) unsigned char ae_lds_byte;

extern "C" __global__ __launch_bounds__(AE_NT)
__attribute__((amdgpu_waves_per_eu(1, 1)))
void ae_mla_decode_split_kernel(const ae_attn_params p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ae_smem[];
  ae_lds_byte* lds = (ae_lds_byte*)ae_smem;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hf = lane >> 5;

  // ---- which (head tile, split, kv head, batch): 1-D grid, ids 8 apart share their KV range ---------
  const int group = p.heads_q / p.heads_kv;
  const int n_ht = (group + AE_HEADS_PER_WG - 1) / AE_HEADS_PER_WG;
  const int wg = blockIdx.x;
  const int ht = (wg >> 3) % n_ht;
  const int u = (wg / (8 * n_ht)) * 8 + (wg & 7);        // flattened (batch, kv head, split)
  if (u >= p.batch * p.heads_kv * p.num_splits) return;  // grid padding (whole workgroup exits)
  const int split = u % p.num_splits;
  const int hk = (u / p.num_splits) % p.heads_kv;
  const int b = u / (p.num_splits * p.heads_kv);
  const int hblk = wave >> 1;     // which 32 heads of the workgroup
  const int dvh = wave & 1;       // which half of the value dimension
  const int head_in_group = ht * AE_HEADS_PER_WG + hblk * 32 + l32;
  const bool head_ok = head_in_group < group;
  const int hq = hk * group + (head_ok ? head_in_group : 0);

  // ---- Q fragments: B operand of S^T = K Q^T (n = head, k = d) ------------------------------------
  const ae_elem* q1 = (const ae_elem*)p.q + (int64_t)b * p.q_stride_b + (int64_t)hq * p.q_stride_h;
  const ae_elem* q2 = (const ae_elem*)p.q2 + (int64_t)b * p.q2_stride_b + (int64_t)hq * p.q2_stride_h;
  ae_elem8 qf[AE_D / 16];
#pragma unroll
  for (int ks = 0; ks < AE_D1 / 16; ks++) qf[ks] = *(const ae_elem8*)(q1 + ks * 16 + hf * 8);
#pragma unroll
  for (int ks = 0; ks < AE_D2 / 16; ks++) qf[AE_D1 / 16 + ks] = *(const ae_elem8*)(q2 + ks * 16 + hf * 8);

  const ae_elem* k1 = (const ae_elem*)p.k + (int64_t)b * p.k_stride_b + (int64_t)hk * p.k_stride_h;
  const ae_elem* k2 = (const ae_elem*)p.k2 + (int64_t)b * p.k2_stride_b + (int64_t)hk * p.k2_stride_h;

  const int kv_begin = split * p.kv_per_split;
  int kv_end = kv_begin + p.kv_per_split;
  kv_end = kv_end < p.seqlen_kv ? kv_end : p.seqlen_kv;
  const int n_tiles = kv_end > kv_begin ? (kv_end - kv_begin + AE_BN - 1) / AE_BN : 0;

  ae_u32x4 kreg[AE_LOADS];
  auto load_tile = [&](int t) {
    const int kv0 = kv_begin + t * AE_BN;
#pragma unroll
    for (int i = 0; i < AE_LOADS; i++) {
      int c = tid + i * AE_NT;
      if ((AE_BN * AE_CPR) % AE_NT == 0 || c < AE_BN * AE_CPR) {
        int row = c / AE_CPR, col = c % AE_CPR;
        int kv = kv0 + row;
        kv = kv < p.seqlen_kv ? kv : p.seqlen_kv - 1;
        const ae_elem* src = col < AE_CPR1 ? k1 + (int64_t)kv * p.k_stride_s + col * 8
                                           : k2 + (int64_t)kv * p.k2_stride_s + (col - AE_CPR1) * 8;
        kreg[i] = *(const ae_u32x4*)src;
      }
    }
  };
  auto store_tile = [&](int stage) {
    ae_lds_byte* ks = lds + stage * AE_STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < AE_LOADS; i++) {
      int c = tid + i * AE_NT;
      if ((AE_BN * AE_CPR) % AE_NT == 0 || c < AE_BN * AE_CPR) {
        int row = c / AE_CPR, col = c % AE_CPR;
        *(__attribute__((address_space(3))) ae_u32x4*)(ks + row * AE_KSTR + col * 16) = kreg[i];
      }
    }
  };

  ae_ctx ctx;
  ctx.b = b;
  ctx.h = hq;
  ctx.q_idx = 0;
  ctx.kv_base = 0;
  ae_custom cust;
  ae_load_custom(cust, p, ctx);
  ae_rowstate st;
  ae_rowstate_init(st);
  ae_f32x16 oacc[AE_NDB];
#pragma unroll
  for (int db = 0; db < AE_NDB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[db][r] = 0.f;

  const int k_rd_off = l32 * AE_KSTR + hf * 16;
  const int v_rd_off = (4 * hf + ((lane & 15) >> 2)) * AE_KSTR + ((l32 >> 4) * 16 + 4 * (lane & 3)) * 2;

  if (n_tiles > 0) {
    load_tile(0);
    store_tile(0);
  }
  __syncthreads();

  int stage = 0;
  for (int t = 0; t < n_tiles; t++) {
    const bool more = t + 1 < n_tiles;
    if (more) load_tile(t + 1);
    ae_lds_byte* ks_ = lds + stage * AE_STAGE_BYTES;
    const int kv0 = kv_begin + t * AE_BN;

    ae_f32x16 sacc[AE_NB];
#pragma unroll
    for (int nb = 0; nb < AE_NB; nb++)
#pragma unroll
      for (int r = 0; r < 16; r++) sacc[nb][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < AE_D / 16; ks++) {
#pragma unroll
      for (int nb = 0; nb < AE_NB; nb++) {
        ae_elem8 kf = *(__attribute__((address_space(3))) ae_elem8*)(
            ks_ + k_rd_off + nb * 32 * AE_KSTR + ks * 32);
        sacc[nb] = ae_mfma32(kf, qf[ks], sacc[nb]);
      }
    }
    float s[AE_NS];
#pragma unroll
    for (int nb = 0; nb < AE_NB; nb++)
#pragma unroll
      for (int r = 0; r < 16; r++) s[nb * 16 + r] = sacc[nb][r];

    ctx.kv_base = kv0 + 4 * hf;
    const bool tail = kv0 + AE_BN > kv_end;
    if (tail) {
#pragma unroll
      for (int e = 0; e < AE_NS; e++) s[e] = (ctx.kv_base + ae_kv_off(e) < kv_end) ? s[e] : AE_NEG_INF;
    }
    ae_score_mod<AE_NS>(s, ctx, cust);
    float o_scale = ae_online_fwd<AE_NS>(s, st, ctx, cust);
    if (tail) {
#pragma unroll
      for (int e = 0; e < AE_NS; e++) s[e] = (ctx.kv_base + ae_kv_off(e) < kv_end) ? s[e] : 0.f;
    }
    ae_elem8 pf[AE_BN / 16];
#pragma unroll
    for (int kk = 0; kk < AE_BN / 16; kk++)
#pragma unroll
      for (int j = 0; j < 8; j++) pf[kk][j] = (ae_elem)s[kk * 8 + j];

#if !AE_O_SCALE_ONE
#pragma unroll
    for (int db = 0; db < AE_NDB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[db][r] *= o_scale;
#else
    (void)o_scale;
#endif

    // O^T += V^T P^T with V = the first AE_DV columns of the K rows already in LDS
#pragma unroll
    for (int kk = 0; kk < AE_BN / 16; kk++) {
      const int rb = (kk >> 1) * 32 + (kk & 1) * 16;
#pragma unroll
      for (int db = 0; db < AE_NDB; db++) {
        ae_lds_byte* a0 = ks_ + v_rd_off + rb * AE_KSTR + (dvh * AE_NDB + db) * 64;
        ae_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) ae_s16x4*)a0);
        ae_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) ae_s16x4*)(a0 + 8 * AE_KSTR));
        ae_elem8 vf = __builtin_bit_cast(
            ae_elem8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        oacc[db] = ae_mfma32(vf, pf[kk], oacc[db]);
      }
    }

    if (more) store_tile(stage ^ 1);
    __syncthreads();
    stage ^= 1;
  }

  // ---- per-split epilogue ------------------------------------------------------------------------------
  float o[AE_NO];
#pragma unroll
  for (int db = 0; db < AE_NDB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[db * 16 + r] = oacc[db][r];
  float frs[AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1];
  frs[0] = 0.f;
  if (n_tiles > 0) {
    ae_epilogue<AE_NO>(o, st, frs, ctx, cust);
  } else {
#pragma unroll
    for (int e = 0; e < AE_NO; e++) o[e] = 0.f;
#pragma unroll
    for (int i = 0; i < AE_N_ROWSCALES; i++) frs[i] = AE_NEG_INF;
  }
  if (head_ok) {
    const int64_t row = ((int64_t)b * p.heads_q + hq) * p.num_splits + split;
    float* po = p.partial_o + row * AE_DV + dvh * (AE_DV / 2);
#pragma unroll
    for (int db = 0; db < AE_NDB; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        ae_f32x4 w = {o[db * 16 + rg * 4 + 0], o[db * 16 + rg * 4 + 1], o[db * 16 + rg * 4 + 2],
                      o[db * 16 + rg * 4 + 3]};
        *(ae_f32x4*)(po + db * 32 + rg * 8 + hf * 4) = w;
      }
    if (hf == 0 && dvh == 0) {
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++)
        p.partial_rs[(int64_t)i * p.batch * p.heads_q * p.num_splits + row] = frs[i];
    }
  }
}

#include "ae_combine.h"
