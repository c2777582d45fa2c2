// Split-KV attention decode (one query token per sequence) for gfx950 / CDNA4, and the kernel
// that merges the per-split partial results.
//
// Takes the place of the reference's TileLang GQA decode template
// (attention_engine/core/template/tl_template/attn/attn_gqa_decode_tl.py: flash_attn_split 141-222,
// combine 224-266).  Unlike that template, which hard-codes softmax (52-67), score_mod / online_func
// / combine come from the traced user functions ("ae_config.h" / "ae_functors.h").
//
// The kernel is HBM-bound: every K and V element is read exactly once and used for all query
// heads of its group, so the design goal is bytes in flight, not MFMA occupancy.
//   * one WAVE owns an independent partial result ("split"): it walks its own 32-row kv tiles,
//     keeps (acc_o, rowstate) in registers and writes fp32 partial (o, rowscales); waves never
//     synchronise with each other, there is no workgroup barrier in the loop;
//   * the query heads of one kv head (<= 16 per workgroup) are the N dimension of
//     v_mfma_f32_16x16x32: S^T[kv,head] = K Q^T, O^T[dv,head] += V^T P^T, the same transposed
//     scheme as the prefill kernel, so a lane owns one head's row state;
//   * K rows go straight from HBM into the MFMA A-operand registers (no transpose needed: the
//     contraction index d is contiguous in memory), prefetched one tile ahead;
//   * V rows are loaded with coalesced 16-byte accesses into a wave-private LDS tile and read back
//     with ds_read_b64_tr_b16, which delivers the kv-contiguous A operand of the PV product;
//   * partials are fp32 [B,Hq,splits,DV] + fp32 rowscales [n,B,Hq,splits] (the CuTe backend's
//     convention, cute_template_kvshared/flash_api.cpp:180-181); the combine kernel evaluates the
//     user's combine() per (batch, head) and writes out [B,1,Hq,DV] and the merged rowscales.

#define AE_LAYOUT 1
#include "ae_hip.h"
#include "ae_config.h"
#include "ae_device.h"
#include "ae_functors.h"

#define AE_NT (AE_NWAVES * 64)
#define AE_TILE 32                      // kv rows per wave tile
#define AE_NS 8                         // score elements per lane per tile (2 blocks of 4)
#define AE_NDB (AE_DV / 16)             // 16-wide dv blocks
#define AE_NO (AE_NDB * 4)              // output elements per lane
#define AE_NKS (AE_D / 32)              // 32-deep k-steps of QK^T
#define AE_VSTR (AE_DV * 2 + AE_V_PAD)  // LDS row pitch of the V tile, bytes
#define AE_V_WAVE_BYTES (AE_TILE * AE_VSTR)
#define AE_VCPR (AE_DV / 8)             // 16-byte chunks per V row
#define AE_V_LOADS ((AE_TILE * AE_VCPR) / 64)

// 1: the launch has ONE workgroup per (batch, kv head, head tile), i.e. its AE_NWAVES waves hold all AE_NSPLIT
// partial results: they meet in LDS (each wave's V tile region, 16 heads x DV fp32, and the row scales behind
// the tiles) and the workgroup merges them and writes out and the merged row scales itself - no work buffers,
// no second launch (5 us of a batched decode call, 1.3 % of the C4 one).
#ifndef AE_MERGE_IN_WG
#define AE_MERGE_IN_WG 0
#endif
// 1: launches that share the kv axis of a (batch, kv head, head tile) out over SEVERAL workgroups merge in the
// workgroup that finishes last instead of in a second launch: every workgroup writes its partial results with
// device-scope stores, waits for them, then counts itself in with an atomic add on a counter of its (batch, kv head,
// head tile); the one that reads gridDim.x - 1 is the last, sets the counter back to zero for the next launch, and
// merges all AE_NSPLIT partial results in the order of ae_decode_combine_kernel (equal results to the last bit).  The
// counters are 32-bit integers behind the row scales in p.partial_rs (after max(1, AE_N_ROWSCALES) * batch * heads_q *
// num_splits floats), one per (batch, blockIdx.y); they must be zero before the first launch and are left at zero by
// every launch.  Saves the second launch and the gap in front of it: 2 to 4 us of a 20 us call at batch 1.
#ifndef AE_MERGE_LAST
#define AE_MERGE_LAST 0
#endif
static_assert(!(AE_MERGE_IN_WG && AE_MERGE_LAST), "one way to merge");
static_assert(!AE_MERGE_IN_WG || AE_NSPLIT == AE_NWAVES, "the workgroup merges exactly its own waves' partial results");
static_assert(AE_D % 32 == 0, "head dim must be a multiple of 32");
static_assert(AE_DV % 16 == 0, "value head dim must be a multiple of 16");
static_assert((AE_TILE * AE_VCPR) % 64 == 0, "V tile must split evenly over a wave");

typedef __attribute__((address_space(3))) unsigned char ae_lds_byte;

extern "C" __global__ __launch_bounds__(AE_NT)
__attribute__((amdgpu_waves_per_eu(AE_WAVES_PER_EU, AE_WAVES_PER_EU)))
void ae_decode_split_kernel(const ae_attn_params p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ae_smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15;
  const int g4 = lane >> 4;
  ae_lds_byte* vs = (ae_lds_byte*)ae_smem + wave * AE_V_WAVE_BYTES;

  // ---- which (batch, kv head, head tile, split) ------------------------------------------------
  const int group = p.heads_q / p.heads_kv;
  const int b = blockIdx.z;
  const int hk = blockIdx.y % p.heads_kv;
  const int ht = blockIdx.y / p.heads_kv;
  const int split = blockIdx.x * AE_NWAVES + wave;       // index of this wave's partial
  const int head_in_group = ht * 16 + l16;
  const bool head_ok = head_in_group < group;
  const int hq = hk * group + (head_ok ? head_in_group : 0);

  // this workgroup covers kv [wg_base, wg_base + AE_NWAVES*kv_per_split); wave w takes the tiles
  // w, w+NWAVES, ... of that range, so the workgroup streams one contiguous region of HBM
  const int wg_base = blockIdx.x * AE_NWAVES * p.kv_per_split;
  const int n_tiles = p.kv_per_split / AE_TILE;

  // ---- Q fragments (B operand of S^T = K Q^T): n = head = l16, k = d = 32*ks + 8*g4 + j ---------
  const ae_elem* qptr = (const ae_elem*)p.q + (int64_t)b * p.q_stride_b + (int64_t)hq * p.q_stride_h;
  ae_elem8 qf[AE_NKS];
#pragma unroll
  for (int ks = 0; ks < AE_NKS; ks++) qf[ks] = *(const ae_elem8*)(qptr + ks * 32 + g4 * 8);

  const ae_elem* kbase = (const ae_elem*)p.k + (int64_t)b * p.k_stride_b + (int64_t)hk * p.k_stride_h;
  const ae_elem* vbase = (const ae_elem*)p.v + (int64_t)b * p.v_stride_b + (int64_t)hk * p.v_stride_h;

  ae_elem8 kf[2][AE_NKS];       // K of the current tile, A-operand layout: m = kv = 16*rb + l16
  ae_elem8 kf_next[2][AE_NKS];
  ae_u32x4 vreg[AE_V_LOADS];

  auto tile_kv0 = [&](int i) AE_LAMBDA { return wg_base + (wave + i * AE_NWAVES) * AE_TILE; };
  auto clamp_kv = [&](int kv) AE_LAMBDA {
#if AE_EVEN_KV
    return kv;
#else
    return kv < p.seqlen_kv ? kv : p.seqlen_kv - 1;
#endif
  };
  auto load_k = [&](int kv0, ae_elem8 (&dst)[2][AE_NKS]) AE_LAMBDA {
#pragma unroll
    for (int rb = 0; rb < 2; rb++) {
      const ae_elem* row = kbase + (int64_t)clamp_kv(kv0 + rb * 16 + l16) * p.k_stride_s + g4 * 8;
#pragma unroll
      for (int ks = 0; ks < AE_NKS; ks++) dst[rb][ks] = *(const ae_elem8*)(row + ks * 32);
    }
  };
  auto load_v = [&](int kv0) AE_LAMBDA {
#pragma unroll
    for (int i = 0; i < AE_V_LOADS; i++) {
      int c = lane + i * 64;
      int row = c / AE_VCPR, col = c % AE_VCPR;
      vreg[i] = *(const ae_u32x4*)(vbase + (int64_t)clamp_kv(kv0 + row) * p.v_stride_s + col * 8);
    }
  };
  auto store_v = [&]() AE_LAMBDA {
#pragma unroll
    for (int i = 0; i < AE_V_LOADS; i++) {
      int c = lane + i * 64;
      int row = c / AE_VCPR, col = c % AE_VCPR;
      *(__attribute__((address_space(3))) ae_u32x4*)(vs + row * AE_VSTR + col * 16) = vreg[i];
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
  ae_f32x4 oacc[AE_NDB];
#pragma unroll
  for (int db = 0; db < AE_NDB; db++) oacc[db] = (ae_f32x4){0.f, 0.f, 0.f, 0.f};

  // tiles of this wave that start inside the sequence
  int my_tiles = 0;
  for (int i = 0; i < n_tiles; i++)
    if (tile_kv0(i) < p.seqlen_kv) my_tiles = i + 1;

  if (my_tiles > 0) {
    load_k(tile_kv0(0), kf);
    load_v(tile_kv0(0));
  }
  // transpose-read offset: lane i of a 16-lane group reads row (i/4), 4 columns from 4*(i%4)
  const int v_rd_off = (4 * g4 + (l16 >> 2)) * AE_VSTR + (4 * (l16 & 3)) * 2;

  for (int i = 0; i < my_tiles; i++) {
    const int kv0 = tile_kv0(i);
    store_v();                          // V(i): registers -> LDS (previous tile's reads are done)
    const bool more = i + 1 < my_tiles;
    if (more) {
      load_k(tile_kv0(i + 1), kf_next);
      load_v(tile_kv0(i + 1));
    }

    // ---- S^T = K Q^T: two 16-row kv blocks -------------------------------------------------------
    ae_f32x4 sacc[2];
#pragma unroll
    for (int rb = 0; rb < 2; rb++) {
      sacc[rb] = (ae_f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < AE_NKS; ks++) sacc[rb] = ae_mfma16(kf[rb][ks], qf[ks], sacc[rb]);
    }
    float s[AE_NS];
#pragma unroll
    for (int rb = 0; rb < 2; rb++)
#pragma unroll
      for (int r = 0; r < 4; r++) s[rb * 4 + r] = sacc[rb][r];

    ctx.kv_base = kv0 + 4 * g4;
#if !AE_EVEN_KV
    if (kv0 + AE_TILE > p.seqlen_kv) {
#pragma unroll
      for (int e = 0; e < AE_NS; e++)
        s[e] = (ctx.kv_base + ae_kv_off(e) < p.seqlen_kv) ? s[e] : AE_NEG_INF;
    }
#endif
    ae_score_mod<AE_NS>(s, ctx, cust);
    float o_scale = ae_online_fwd<AE_NS>(s, st, ctx, cust);
#if !AE_EVEN_KV
    if (kv0 + AE_TILE > p.seqlen_kv) {
#pragma unroll
      for (int e = 0; e < AE_NS; e++)
        s[e] = (ctx.kv_base + ae_kv_off(e) < p.seqlen_kv) ? s[e] : 0.f;
    }
#endif
    // P as B operand of O^T += V^T P^T: slot j<4 is kv 4*g4+j, slot j>=4 is kv 16+4*g4+(j-4)
    ae_elem8 pf;
#pragma unroll
    for (int t = 0; t < 8; t++) pf[t] = (ae_elem)s[t];

#if !AE_O_SCALE_ONE
#pragma unroll
    for (int db = 0; db < AE_NDB; db++)
#pragma unroll
      for (int r = 0; r < 4; r++) oacc[db][r] *= o_scale;
#else
    (void)o_scale;
#endif

    // make this wave's LDS writes visible to its own transpose reads
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int db = 0; db < AE_NDB; db++) {
      ae_lds_byte* a0 = vs + v_rd_off + db * 32;
      ae_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) ae_s16x4*)a0);
      ae_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) ae_s16x4*)(a0 + 16 * AE_VSTR));
      ae_elem8 vf = __builtin_bit_cast(
          ae_elem8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      oacc[db] = ae_mfma16(vf, pf, oacc[db]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    if (more) {
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int ks = 0; ks < AE_NKS; ks++) kf[rb][ks] = kf_next[rb][ks];
    }
  }

  // ---- per-split epilogue: normalise within the split, emit its final rowscales ------------------
  float o[AE_NO];
#pragma unroll
  for (int db = 0; db < AE_NDB; db++)
#pragma unroll
    for (int r = 0; r < 4; r++) o[db * 4 + r] = oacc[db][r];
  float frs[AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1];
  frs[0] = 0.f;
  if (my_tiles > 0) {
    ae_epilogue<AE_NO>(o, st, frs, ctx, cust);
  } else {
    // this split saw no kv at all: contributes nothing to the merge
#pragma unroll
    for (int e = 0; e < AE_NO; e++) o[e] = 0.f;
#pragma unroll
    for (int i = 0; i < AE_N_ROWSCALES; i++) frs[i] = AE_NEG_INF;
  }
#if AE_MERGE_IN_WG
  {
    // (the wave's V tile region is its own, and its last transposed reads have returned: O was computed from them)
    __attribute__((address_space(3))) float* mo = (__attribute__((address_space(3))) float*)vs;
    __attribute__((address_space(3))) float* mrs =
        (__attribute__((address_space(3))) float*)((ae_lds_byte*)ae_smem + AE_NWAVES * AE_V_WAVE_BYTES);
#pragma unroll
    for (int db = 0; db < AE_NDB; db++) {
      ae_f32x4 w = {o[db * 4 + 0], o[db * 4 + 1], o[db * 4 + 2], o[db * 4 + 3]};
      *(__attribute__((address_space(3))) ae_f32x4*)(mo + l16 * AE_DV + db * 16 + g4 * 4) = w;
    }
    if (g4 == 0) {
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++) mrs[(i * AE_NWAVES + wave) * 16 + l16] = frs[i];
    }
    __syncthreads();
    for (int idx = tid; idx < 16 * AE_DV; idx += AE_NT) {
      const int hl = idx / AE_DV, dv = idx % AE_DV;
      if (ht * 16 + hl >= group) continue;
      const int hq2 = hk * group + ht * 16 + hl;
      float rs[AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1][AE_NSPLIT];
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++)
#pragma unroll
        for (int k = 0; k < AE_NSPLIT; k++) rs[i][k] = mrs[(i * AE_NWAVES + k) * 16 + hl];
      float w[AE_NSPLIT];
      float merged[AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1];
      ae_combine(rs, w, merged);
      float acc = 0.f;
#pragma unroll
      for (int k = 0; k < AE_NSPLIT; k++)
        acc += ((__attribute__((address_space(3))) float*)((ae_lds_byte*)ae_smem + k * AE_V_WAVE_BYTES))[hl * AE_DV + dv] * w[k];
      ((ae_elem*)p.out)[(int64_t)b * p.o_stride_b + (int64_t)hq2 * p.o_stride_h + dv] = (ae_elem)acc;
      if (dv == 0) {
#pragma unroll
        for (int i = 0; i < AE_N_ROWSCALES; i++)
          if (p.rowscale_out[i]) p.rowscale_out[i][(int64_t)b * p.heads_q + hq2] = merged[i];
      }
    }
    (void)split;
    return;
  }
#endif
#if AE_MERGE_LAST
  // The partial results of the tile's heads, as one buffer for device-scope accesses (sc1: stores are written
  // through this XCD's L2, loads do not take a line the L2 may still hold from an earlier launch -- the merging
  // workgroup may sit on another XCD.  A device-scope release / acquire fence pair instead writes back and
  // invalidates the whole L2: measured at several microseconds a workgroup, twice the call at batch 4).
  constexpr int kDeviceScope = 16;     // the sc1 bit of a buffer instruction's cache policy
  const int tile_heads = group - ht * 16 < 16 ? group - ht * 16 : 16;
  const int64_t tile_row0 = ((int64_t)b * p.heads_q + hk * group + ht * 16) * p.num_splits;
  __amdgpu_buffer_rsrc_t po_buf = __builtin_amdgcn_make_buffer_rsrc(
      p.partial_o + tile_row0 * AE_DV, 0, tile_heads * p.num_splits * AE_DV * 4, 0x00020000);
  if (head_ok) {
    const int row_in_tile = l16 * p.num_splits + split;
#pragma unroll
    for (int db = 0; db < AE_NDB; db++) {
      ae_f32x4 w = {o[db * 4 + 0], o[db * 4 + 1], o[db * 4 + 2], o[db * 4 + 3]};
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(ae_u32x4, w), po_buf,
                                             (row_in_tile * AE_DV + db * 16 + g4 * 4) * 4, 0, kDeviceScope);
    }
    if (g4 == 0) {
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++)
        __hip_atomic_store(p.partial_rs + (int64_t)i * p.batch * p.heads_q * p.num_splits + tile_row0 + row_in_tile,
                           frs[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  {
    // Every wave waits until its stores above have been acknowledged (stores count in vmcnt; the barrier alone
    // does not wait for them: a workgroup-scope release on this target orders only what the waves of one CU see),
    // then the workgroup meets and counts itself in: no partial result is still travelling when the counter moves.
    __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0), the other counters left alone
    __syncthreads();                   // (every wave is also past its last tile: the V tile regions are free)
    __attribute__((address_space(3))) int* flag = (__attribute__((address_space(3))) int*)ae_smem;
    if (tid == 0) {
      int* counter = (int*)(p.partial_rs + (int64_t)(AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1) * p.batch * p.heads_q *
                                               p.num_splits) + (blockIdx.z * gridDim.y + blockIdx.y);
      const int seen = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int last = seen == (int)gridDim.x - 1;
      // (nobody else touches the counter until the next launch)
      if (last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *flag = last;
    }
    __syncthreads();
    if (*flag == 0) return;
    // Every other workgroup's partial results were in memory before it counted itself in.  One thread merges four
    // neighbouring output columns of one head; its loads of the row scales (the same addresses for the 32 threads
    // of a head) and of the first partial results go out together: one trip to memory, not one after the other.
    for (int idx = tid; idx < tile_heads * (AE_DV / 4); idx += AE_NT) {
      const int hl = idx / (AE_DV / 4), dv = (idx % (AE_DV / 4)) * 4;
      const int hq2 = hk * group + ht * 16 + hl;
      float rs[AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1][AE_NSPLIT];
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++)
#pragma unroll
        for (int k = 0; k < AE_NSPLIT; k++)
          rs[i][k] = __hip_atomic_load(p.partial_rs + (int64_t)i * p.batch * p.heads_q * p.num_splits + tile_row0 +
                                           hl * AE_NSPLIT + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      constexpr int G = AE_NSPLIT < 16 ? AE_NSPLIT : 16;     // partial results in flight at a time
      ae_f32x4 val[G];
#pragma unroll
      for (int i = 0; i < G; i++)
        val[i] = __builtin_bit_cast(ae_f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                                  po_buf, ((hl * AE_NSPLIT + i) * AE_DV + dv) * 4, 0, kDeviceScope));
      float w[AE_NSPLIT];
      float merged[AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1];
      ae_combine(rs, w, merged);
      // (the sum runs over the splits in ascending order, as in ae_decode_combine_kernel: equal to the last bit)
      ae_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int k0 = 0; k0 < AE_NSPLIT; k0 += G) {
        if (k0 > 0) {
#pragma unroll
          for (int i = 0; i < G; i++)
            if (k0 + i < AE_NSPLIT)
              val[i] = __builtin_bit_cast(ae_f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                                        po_buf, ((hl * AE_NSPLIT + k0 + i) * AE_DV + dv) * 4, 0, kDeviceScope));
        }
#pragma unroll
        for (int i = 0; i < G; i++)
          if (k0 + i < AE_NSPLIT) {
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] += val[i][r] * w[k0 + i];
          }
      }
      ae_elem* orow = (ae_elem*)p.out + (int64_t)b * p.o_stride_b + (int64_t)hq2 * p.o_stride_h + dv;
#pragma unroll
      for (int r = 0; r < 4; r++) orow[r] = (ae_elem)acc[r];
      if (dv == 0) {
#pragma unroll
        for (int i = 0; i < AE_N_ROWSCALES; i++)
          if (p.rowscale_out[i]) p.rowscale_out[i][(int64_t)b * p.heads_q + hq2] = merged[i];
      }
    }
  }
#else
  if (head_ok) {
    const int64_t row = ((int64_t)b * p.heads_q + hq) * p.num_splits + split;
    float* po = p.partial_o + row * AE_DV;
#pragma unroll
    for (int db = 0; db < AE_NDB; db++) {
      ae_f32x4 w = {o[db * 4 + 0], o[db * 4 + 1], o[db * 4 + 2], o[db * 4 + 3]};
      *(ae_f32x4*)(po + db * 16 + g4 * 4) = w;
    }
    if (g4 == 0) {
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++)
        p.partial_rs[(int64_t)i * p.batch * p.heads_q * p.num_splits + row] = frs[i];
    }
  }
#endif
}

#if !(AE_MERGE_IN_WG || AE_MERGE_LAST)
#include "ae_combine.h"      // the merge kernel of the two-launch form
#endif
