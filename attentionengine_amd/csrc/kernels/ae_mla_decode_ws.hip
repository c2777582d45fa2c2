// MLA (shared latent KV) split-KV decode for gfx950 / CDNA4, wave-specialised: online softmax only.
//
// Same role as ae_mla_decode.hip (the reference's TileLang MLA decode template,
// attention_engine/core/template/tl_template/attn/mla_decode_tl.py: flash_attn_split 104-179, and the
// CuTe/FlashMLA split kernel, core/template/cute_template_kvshared/kernels/splitkv_mla.cu:1061-1393),
// for the case the lowering has proven to be the online softmax of `score * constant`
// (attn_script/mha.py:47-72); anything else uses ae_mla_decode.hip, which runs the generated functors.
//
// Why a second kernel: in ae_mla_decode.hip every one of 8 waves reads the whole KV tile from LDS for
// both products (416 KiB of LDS reads per 32-token tile and workgroup) and the two value halves of a
// head block compute the same scores; LDS bandwidth bounds it at ~0.21 ms for B128 H128 S4096.  Here
// the waves of a workgroup (64 query heads of one (batch, kv head, split)) have different jobs:
//   * 2 "score waves" (32 heads each): S^T[kv,head] = K Q^T with v_mfma_f32_32x32x16 (Q^T in registers for
//     the whole kernel, K fragments from LDS, each feeding a 32x32 block: with 16 heads per wave the four
//     waves' fragment reads, 144 KiB per tile, took 2.6x the time of their MFMAs), lazy online softmax,
//     P^T written to LDS as the B operand of the second product, per-head rescale factors next to it;
//   * 4 "value waves" (a quarter of the value columns each, all 64 heads): O^T[dv,head] += V^T P^T with
//     v_mfma_f32_32x32x16, V^T fragments read from the SAME LDS rows through ds_read_b64_tr_b16, every
//     fragment feeding both 32-head blocks.
// Wave i runs on SIMD i % 4.  The workgroup is launched with 8 waves: waves 0, 1 are the score waves
// (SIMD 0, 1: 1152 matrix-pipe cycles per tile each), waves 2, 3, 6, 7 the value waves (two each on SIMD
// 2, 3: 2 x 512 cycles), waves 4, 5 leave at once - so the four SIMDs carry about the same MFMA work.
// The score waves run one tile ahead of the value waves: one workgroup barrier per tile hands P over.
// Scores are computed once: 124 KiB of LDS reads per tile instead of 416.  KV tiles go HBM -> LDS
// directly (16 B per lane, chunk-swizzled as in ae_mla_decode.hip), AE_NSTAGE tiles deep; a trip ends by
// waiting until only the newest tile request is outstanding.
//
// Configuration ("ae_config.h"): AE_D1 AE_D2 AE_DV AE_DTYPE_BF16 AE_N_ROWSCALES AE_NSPLIT
// AE_COMBINE_THREADS AE_PAGED (1: the cache is paged, rows are found through ae_attn_params.block_table and
// every batch entry has its own length seqlens_k[b], as in the reference's
// cute_template_kvshared/kernels/params.h:33-36; a kv tile never straddles two pages), plus AE_SM_SCALE (the constant c > 0) and AE_SM_M / AE_SM_R (names of the
// running-max and running-sum fields of ae_rowstate).  Functors used ("ae_functors.h"): ae_rowstate,
// ae_rowstate_init, ae_epilogue, ae_load_custom, ae_combine.

#define AE_LAYOUT 1
#include "ae_hip.h"
#include "ae_config.h"
#include "ae_device.h"
#include "ae_functors.h"

#define AE_D (AE_D1 + AE_D2)
#define AE_NWAVES 8
#define AE_NT (AE_NWAVES * 64)
#define AE_HEADS_PER_WG 64
#define AE_BN 32                          // kv rows per tile
#define AE_NKS (AE_D / 16)                // 16-deep k-steps of S^T = K Q^T
#define AE_NLOADERS 4                     // the value waves also request the KV tiles
#define AE_DVW (AE_DV / 4)                // value columns of one value wave
#define AE_NDB (AE_DVW / 32)              // 32-wide dv blocks of a value wave
#define AE_NO (AE_NDB * 16)               // output elements per lane and head block
#define AE_KSTR (AE_D * 2)                // LDS row pitch, bytes (unpadded: swizzled)
#define AE_STAGE_BYTES (AE_BN * AE_KSTR)
#define AE_CPR (AE_D / 8)                 // 16-byte chunks per K row
#define AE_CPR1 (AE_D1 / 8)
#define AE_BLOCKS ((AE_BN * AE_CPR) / 64) // 1 KiB blocks per tile
#define AE_LOADS ((AE_BLOCKS + AE_NLOADERS - 1) / AE_NLOADERS)
#define AE_L1 ((AE_LOADS + 1) / 2)        // a wave's loads of one tile go out as two bursts
#define AE_L2 (AE_LOADS - AE_L1)
#ifndef AE_NSTAGE
#define AE_NSTAGE 4
#define AE_PTAB 1024      // paged cache: block-table entries of one split kept in LDS
#endif
#define AE_PSTR 80                        // LDS pitch of one head's P row (32 kv * 2 B, padded against bank conflicts)
#define AE_P_BYTES (AE_HEADS_PER_WG * AE_PSTR)
#define AE_X_BYTES (AE_HEADS_PER_WG * 4 + 16)   // per-head rescale factors + one flag word per score wave (2 used)
#define AE_TAU2 8.0f                      // the running maximum (log2 units) is refreshed only when it moved by more
#define AE_SWZ(r) ((((r) >> 1) & 3) * 2 + (((r) >> 3) & 1))
#define AE_VMCNT(n) (0x0F70 | ((n) & 15) | (((n) >> 4) << 14))
#define AE_VMCNT_LGKM0(n) (0x0070 | ((n) & 15) | (((n) >> 4) << 14))
#ifndef AE_AHEAD
#define AE_AHEAD 4
#endif
#define AE_RING (AE_AHEAD + 1)

static_assert(AE_D1 % 32 == 0 && AE_D2 % 32 == 0, "latent / rope dims must be multiples of 32");
static_assert(AE_NKS % 2 == 0, "two accumulation chains over the k-steps");
static_assert(AE_DV % 128 == 0 && AE_DV <= AE_D1, "V must be a prefix of the latent part, four 32-column blocks wide");
static_assert(AE_CPR % 8 == 0 && AE_CPR1 % 8 == 0, "chunk groups of eight must not straddle the two K tensors");
static_assert((AE_BN * AE_CPR) % 64 == 0, "tile must be a whole number of 1 KiB blocks");
static_assert(AE_L1 <= 8 && AE_L2 >= 1 && AE_BLOCKS >= AE_LOADS, "two bursts of at most eight loads per wave and tile");
static_assert(AE_NSTAGE >= 3, "a tile is multiplied by K one trip before it is multiplied as V");

#ifndef AE_PAGED
#define AE_PAGED 0
#endif
// 1 (single-split builds only, a measurement switch): every workgroup reports the shader-clock cycles (s_memtime)
// and the constant-rate 100 MHz ticks (s_memrealtime) between its entry and its last store, as two 64-bit values
// at ((unsigned long long*)p.partial_o)[2 * blockIdx.x] - a buffer a single-split launch does not otherwise use -
// and, behind the pairs of all workgroups (at index 2 * gridDim.x + 4 * blockIdx.x), four more tick values of one
// value wave: entry, first tile landed, last trip done, last store acknowledged (absolute 100 MHz ticks).
#ifndef AE_CLOCK_STAMPS
#define AE_CLOCK_STAMPS 0
#endif
static_assert(!AE_CLOCK_STAMPS || AE_NSPLIT == 1, "the clock stamps go where a split launch keeps its partial results");
#if AE_PAGED
#include "ae_mla_paged.h"
#endif

typedef __attribute__((address_space(3))) unsigned char ae_lds_byte;
typedef __attribute__((address_space(3))) float ae_lds_f32;
typedef __attribute__((address_space(3))) int ae_lds_i32;
template <bool B> struct ae_const_bool { static constexpr bool value = B; };

extern "C" __global__ __launch_bounds__(AE_NT) __attribute__((amdgpu_waves_per_eu(2, 2)))
void ae_mla_decode_split_kernel(const ae_attn_params p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ae_smem[];
  ae_lds_byte* lds = (ae_lds_byte*)ae_smem;                     // AE_NSTAGE kv tiles
  ae_lds_byte* pbuf = lds + AE_NSTAGE * AE_STAGE_BYTES;         // 2 x P^T [head][kv]
  ae_lds_byte* xbuf = pbuf + 2 * AE_P_BYTES;                    // 2 x (rescale factors, flags)
  ae_lds_f32* fin = (ae_lds_f32*)(xbuf + 2 * AE_X_BYTES);       // final (m, r) per head
#if AE_PAGED
  ae_lds_i32* ptab = (ae_lds_i32*)(fin + 2 * AE_HEADS_PER_WG);  // AE_PTAB page numbers: this split's part of the block table
#endif

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool score_wave = wave < 2;
#if AE_CLOCK_STAMPS
  const unsigned long long ae_t0 = __builtin_amdgcn_s_memtime();
  const unsigned long long ae_w0 = __builtin_amdgcn_s_memrealtime();
#endif

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

#if AE_PAGED
  const ae_elem* k1 = (const ae_elem*)p.k + (int64_t)hk * p.k_stride_h;
  const ae_elem* k2 = (const ae_elem*)p.k2 + (int64_t)hk * p.k2_stride_h;
  const int32_t* pages = p.block_table + (int64_t)b * p.block_table_stride;
  int seqlen_b = p.seqlens_k[b];
  seqlen_b = seqlen_b < p.seqlen_kv ? seqlen_b : p.seqlen_kv;
  seqlen_b = __builtin_amdgcn_readfirstlane(seqlen_b > 0 ? seqlen_b : 0);
#else
  const ae_elem* k1 = (const ae_elem*)p.k + (int64_t)b * p.k_stride_b + (int64_t)hk * p.k_stride_h;
  const ae_elem* k2 = (const ae_elem*)p.k2 + (int64_t)b * p.k2_stride_b + (int64_t)hk * p.k2_stride_h;
  const int seqlen_b = p.seqlen_kv;
#endif

  // (wave-uniform values are pinned to scalar registers: a copy in a vector register that gets spilled is
  // reloaded with a scratch load, which the tile loads' vmcnt bookkeeping would have to wait for)
  const int kv_begin = __builtin_amdgcn_readfirstlane(split * p.kv_per_split);
  int kv_end_ = kv_begin + p.kv_per_split;
  kv_end_ = kv_end_ < seqlen_b ? kv_end_ : seqlen_b;
  const int kv_end = __builtin_amdgcn_readfirstlane(kv_end_);
  const int n_tiles = __builtin_amdgcn_readfirstlane(kv_end > kv_begin ? (kv_end - kv_begin + AE_BN - 1) / AE_BN : 0);
#if AE_PAGED
  // a split beyond this entry's length: nothing to read (its table entries may be unset) and nothing to write,
  // the merge passes it over; split 0 of an entry of length 0 writes that entry's "no keys" result
  if (n_tiles == 0) {
    if (split == 0) ae_mla_write_no_keys(p, b, hk, ht, group, tid);
    return;
  }
#endif
  // who writes `out`: this workgroup (a launch without splits; a paged entry whose keys all lie in split 0), or the
  // merge kernel from the splits' partial results
#if AE_NSPLIT == 1
  constexpr bool direct = true;
#elif AE_PAGED
  const bool direct = ae_mla_splits_used(p, seqlen_b) <= 1;
#else
  constexpr bool direct = false;
#endif
  if (wave == 4 || wave == 5) return;      // placeholders: they only steer the value waves onto SIMD 2, 3

  if (score_wave) {
    // =============================== score wave: 32 heads ==============================================
    const int l32s = lane & 31;
    const int hfs = lane >> 5;
    const int head_in_group = ht * AE_HEADS_PER_WG + wave * 32 + l32s;
    const bool head_ok = head_in_group < group;
    const int hq = hk * group + (head_ok ? head_in_group : 0);
    // Q^T fragments: B operand (n = head = lane%32, k = d = 16*ks + 8*(lane/32) + j)
    const ae_elem* q1 = (const ae_elem*)p.q + (int64_t)b * p.q_stride_b + (int64_t)hq * p.q_stride_h;
    const ae_elem* q2 = (const ae_elem*)p.q2 + (int64_t)b * p.q2_stride_b + (int64_t)hq * p.q2_stride_h;
    ae_elem8 qf[AE_NKS];
#pragma unroll
    for (int ks = 0; ks < AE_D1 / 16; ks++) qf[ks] = *(const ae_elem8*)(q1 + ks * 16 + hfs * 8);
#pragma unroll
    for (int ks = 0; ks < AE_D2 / 16; ks++) qf[AE_D1 / 16 + ks] = *(const ae_elem8*)(q2 + ks * 16 + hfs * 8);

    ae_rowstate st;
    ae_rowstate_init(st);
    float m2 = st.AE_SM_M * AE_LOG2E;   // running reference, log2 units
    float r_run = st.AE_SM_R;           // this lane's part of the row sum (a row lives in lanes l, l^32)

    // (the value waves request the tiles: this wave's registers are taken by Q^T)
    __builtin_amdgcn_s_waitcnt(AE_VMCNT(0));   // Q has landed
    __syncthreads();                           // tile 0 has landed

    // K fragment of k-step ks: row lane%32, global chunk 2*ks + lane/32.  The swizzle touches the three low
    // bits of the chunk number only, so a lane has four distinct offsets (ks % 4) and the rest is an immediate.
    int k_base[4];
#pragma unroll
    for (int i = 0; i < 4; i++) k_base[i] = l32s * AE_KSTR + (((2 * i + hfs) ^ AE_SWZ(l32s)) << 4);
    // A trip multiplies tile n by Q^T and, in the issue slots between those MFMAs, runs the softmax of tile
    // n - 1 (its raw scores wait in `xs`): the wave's matrix work and its softmax overlap instead of
    // following each other.  P of tile n - 1 is handed over by the barrier that ends trip n.
    ae_f32x16 xs;        // raw scores of the tile before the one being multiplied
#pragma unroll
    for (int r = 0; r < 16; r++) xs[r] = 0.f;
    // lane owns head lane%32 and kv rows 8*(e/4) + 4*(lane/32) + e%4 of a tile
    float mx, mn, osc, rs;
    bool need;
    ae_lds_byte* prow;
    ae_lds_byte* xb;
    // start of the softmax of tile tp: scores beyond the end of the range are taken out (ragged tail only)
    auto soft_begin = [&](int tp) AE_LAMBDA {
      // (xs holds raw scores: the scale is folded into the exponent; the softmax works on it in place)
      const bool tail = kv_begin + tp * AE_BN + AE_BN > kv_end;
      if (__builtin_expect(tail, 0)) {
        // the empty asm keeps this a branch: flattened into selects it costs 5 instructions per score
        // on every tile
        asm volatile("" ::: "memory");
        const int kvb = kv_begin + tp * AE_BN + 4 * hfs;
#pragma unroll
        for (int e = 0; e < 16; e++) xs[e] = (kvb + 8 * (e >> 2) + (e & 3) < kv_end) ? xs[e] : AE_NEG_INF;
      }
      mx = AE_NEG_INF;
      rs = 0.f;
      prow = pbuf + (tp & 1) * AE_P_BYTES + (wave * 32 + l32s) * AE_PSTR + 8 * hfs;
      xb = xbuf + (tp & 1) * AE_X_BYTES;
    };
    // the softmax of one tile in AE_NKS pieces, piece f issued behind the MFMA of k-step f
    auto soft_slot = [&](int f) AE_LAMBDA {
      if (f < 4) {
        mx = __builtin_fmaxf(__builtin_fmaxf(mx, xs[4 * f]), xs[4 * f + 1]);
        mx = __builtin_fmaxf(__builtin_fmaxf(mx, xs[4 * f + 2]), xs[4 * f + 3]);
      } else if (f == 4) {
        float hi;
        const float lo = ae_swap32_lo_hi(mx, hi);
        mx = __builtin_fmaxf(lo, hi) * (AE_SM_SCALE * AE_LOG2E);   // the scale is positive
      } else if (f == 5) {
        need = (mx - m2) > AE_TAU2;
        mn = need ? mx : m2;
        osc = need ? ae_exp2(m2 - mn) : 1.0f;
        m2 = mn;
      } else if (f < 22) {
        const int e = f - 6;
        xs[e] = ae_exp2(__builtin_fmaf(xs[e], AE_SM_SCALE * AE_LOG2E, -mn));
        rs += xs[e];
      } else if (f < 26) {
        const int rb = f - 22;
        ae_elem4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (ae_elem)xs[4 * rb + i];
        *(__attribute__((address_space(3))) ae_elem4*)(prow + 16 * rb) = w;
      } else if (f == 26) {
        r_run = r_run * osc + rs;
        if (hfs == 0) ((ae_lds_f32*)xb)[wave * 32 + l32s] = osc;
        const bool any = __builtin_amdgcn_ballot_w64(need) != 0;
        if (lane == 0) ((ae_lds_i32*)(xb + AE_HEADS_PER_WG * 4))[wave] = any ? 1 : 0;
      }
    };
    static_assert(AE_NKS >= 27, "the softmax of a tile is spread over 27 k-steps");
    // S^T of tile tn into xs; with SOFT the softmax of tile tn - 1 rides along
    auto score_trip = [&](int tn, auto with_soft) AE_LAMBDA {
      constexpr bool SOFT = decltype(with_soft)::value;
      int ka[4];
#pragma unroll
      for (int i = 0; i < 4; i++) ka[i] = k_base[i] + (tn % AE_NSTAGE) * AE_STAGE_BYTES;
      // read AE_AHEAD fragments before the MFMA that uses them (the compiler on its own keeps one read
      // in flight, which leaves the LDS latency exposed)
      auto read_kfrag = [&](int ks) AE_LAMBDA -> ae_elem8 {
        return *(const __attribute__((address_space(3))) ae_elem8*)(lds + ka[ks & 3] + (ks >> 2) * 128);
      };
      ae_elem8 ring[AE_RING];
#pragma unroll
      for (int f = 0; f < AE_AHEAD; f++) ring[f] = read_kfrag(f);
      if (SOFT) soft_begin(tn - 1);
      // even / odd k-steps accumulate separately (two independent MFMA chains)
      ae_f32x16 sacc[2];
#pragma unroll
      for (int c = 0; c < 2; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[c][r] = 0.f;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int f = 0; f < AE_NKS; f++) {
        if (f + AE_AHEAD < AE_NKS) ring[(f + AE_AHEAD) % AE_RING] = read_kfrag(f + AE_AHEAD);
        sacc[f & 1] = ae_mfma32(ring[f % AE_RING], qf[f], sacc[f & 1]);
        if (SOFT) soft_slot(f);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int r = 0; r < 16; r++) xs[r] = sacc[0][r] + sacc[1][r];
    };
    if (n_tiles > 0) score_trip(0, ae_const_bool<false>());
    __syncthreads();                             // end of trip 0: tile 1 has landed
    for (int tn = 1; tn < n_tiles; tn++) {
      score_trip(tn, ae_const_bool<true>());
      __syncthreads();                           // end of the trip: P of tile tn - 1 is handed over, tile tn + 1 has landed
    }
    if (n_tiles > 0) {                           // the last tile's softmax has no MFMAs to hide behind
      soft_begin(n_tiles - 1);
#pragma unroll
      for (int f = 0; f < 27; f++) soft_slot(f);
      __syncthreads();
    }
    // final row state for the value waves
    {
      float hi;
      const float lo = ae_swap32_lo_hi(r_run, hi);
      if (hfs == 0) {
        fin[(wave * 32 + l32s) * 2] = m2 * AE_LN2;
        fin[(wave * 32 + l32s) * 2 + 1] = lo + hi;
      }
    }
    __syncthreads();
    return;
  }

  // ================================= value wave: AE_DVW value columns, 64 heads ========================
  const int l32 = lane & 31;
  const int hf = lane >> 5;
  const int dvw = wave < 4 ? wave - 2 : wave - 4;   // waves 2, 3, 6, 7
  // Direct HBM -> LDS tile load, by the four value waves: wave w fills AE_LOADS consecutive 1 KiB blocks of
  // the tile, starting at block min(w*AE_LOADS, AE_BLOCKS-AE_LOADS) (the last wave overlaps its neighbour, so
  // every wave issues the same number of loads); LDS chunk c' of row r receives global chunk c' ^ f(r).
  // Which row and chunk a lane fetches never changes: its byte offset inside a tile is computed once (one
  // register per load) and added per tile to the tile's wave-uniform address in the latent or in the rope
  // tensor.  The loads of a wave go out as two bursts, each behind a single write of M0 (see
  // ae_load_lds16_burst; the offsets carry the compensation for its immediate offsets).  Tiles past the
  // end re-read the last tile, so every trip issues the same number of loads; rows past the end re-read
  // the last row.
  const int blk0 = dvw * AE_LOADS < AE_BLOCKS - AE_LOADS ? dvw * AE_LOADS : AE_BLOCKS - AE_LOADS;
  int ld_off[AE_LOADS];           // this lane's byte offset of load i inside a tile (may be negative)
  unsigned ld_rope = 0;           // bit i: load i reads from the rope tensor (k2), else from the latent (k1)
  const unsigned stride1 = (unsigned)p.k_stride_s * 2, stride2 = (unsigned)p.k2_stride_s * 2;   // bytes per kv row
#pragma unroll
  for (int i = 0; i < AE_LOADS; i++) {
    const int sidx = (blk0 + i) * 64 + lane;
    const int row = sidx / AE_CPR, cp = sidx % AE_CPR;
    const int c = cp ^ AE_SWZ(row);
    if (c < AE_CPR1) {
      ld_off[i] = c * 16 + row * (int)stride1;
    } else {
      ld_off[i] = (c - AE_CPR1) * 16 + row * (int)stride2;
      ld_rope |= 1u << i;
    }
    // immediate offset of load i inside its burst
    ld_off[i] -= i < AE_L1 ? (i - AE_L1 / 2) * 1024 : (i - AE_L1 - AE_L2 / 2) * 1024;
  }
#if AE_PAGED
  // Paged cache: the latent and the rope part are column ranges of ONE cache tensor (equal strides, the rope
  // columns rope_delta bytes behind the latent ones: checked by ae_mla_decode_fwd), so every load of a tile is
  // (the tile's wave-uniform address) + (an offset of the lane that never changes): scalar base + 32-bit offset
  // loads, no address arithmetic per tile at all.  Bases are passed 4 KiB low and the offsets 4 KiB high, so
  // that the offsets, which carry the compensation for the immediate offsets, stay >= 0.
  const unsigned rope_delta = (unsigned)((const char*)k2 - (const char*)k1);
  unsigned ld_uoff[AE_LOADS];
#pragma unroll
  for (int i = 0; i < AE_LOADS; i++)
    ld_uoff[i] = (unsigned)(ld_off[i] + 4096) + (((ld_rope >> i) & 1u) ? rope_delta : 0u);
#else
  // Dense cache: the requests go tile by tile, so a lane keeps the source address of each of its loads for the
  // NEXT tile to request and adds the tile pitch after every request - two instructions per load and tile.
  // (Two waves share a SIMD here: address arithmetic of ~140 instructions per tile and wave, as a base + offset
  // form needs, made these waves, not the matrix pipe, set the pace of the whole workgroup.)
  const char* ld_ptr[AE_LOADS];
  unsigned ld_adv[AE_LOADS];
#pragma unroll
  for (int i = 0; i < AE_LOADS; i++) {
    const bool rope = (ld_rope >> i) & 1u;
    const unsigned stride = rope ? stride2 : stride1;
    ld_ptr[i] = (const char*)(rope ? (const void*)k2 : (const void*)k1) + (uint64_t)((unsigned)kv_begin * (uint64_t)stride) +
                (int64_t)ld_off[i];
    ld_adv[i] = AE_BN * stride;
  }
#endif
#if AE_PAGED
  // Paged cache: page, and row inside it, of the tile the NEXT request reads (wave-uniform; requests go tile by
  // tile, so no division per tile).  The split's part of the block table is copied into LDS first and looked up
  // there: once the tile loads are in flight, a table entry read from memory comes back through the same counter
  // as they do (the compiler cannot use a scalar load behind the loads' asm statements), and waiting for it means
  // waiting for every tile requested so far - 0.190 against 0.170 ms for the dense cache at B128 H128 S4096,
  // 0.166 ms with the table in LDS.  Every value wave writes the same entries and reads them back itself (a wave's
  // LDS operations complete in order), so no barrier is needed.
  const int rq_slot0 = kv_begin / p.page_block_size;
  {
    const int n_ent = (kv_end - 1) / p.page_block_size - rq_slot0 + 1;     // <= AE_PTAB: checked by ae_mla_decode_fwd
    for (int i = lane; i < n_ent && i < AE_PTAB; i += 64) ptab[i] = pages[rq_slot0 + i];
  }
  int rq_idx = 0;
  int rq_in_page = kv_begin - rq_slot0 * p.page_block_size;
  int rq_page = pages[rq_slot0];
#endif
  // requests are made for t = 0, 1, 2, ... in this order
  auto load_tile = [&](int t_) AE_LAMBDA {
    const int t = __builtin_amdgcn_readfirstlane(t_);
    int tt = t < n_tiles ? t : n_tiles - 1;
    tt = tt < 0 ? 0 : tt;
    const int kv0 = kv_begin + tt * AE_BN;
    ae_lds_byte* dst = lds + (t % AE_NSTAGE) * AE_STAGE_BYTES;
    const bool ragged = kv0 + AE_BN > seqlen_b;     // wave-uniform
#if AE_PAGED
    // the tile's page was looked up when the previous request went out (rq_*, below); kv0 < seqlen_b, so its
    // table entry is set, and an entry outside the cache is clamped
    int page = rq_page < 0 ? 0 : (rq_page < p.num_pages ? rq_page : p.num_pages - 1);
    page = __builtin_amdgcn_readfirstlane(page);
    const char* tile = (const char*)k1 + ((int64_t)page * p.k_stride_b + (int64_t)rq_in_page * p.k_stride_s) * 2 - 4096;
    unsigned o1[8], o2[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      o1[i] = ld_uoff[i < AE_L1 ? i : 0];
      o2[i] = ld_uoff[i < AE_L2 ? AE_L1 + i : AE_L1];
    }
    if (__builtin_expect(ragged, 0)) {                        // rows past the end re-read the last row
      asm volatile("" ::: "memory");                          // (keeps this ONE branch, out of the common path)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int j = i < 8 ? (i < AE_L1 ? i : 0) : (i - 8 < AE_L2 ? AE_L1 + i - 8 : AE_L1);
        const int row = ((blk0 + j) * 64 + lane) / AE_CPR;
        int over = kv0 + row - (seqlen_b - 1);
        over = over > 0 ? over : 0;                           // <= row: the offset stays >= 0
        const unsigned back = (unsigned)over * stride1;
        if (i < 8) o1[i] -= back;
        else o2[i - 8] -= back;
      }
    }
    ae_load_lds16_burst_base<AE_L1>(tile, o1, dst + (blk0 + AE_L1 / 2) * 1024);
    ae_load_lds16_burst_base<AE_L2>(tile, o2, dst + (blk0 + AE_L1 + AE_L2 / 2) * 1024);
#else
    const char* g1[8];
    const char* g2[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      g1[i] = ld_ptr[i < AE_L1 ? i : 0];
      g2[i] = ld_ptr[i < AE_L2 ? AE_L1 + i : AE_L1];
    }
    if (__builtin_expect(ragged, 0)) {                        // rows past the end re-read the last row
      asm volatile("" ::: "memory");                          // (keeps this ONE branch, out of the common path)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int j = i < 8 ? (i < AE_L1 ? i : 0) : (i - 8 < AE_L2 ? AE_L1 + i - 8 : AE_L1);
        const int row = ((blk0 + j) * 64 + lane) / AE_CPR;
        int over = kv0 + row - (seqlen_b - 1);
        over = over > 0 ? over : 0;
        const int back = over * (int)(((ld_rope >> j) & 1u) ? stride2 : stride1);
        if (i < 8) g1[i] -= back;
        else g2[i - 8] -= back;
      }
    }
    ae_load_lds16_burst<AE_L1>((const void* const*)g1, dst + (blk0 + AE_L1 / 2) * 1024);
    ae_load_lds16_burst<AE_L2>((const void* const*)g2, dst + (blk0 + AE_L1 + AE_L2 / 2) * 1024);
#endif
#if !AE_PAGED
    if (t + 1 < n_tiles) {                                    // (requests past the end repeat the last tile)
#pragma unroll
      for (int i = 0; i < AE_LOADS; i++) ld_ptr[i] += ld_adv[i];
    }
#else
    if (t + 1 < n_tiles) {                                    // where the next request reads: an LDS lookup per new
      rq_in_page += AE_BN;                                    // page, a whole trip before its result is used
      if (rq_in_page >= p.page_block_size) {
        rq_in_page = 0;
        rq_idx++;
        rq_page = ptab[rq_idx];
      }
    }
#endif
  };
  // end of a trip: tile t+2 has landed when only the newest request is outstanding; after the barrier
  // everyone is done with tile t, whose stage takes the next request
  auto end_trip = [&](int t) AE_LAMBDA {
    __builtin_amdgcn_s_waitcnt(AE_VMCNT_LGKM0(AE_LOADS));   // ... and this trip's LDS reads have returned
    __syncthreads();
    load_tile(t + AE_NSTAGE);
  };

  ae_f32x16 oacc[2][AE_NDB];     // [head block][dv block]: O^T
#pragma unroll
  for (int hb = 0; hb < 2; hb++)
#pragma unroll
    for (int db = 0; db < AE_NDB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[hb][db][r] = 0.f;

  __builtin_amdgcn_s_waitcnt(AE_VMCNT(0));
#pragma unroll
  for (int t = 0; t < AE_NSTAGE - 1; t++) load_tile(t);
  __builtin_amdgcn_s_waitcnt(AE_VMCNT((AE_NSTAGE - 2) * AE_LOADS));
  __syncthreads();
#if AE_CLOCK_STAMPS
  const unsigned long long ae_w1 = __builtin_amdgcn_s_memrealtime();     // tile 0 (and Q) have landed
#endif

  // V^T fragment (k-step kk, dv block db): A[m = dv][k = kv]: lane i of a 16-lane group supplies the
  // address of row 16*kk + 8*hf + i/4 (+4 for slots 4..7), 8 bytes at value column
  // 32*db + 16*((lane%32)/16) + 4*(i%4), and receives column i of those four rows.  The swizzle of a
  // row's chunks touches the three low bits of the chunk number only, so a lane has four distinct
  // offsets (parity of db, first / second group of four rows) and everything else is an immediate.
  const int v_row = 8 * hf + ((lane & 15) >> 2);
  const int v_c0 = 2 * (l32 >> 4) + ((lane & 3) >> 1);
  const int v_half = (lane & 1) * 8;
  int v_base[2][2];     // [db & 1][row group]
#pragma unroll
  for (int par = 0; par < 2; par++)
#pragma unroll
    for (int rg = 0; rg < 2; rg++) {
      const int r = v_row + 4 * rg;
      v_base[par][rg] = r * AE_KSTR + ((((4 * par + v_c0) ^ AE_SWZ(r)) + 4 * AE_NDB * dvw) << 4) + v_half;
    }
  static_assert(AE_NDB % 2 == 0, "a value wave's first chunk must be a multiple of eight");
  auto read_vfrag = [&](const int (&va)[2][2], int kk, int db) AE_LAMBDA -> ae_elem8 {
    const int imm = 16 * kk * AE_KSTR + (db >> 1) * 128;
    ae_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) ae_s16x4*)(
        lds + va[db & 1][0] + imm));
    ae_s16x4 hi2 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) ae_s16x4*)(
        lds + va[db & 1][1] + imm));
    return __builtin_bit_cast(ae_elem8, __builtin_shufflevector(lo, hi2, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  // A trip of a value wave: O^T += V^T P^T for tile n - 2 with the V^T fragments it holds in registers (PV),
  // and the fragments of tile n - 1 read from LDS into those registers as they fall free (RD) - the read
  // has a whole trip to complete, and tile n - 1's stage can take the next request when the trip ends.
  ae_elem8 vreg[2 * AE_NDB];     // fragment f = (k-step f / AE_NDB, dv block f % AE_NDB)
#pragma unroll
  for (int f = 0; f < 2 * AE_NDB; f++) vreg[f] = (ae_elem8){};
  auto value_trip = [&](int n, auto with_pv, auto with_rd) AE_LAMBDA {
    constexpr bool PV = decltype(with_pv)::value;
    constexpr bool RD = decltype(with_rd)::value;
    int va[2][2];          // the lane's four fragment offsets inside tile n - 1's stage
#pragma unroll
    for (int i = 0; i < 4; i++) va[i >> 1][i & 1] = v_base[i >> 1][i & 1] + ((n - 1) % AE_NSTAGE) * AE_STAGE_BYTES;
    ae_elem8 pf[2][2];
    if (PV) {
      const int t = n - 2;
      const ae_lds_byte* pb = pbuf + (t & 1) * AE_P_BYTES;
      const ae_lds_byte* xb = xbuf + (t & 1) * AE_X_BYTES;
      // rescale O for the heads whose reference moved (rare once the maxima have settled)
      const ae_lds_i32* flags = (const ae_lds_i32*)(xb + AE_HEADS_PER_WG * 4);
      if (__builtin_amdgcn_readfirstlane(flags[0] | flags[1]) != 0) {
#pragma unroll
        for (int hb = 0; hb < 2; hb++) {
          const float osc = ((const ae_lds_f32*)xb)[hb * 32 + l32];
#pragma unroll
          for (int db = 0; db < AE_NDB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[hb][db][r] *= osc;
        }
      }
      // P^T fragments: B[k = kv = 16*kk + 8*hf + j][n = head = 32*hb + l32]
#pragma unroll
      for (int hb = 0; hb < 2; hb++)
#pragma unroll
        for (int kk = 0; kk < 2; kk++)
          pf[hb][kk] = *(const __attribute__((address_space(3))) ae_elem8*)(
              pb + (hb * 32 + l32) * AE_PSTR + 32 * kk + 16 * hf);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int f = 0; f < 2 * AE_NDB; f++) {
      if (PV) {
#pragma unroll
        for (int hb = 0; hb < 2; hb++)
          oacc[hb][f % AE_NDB] = ae_mfma32(vreg[f], pf[hb][f / AE_NDB], oacc[hb][f % AE_NDB]);
      }
      if (RD) vreg[f] = read_vfrag(va, f / AE_NDB, f % AE_NDB);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  end_trip(-1);                                                    // trip 0: the score waves multiply tile 0
  value_trip(1, ae_const_bool<false>(), ae_const_bool<true>());    // trip 1: fragments of tile 0
  end_trip(0);
  for (int n = 2; n <= n_tiles; n++) {
    value_trip(n, ae_const_bool<true>(), ae_const_bool<true>());
    end_trip(n - 1);
  }
  if (n_tiles > 0) {                                               // trip n_tiles + 1: the last tile's product
    value_trip(n_tiles + 1, ae_const_bool<true>(), ae_const_bool<false>());
    end_trip(n_tiles);
  }
  __builtin_amdgcn_s_waitcnt(AE_VMCNT(0));   // (the last barrier also made the final (m, r) of every head visible)
#if AE_CLOCK_STAMPS
  const unsigned long long ae_w2 = __builtin_amdgcn_s_memrealtime();     // the last trip is done
#endif

  // ---- per-split epilogue: lane owns head 32*hb + l32, value columns AE_DVW*dvw + 32*db + 8*(r/4) + 4*hf + r%4
#pragma unroll
  for (int hb = 0; hb < 2; hb++) {
    const int head_in_group = ht * AE_HEADS_PER_WG + hb * 32 + l32;
    const bool head_ok = head_in_group < group;
    const int hq = hk * group + (head_ok ? head_in_group : 0);
    ae_ctx ctx;
    ctx.b = b;
    ctx.h = hq;
    ctx.q_idx = 0;
    ctx.kv_base = 0;
    ae_custom cust;
    ae_load_custom(cust, p, ctx);
    ae_rowstate st;
    ae_rowstate_init(st);
    float o[AE_NO];
#pragma unroll
    for (int db = 0; db < AE_NDB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[db * 16 + r] = oacc[hb][db][r];
    float frs[AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1];
    frs[0] = 0.f;
    if (n_tiles > 0) {
      st.AE_SM_M = fin[(hb * 32 + l32) * 2];
      st.AE_SM_R = fin[(hb * 32 + l32) * 2 + 1];
      ae_epilogue<AE_NO>(o, st, frs, ctx, cust);
    } else {
#pragma unroll
      for (int e = 0; e < AE_NO; e++) o[e] = 0.f;
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++) frs[i] = AE_NEG_INF;
    }
    if (!head_ok) continue;
    if (direct) {
    ae_elem* optr = (ae_elem*)p.out + (int64_t)b * p.o_stride_b + (int64_t)hq * p.o_stride_h + dvw * AE_DVW;
#pragma unroll
    for (int db = 0; db < AE_NDB; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        ae_elem4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (ae_elem)o[db * 16 + rg * 4 + i];
        *(ae_elem4*)(optr + db * 32 + rg * 8 + hf * 4) = w;
      }
    if (hf == 0 && dvw == 0) {
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++)
        if (p.rowscale_out[i]) p.rowscale_out[i][(int64_t)b * p.heads_q + hq] = frs[i];
    }
    continue;
    }
    const int64_t row = ((int64_t)b * p.heads_q + hq) * p.num_splits + split;
    float* po = p.partial_o + row * AE_DV + dvw * AE_DVW;
#pragma unroll
    for (int db = 0; db < AE_NDB; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        ae_f32x4 w = {o[db * 16 + rg * 4 + 0], o[db * 16 + rg * 4 + 1], o[db * 16 + rg * 4 + 2], o[db * 16 + rg * 4 + 3]};
        *(ae_f32x4*)(po + db * 32 + rg * 8 + hf * 4) = w;
      }
    if (hf == 0 && dvw == 0) {
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++)
        p.partial_rs[(int64_t)i * p.batch * p.heads_q * p.num_splits + row] = frs[i];
    }
  }
#if AE_CLOCK_STAMPS
  __builtin_amdgcn_s_waitcnt(0);          // the stores have been acknowledged
  if (wave == 2) {
    const unsigned long long t1 = __builtin_amdgcn_s_memtime();
    const unsigned long long w1 = __builtin_amdgcn_s_memrealtime();
    if (lane == 0) {
      unsigned long long* st = (unsigned long long*)p.partial_o + 2 * (unsigned long long)blockIdx.x;
      st[0] = t1 - ae_t0;
      st[1] = w1 - ae_w0;
      unsigned long long* ph = (unsigned long long*)p.partial_o + 2 * (unsigned long long)gridDim.x +
                               4 * (unsigned long long)blockIdx.x;
      ph[0] = ae_w0;
      ph[1] = ae_w1;
      ph[2] = ae_w2;
      ph[3] = w1;
    }
  }
#endif
}

#include "ae_combine.h"
