// Flash-style attention forward (prefill) for gfx950 / CDNA4.
//
// Takes the place of the reference's TileLang prefill template
// (attention_engine/core/template/tl_template/attn/attn_tl.py:76-174) and its block-sparse
// sibling (blockattn_tl.py:49-160). Per KV tile it keeps the reference's order of operations
// (attn_tl.py:124-164): mask -> +QK^T -> score_mod -> online_func -> cast P -> rescale O ->
// O += P V, then the epilogue and the final-rowscale store.
//
// The user-defined parts arrive in "ae_config.h" / "ae_functors.h", generated from the traced
// score_mod / mask_mod / OnlineFunc graphs:
//   configuration  AE_D AE_DV AE_BN AE_NWAVES AE_RB AE_DTYPE_BF16 AE_MASK_MODE AE_HAS_MASK_MOD
//                  AE_N_ROWSCALES AE_O_SCALE_ONE AE_EVEN_Q AE_EVEN_KV AE_WAVES_PER_EU
//                  AE_K_PAD AE_V_PAD
//   functors       ae_rowstate, ae_rowstate_init, ae_mask_mod, ae_score_mod, ae_online_fwd,
//                  ae_epilogue, ae_load_custom
//
// Mapping to the hardware
//   * one workgroup = AE_NWAVES waves of one (batch, head); a wave owns AE_RB blocks of 32
//     query rows.  Every K / V fragment read from LDS feeds one MFMA per row block, so AE_RB = 2
//     halves the LDS (and HBM/L2) bytes moved per flop -- LDS read bandwidth (128 B/clk per CU,
//     exactly what four SIMDs of 32x32x16 MFMAs consume with one row block) is what bounds the
//     one-block variant;
//   * scores are computed TRANSPOSED, S^T = K Q^T, with v_mfma_f32_32x32x16: in the
//     accumulator layout every lane then owns ONE query row (column l%32) and 16 kv
//     positions per 32x32 block, so row max / row sum are in-register reductions plus one
//     exchange with lane l^32, and the online row state (m, r, o_scale, ...) is a scalar
//     per lane;
//   * the same registers, converted to fp16/bf16, are directly the B operand of
//     O^T += V^T P^T (the contraction index only has to be enumerated in the same order by
//     both operands), so P never goes through LDS;
//   * Q stays in registers as B-operand fragments for the whole kernel; K and V tiles are
//     staged HBM -> VGPR -> LDS with 16-byte coalesced loads, double-buffered so the loads
//     of tile j+1 are in flight while tile j is being multiplied; K rows are read back with
//     ds_read_b128, V is read through ds_read_b64_tr_b16 (LDS transpose load), which hands
//     each lane four kv-consecutive values of its dv column from the row-major tile.
//   * causal and block-sparse masks skip whole tiles; the elementwise mask is evaluated
//     only on tiles that are not known to be fully visible.

#include "ae_hip.h"
#include "ae_config.h"    // generated: the AE_* configuration macros
#include "ae_device.h"
// custom inputs with a kv dimension (one element per score) are fetched a tile ahead: a lane's groups of four
// consecutive kv positions per tile
#define AE_KV_PF_GROUPS (AE_BN / 8)
#include "ae_functors.h"  // generated: the functor bodies
#include "ae_tile_table.h"
#ifndef AE_HEAVY_LAST
#define AE_HEAVY_LAST 0      // 1: the tile table gives late q tiles more work than early ones
#endif

// value given to score positions past seqlen_kv before the user functors run: -inf, or 0 for graphs
// declared with mask_value="0" (no additive -inf mask anywhere, attn_tl.py:124-137 / lower.py:637)
#if defined(AE_MASK_VALUE_ZERO) && AE_MASK_VALUE_ZERO
#define AE_KV_PAD 0.f
#else
#define AE_KV_PAD AE_NEG_INF
#endif

#ifndef AE_RB
#define AE_RB 1
#endif
#define AE_WROWS (AE_RB * 32)     // query rows per wave
#define AE_BM (AE_NWAVES * AE_WROWS)
#define AE_NT (AE_NWAVES * 64)
#define AE_NB (AE_BN / 32)        // 32-wide kv blocks per tile
#define AE_NS (AE_NB * 16)        // score elements per lane per tile
#define AE_NDB (AE_DV / 32)       // 32-wide dv blocks
#define AE_NO (AE_NDB * 16)       // output elements per lane
#define AE_KSTR (AE_D * 2 + AE_K_PAD)    // LDS row pitch of the K tile, bytes
#define AE_VSTR (AE_DV * 2 + AE_V_PAD)   // LDS row pitch of the V tile, bytes
#define AE_K_BYTES (AE_BN * AE_KSTR)
#define AE_V_BYTES (AE_BN * AE_VSTR)
#define AE_STAGE_BYTES (AE_K_BYTES + AE_V_BYTES)
#define AE_KCPR (AE_D / 8)        // 16-byte chunks per K row
#define AE_VCPR (AE_DV / 8)
#define AE_K_LOADS ((AE_BN * AE_KCPR) / AE_NT)
#define AE_V_LOADS ((AE_BN * AE_VCPR) / AE_NT)

static_assert(AE_D % 16 == 0, "head dim must be a multiple of 16");
static_assert(AE_DV % 32 == 0, "value head dim must be a multiple of 32");
static_assert(AE_BN % 32 == 0, "kv tile must be a multiple of 32");
static_assert((AE_BN * AE_KCPR) % AE_NT == 0, "K tile must split evenly over the workgroup");
static_assert((AE_BN * AE_VCPR) % AE_NT == 0, "V tile must split evenly over the workgroup");
static_assert(AE_KSTR % 16 == 0 && AE_VSTR % 8 == 0, "LDS pitches must keep vector alignment");

typedef __attribute__((address_space(3))) unsigned char ae_lds_byte;

extern "C" __global__ __launch_bounds__(AE_NT)
__attribute__((amdgpu_waves_per_eu(AE_WAVES_PER_EU, AE_WAVES_PER_EU)))
void ae_prefill_kernel(const ae_attn_params p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ae_smem[];
  ae_lds_byte* lds = (ae_lds_byte*)ae_smem;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hf = lane >> 5;

  // ---- which (q-tile, head, batch) -----------------------------------------------------
  // The dispatcher deals consecutive workgroup ids round-robin to the 8 XCDs, each with its own
  // L2.  All q-tiles of one (batch, head) read the same K/V, so they are given ids that land on
  // ONE XCD back to back (id = 8*slot + xcd, slot = bh_local*n_qt + qt_i): the tiles run
  // concurrently, walk the kv axis roughly in step and share K/V through that XCD's L2.
  // With a causal mask the tiles with the most kv work (last q-tiles) are issued first.
  // The grid is padded to 8*ceil(n_bh/8)*n_qt ids; surplus workgroups exit immediately.
  const int n_qt = (p.seqlen_q + AE_BM - 1) / AE_BM;
  const int n_bh = p.batch * p.heads_q;
  const int wg = blockIdx.x;
  const int xcd = wg & 7;
  const int slot = wg >> 3;
  const int qt_i = slot % n_qt;
  const int bh = (slot / n_qt) * 8 + xcd;
  if (bh >= n_bh) return;
#if AE_MASK_MODE == 1 || (AE_MASK_MODE == 2 && AE_HEAVY_LAST)     // (long q tiles first)
  const int qt = n_qt - 1 - qt_i;
#else
  const int qt = qt_i;
#endif
  const int h = bh % p.heads_q;
  const int b = bh / p.heads_q;
  const int hk = h / (p.heads_q / p.heads_kv);
  const int q0 = qt * AE_BM;
  const int q0w = q0 + wave * AE_WROWS;       // first row of this wave
  int qrow[AE_RB];                             // this lane's row in each row block
  bool q_ok[AE_RB];
#pragma unroll
  for (int rb = 0; rb < AE_RB; rb++) {
    qrow[rb] = q0w + rb * 32 + l32;
#if AE_EVEN_Q
    q_ok[rb] = true;
#else
    q_ok[rb] = qrow[rb] < p.seqlen_q;
#endif
  }

  // ---- Q fragments: B operand of S^T = K Q^T, resident for the whole kernel -------------
  ae_elem8 qf[AE_RB][AE_D / 16];
#pragma unroll
  for (int rb = 0; rb < AE_RB; rb++) {
    const int qr = q_ok[rb] ? qrow[rb] : p.seqlen_q - 1;
    const ae_elem* qptr = (const ae_elem*)p.q + (int64_t)b * p.q_stride_b +
                          (int64_t)qr * p.q_stride_s + (int64_t)h * p.q_stride_h;
#pragma unroll
    for (int ks = 0; ks < AE_D / 16; ks++) qf[rb][ks] = *(const ae_elem8*)(qptr + ks * 16 + hf * 8);
  }

  // ---- KV tile range ---------------------------------------------------------------------
  const int n_kvt = (p.seqlen_kv + AE_BN - 1) / AE_BN;
  int j_end = n_kvt;
#if AE_MASK_MODE == 1
  {
    int lim = (q0 + AE_BM + AE_BN - 1) / AE_BN;  // attn_tl.py:113-115
    j_end = lim < n_kvt ? lim : n_kvt;
  }
#endif
#if AE_MASK_MODE == 2
  // Tile classes from the block table (ae_tile_table.h): 0 = skip, 1 = visit with the elementwise mask (every
  // position, where the graph has no mask_mod: a block mask of the user), 2 = fully visible.  A q tile may span
  // several table rows: a kv tile is skipped only if every row says so, and every lane applies the class of
  // its own row.
  ae_tile_table tt;
  ae_tt_init(tt, p, b, h, q0, AE_BM);
#endif

  const ae_elem* kbase = (const ae_elem*)p.k + (int64_t)b * p.k_stride_b + (int64_t)hk * p.k_stride_h;
  const ae_elem* vbase = (const ae_elem*)p.v + (int64_t)b * p.v_stride_b + (int64_t)hk * p.v_stride_h;

  ae_u32x4 kreg[AE_K_LOADS];
  ae_u32x4 vreg[AE_V_LOADS];

  auto load_tile = [&](int j) AE_LAMBDA {
    const int kv0 = j * AE_BN;
#pragma unroll
    for (int i = 0; i < AE_K_LOADS; i++) {
      int c = tid + i * AE_NT;
      int row = c / AE_KCPR, col = c % AE_KCPR;
      int kv = kv0 + row;
#if !AE_EVEN_KV
      kv = kv < p.seqlen_kv ? kv : p.seqlen_kv - 1;
#endif
      kreg[i] = *(const ae_u32x4*)(kbase + (int64_t)kv * p.k_stride_s + col * 8);
    }
#pragma unroll
    for (int i = 0; i < AE_V_LOADS; i++) {
      int c = tid + i * AE_NT;
      int row = c / AE_VCPR, col = c % AE_VCPR;
      int kv = kv0 + row;
#if !AE_EVEN_KV
      kv = kv < p.seqlen_kv ? kv : p.seqlen_kv - 1;
#endif
      vreg[i] = *(const ae_u32x4*)(vbase + (int64_t)kv * p.v_stride_s + col * 8);
    }
  };
  auto store_tile = [&](int stage) AE_LAMBDA {
    ae_lds_byte* ks = lds + stage * AE_STAGE_BYTES;
    ae_lds_byte* vs = ks + AE_K_BYTES;
#pragma unroll
    for (int i = 0; i < AE_K_LOADS; i++) {
      int c = tid + i * AE_NT;
      int row = c / AE_KCPR, col = c % AE_KCPR;
      *(__attribute__((address_space(3))) ae_u32x4*)(ks + row * AE_KSTR + col * 16) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < AE_V_LOADS; i++) {
      int c = tid + i * AE_NT;
      int row = c / AE_VCPR, col = c % AE_VCPR;
      *(__attribute__((address_space(3))) ae_u32x4*)(vs + row * AE_VSTR + col * 16) = vreg[i];
    }
  };
  // next tile index >= j that has work (block table) or j itself
  auto next_tile = [&](int j) AE_LAMBDA {
#if AE_MASK_MODE == 2
    j = ae_tt_next(tt, p, j, j_end, AE_BN, n_kvt);
#endif
    return j;
  };
  // class of tile j for this lane's row of row block rb (right after next_tile() found j)
  auto row_class = [&](int j, int rb) AE_LAMBDA -> int {
#if AE_MASK_MODE == 2
    return j < j_end ? ae_tt_class(tt, p, j, qrow[rb]) : 0;
#else
    return 2;
#endif
  };

  // ---- state ------------------------------------------------------------------------------
  ae_ctx ctx[AE_RB];
  ae_custom cust[AE_RB];
  ae_rowstate st[AE_RB];
  ae_f32x16 oacc[AE_RB][AE_NDB];
#pragma unroll
  for (int rb = 0; rb < AE_RB; rb++) {
    ctx[rb].b = b;
    ctx[rb].h = h;
    ctx[rb].q_idx = qrow[rb];
    ctx[rb].kv_base = 0;
    ae_load_custom(cust[rb], p, ctx[rb]);
    ae_rowstate_init(st[rb]);
#pragma unroll
    for (int db = 0; db < AE_NDB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[rb][db][r] = 0.f;
  }

  // lane-constant LDS offsets
  const int k_rd_off = l32 * AE_KSTR + hf * 16;                     // + nb*32*KSTR + ks*32
  const int v_rd_off = (4 * hf + ((lane & 15) >> 2)) * AE_VSTR +     // + rowbase*VSTR + db*64
                       ((l32 >> 4) * 16 + 4 * (lane & 3)) * 2;

  int j = next_tile(0);
  bool any_tile = j < j_end;
  int cls[AE_RB];          // class of tile j for this lane's row of each row block
  // 1 once this lane's row of a row block has met a key it may see.  A row that never does - inside a q tile whose
  // other rows do: block masks finer than the q tile, masks such as q - 100 >= kv - ends with out = 0 and row
  // scales of -inf, like the rows of a q tile without any tile (not with the 0 / 0 its epilogue would make of it)
  float seen[AE_RB];
#pragma unroll
  for (int rb = 0; rb < AE_RB; rb++) seen[rb] = 0.f;
#pragma unroll
  for (int rb = 0; rb < AE_RB; rb++) cls[rb] = row_class(j, rb);
  if (any_tile) {
    load_tile(j);
    store_tile(0);
#ifdef AE_HAS_KV_PREFETCH
#pragma unroll
    for (int rb = 0; rb < AE_RB; rb++) ae_prefetch_custom(cust[rb], j * AE_BN + 4 * hf, q0w + rb * 32, j * AE_BN, p);
#endif
  }
  // Drain every outstanding load (Q fragments, first tile) before the loop: with loads still
  // pending at the loop header the compiler's wait-count insertion makes the QK^T MFMAs of every
  // iteration wait for that iteration's K/V prefetch, which serialises the pipeline.
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();

  int stage = 0;
  while (j < j_end) {
    const int jn = next_tile(j + 1);
    int cls_n[AE_RB];
#pragma unroll
    for (int rb = 0; rb < AE_RB; rb++) cls_n[rb] = row_class(jn, rb);
    if (jn < j_end) load_tile(jn);

    ae_lds_byte* ks_ = lds + stage * AE_STAGE_BYTES;
    ae_lds_byte* vs_ = ks_ + AE_K_BYTES;
    const int kv0 = j * AE_BN;

    // ---- S^T = K Q^T: every K fragment feeds one MFMA per row block -------------------------
    ae_f32x16 sacc[AE_RB][AE_NB];
#pragma unroll
    for (int rb = 0; rb < AE_RB; rb++)
#pragma unroll
      for (int nb = 0; nb < AE_NB; nb++)
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[rb][nb][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < AE_D / 16; ks++) {
#pragma unroll
      for (int nb = 0; nb < AE_NB; nb++) {
        ae_elem8 kf = *(__attribute__((address_space(3))) ae_elem8*)(
            ks_ + k_rd_off + nb * 32 * AE_KSTR + ks * 32);
#pragma unroll
        for (int rb = 0; rb < AE_RB; rb++) sacc[rb][nb] = ae_mfma32(kf, qf[rb][ks], sacc[rb][nb]);
      }
    }

    ae_elem8 pf[AE_RB][AE_BN / 16];
#pragma unroll
    for (int rb = 0; rb < AE_RB; rb++) {
      float s[AE_NS];
#pragma unroll
      for (int nb = 0; nb < AE_NB; nb++)
#pragma unroll
        for (int r = 0; r < 16; r++) s[nb * 16 + r] = sacc[rb][nb][r];
      ctx[rb].kv_base = kv0 + 4 * hf;
      const int kvb = ctx[rb].kv_base;

      // ---- mask (additive -inf before score_mod, attn_tl.py:124-137) --------------------------
      bool masked_here = false;    // some score of this row block was tested on this tile
#if AE_MASK_MODE == 1
      if (kv0 + AE_BN - 1 > q0w + rb * 32) {  // tile crosses the diagonal of this row block
        masked_here = true;
#pragma unroll
        for (int e = 0; e < AE_NS; e++) s[e] = (qrow[rb] >= kvb + ae_kv_off(e)) ? s[e] : AE_NEG_INF;
      }
#elif AE_MASK_MODE == 2 && !(defined(AE_MASK_VALUE_ZERO) && AE_MASK_VALUE_ZERO)
      if (__builtin_amdgcn_ballot_w64(cls[rb] != 2) != 0) {   // some row of this block does not see the whole tile
        masked_here = true;
#pragma unroll
        for (int e = 0; e < AE_NS; e++) {
#if AE_HAS_MASK_MOD
          const bool vis = cls[rb] == 2 || (cls[rb] == 1 && ae_mask_mod(b, h, qrow[rb], kvb + ae_kv_off(e)));
#else
          const bool vis = cls[rb] != 0;
#endif
          s[e] = vis ? s[e] : AE_NEG_INF;
        }
      }
#elif AE_HAS_MASK_MOD
      {
        masked_here = true;
#pragma unroll
        for (int e = 0; e < AE_NS; e++)
          s[e] = ae_mask_mod(b, h, qrow[rb], kvb + ae_kv_off(e)) ? s[e] : AE_NEG_INF;
      }
#endif
#if !AE_EVEN_KV
      if (kv0 + AE_BN > p.seqlen_kv) {
        masked_here = true;
#pragma unroll
        for (int e = 0; e < AE_NS; e++) s[e] = (kvb + ae_kv_off(e) < p.seqlen_kv) ? s[e] : AE_KV_PAD;
      }
#endif
      if (masked_here) {           // (an untested tile is visible to every row)
        float top = s[0];
#pragma unroll
        for (int e = 1; e < AE_NS; e++) top = __builtin_fmaxf(top, s[e]);
        seen[rb] = top > AE_NEG_INF ? 1.f : seen[rb];
      } else {
        seen[rb] = 1.f;
      }

      // ---- user functors ----------------------------------------------------------------------
      ae_score_mod<AE_NS>(s, ctx[rb], cust[rb]);
      float o_scale = ae_online_fwd<AE_NS>(s, st[rb], ctx[rb], cust[rb]);
#ifdef AE_HAS_KV_PREFETCH
      // the functors are done with this tile's elements of the per-score custom inputs: request the next
      // tile's, which travel while the second product runs
      if (jn < j_end) ae_prefetch_custom(cust[rb], jn * AE_BN + 4 * hf, q0w + rb * 32, jn * AE_BN, p);
#endif

#if !AE_EVEN_KV
      if (kv0 + AE_BN > p.seqlen_kv) {
#pragma unroll
        for (int e = 0; e < AE_NS; e++) s[e] = (kvb + ae_kv_off(e) < p.seqlen_kv) ? s[e] : 0.f;
      }
#endif

      // ---- P -> B-operand fragments -----------------------------------------------------------
#pragma unroll
      for (int kk = 0; kk < AE_BN / 16; kk++)
#pragma unroll
        for (int t = 0; t < 8; t++) pf[rb][kk][t] = (ae_elem)s[kk * 8 + t];

#if !AE_O_SCALE_ONE
      // skip the rescale when no row of this block changed its scale (wave-uniform branch)
      if (__builtin_amdgcn_ballot_w64(o_scale != 1.0f) != 0) {
#pragma unroll
        for (int db = 0; db < AE_NDB; db++)
#pragma unroll
          for (int r = 0; r < 16; r++) oacc[rb][db][r] *= o_scale;
      }
#else
      (void)o_scale;
#endif
    }

    // ---- O^T += V^T P^T: every V fragment feeds one MFMA per row block ------------------------
#pragma unroll
    for (int kk = 0; kk < AE_BN / 16; kk++) {
      // slots 0..3 of this k-step are kv rows rb0+4*hf+0..3, slots 4..7 rows rb0+8+4*hf+0..3
      const int rb0 = (kk >> 1) * 32 + (kk & 1) * 16;
#pragma unroll
      for (int db = 0; db < AE_NDB; db++) {
        ae_lds_byte* a0 = vs_ + v_rd_off + rb0 * AE_VSTR + db * 64;
        ae_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) ae_s16x4*)a0);
        ae_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) ae_s16x4*)(a0 + 8 * AE_VSTR));
        ae_elem8 vf = __builtin_bit_cast(
            ae_elem8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
        for (int rb = 0; rb < AE_RB; rb++) oacc[rb][db] = ae_mfma32(vf, pf[rb][kk], oacc[rb][db]);
      }
    }

    if (jn < j_end) store_tile(stage ^ 1);
    __syncthreads();
    stage ^= 1;
    j = jn;
#pragma unroll
    for (int rb = 0; rb < AE_RB; rb++) cls[rb] = cls_n[rb];
  }

  // ---- epilogue -------------------------------------------------------------------------------
#pragma unroll
  for (int rb = 0; rb < AE_RB; rb++) {
    float o[AE_NO];
#pragma unroll
    for (int db = 0; db < AE_NDB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[db * 16 + r] = oacc[rb][db][r];
    float frs[AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1];
    frs[0] = 0.f;
    const bool row_seen = ae_group_max(seen[rb]) > 0.f;     // (both lanes of a row, or neither)
    if (any_tile && row_seen) {
      ae_epilogue<AE_NO>(o, st[rb], frs, ctx[rb], cust[rb]);
    } else {
      // no visible kv block for this q-tile, or no visible key for this row: out = 0 (blockattn_tl.py:153-160),
      // rowscales = -inf
#pragma unroll
      for (int e = 0; e < AE_NO; e++) o[e] = 0.f;
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++) frs[i] = AE_NEG_INF;
    }
    if (q_ok[rb]) {
      ae_elem* optr = (ae_elem*)p.out + (int64_t)b * p.o_stride_b + (int64_t)qrow[rb] * p.o_stride_s +
                      (int64_t)h * p.o_stride_h;
#pragma unroll
      for (int db = 0; db < AE_NDB; db++)
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          ae_elem4 w;
#pragma unroll
          for (int t = 0; t < 4; t++) w[t] = (ae_elem)o[db * 16 + rg * 4 + t];
          *(ae_elem4*)(optr + db * 32 + rg * 8 + hf * 4) = w;
        }
      if (hf == 0) {
#pragma unroll
        for (int i = 0; i < AE_N_ROWSCALES; i++)
          p.rowscale_out[i][((int64_t)b * p.heads_q + h) * p.seqlen_q + qrow[rb]] = frs[i];
      }
    }
  }
}
