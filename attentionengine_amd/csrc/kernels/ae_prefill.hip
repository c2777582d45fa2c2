// Flash-style attention forward (prefill) for gfx950 / CDNA4 with direct-to-LDS tile loads.
//
// Takes the place of the reference's TileLang prefill template
// (attention_engine/core/template/tl_template/attn/attn_tl.py:76-174) and its block-sparse
// sibling (blockattn_tl.py:49-160).  Per KV tile it keeps the reference's order of operations
// (attn_tl.py:124-164): mask -> +QK^T -> score_mod -> online_func -> cast P -> rescale O ->
// O += P V, then the epilogue and the final-rowscale store.
//
// The user-defined parts arrive in "ae_config.h" / "ae_functors.h", generated from the traced
// score_mod / mask_mod / OnlineFunc graphs (head dims 64, 128, 256; value head dims 64 ... 512):
//   configuration  AE_D AE_DV AE_BN AE_NWAVES AE_DTYPE_BF16 AE_MASK_MODE AE_HAS_MASK_MOD
//                  AE_N_ROWSCALES AE_O_SCALE_ONE AE_EVEN_Q AE_EVEN_KV AE_WAVES_PER_EU
//   functors       ae_rowstate, ae_rowstate_init, ae_mask_mod, ae_score_mod, ae_online_fwd,
//                  ae_epilogue, ae_load_custom
//
// Same mapping to the matrix cores as ae_prefill_simple.hip (which documents the register layouts
// in full): S^T = K Q^T and O^T += V^T P^T with v_mfma_f32_32x32x16, one query row per lane, Q in
// registers, P handed from the first product to the second without leaving registers.
//
// What differs is how K / V tiles reach LDS.  Measured on MI355X, staging a tile through VGPRs
// (global_load -> 32 registers -> ds_write_b128) costs this kernel a third of its throughput: the
// wave issues in order, so the extra loads, the wait for them and the LDS writes all sit on the
// critical path of the two waves that share a SIMD.  Here every lane issues
// `global_load_lds_dwordx4` instead: 16 bytes go from HBM/L2 straight into LDS at
// (wave-uniform base) + lane*16, no VGPRs, no ds_write, and the only wait is one vmcnt(0) in front
// of the barrier that publishes the tile.  A direct load cannot pad rows (64 lanes fill 1 KiB
// contiguously), so bank conflicts are avoided by permuting WHICH 16-byte chunk of its row a lane
// fetches:
//     K tile: LDS chunk c' of row r holds global chunk c' ^ (r mod chunks_per_row), so the
//             ds_read_b128 of 16 consecutive rows at one d offset hits 16 different bank groups;
//     V tile: the permutation works on 32-byte pairs, (c'/2) ^ (r mod pairs_per_row), which keeps
//             the 4 rows x 32 bytes of one ds_read_b64_tr_b16 group on distinct banks.
// Tiles are double buffered: tile j+1 streams in while tile j is multiplied.

#include "ae_hip.h"
#include "ae_config.h"    // generated: the AE_* configuration macros
#ifndef AE_NSPLIT
#define AE_NSPLIT 1                // > 1: split-KV, fp32 partial results + the merge kernel of ae_combine.h
#endif
#include "ae_device.h"
// custom inputs with a kv dimension (one element per score) are fetched a tile ahead: a lane's groups of four
// consecutive kv positions per tile
#define AE_KV_PF_GROUPS (AE_BN / 8)
// ... in a coalesced layout that each wave redistributes through AE_KV_SCRATCH bytes of LDS of its own per row block
// (builds with two waves per SIMD; with one, the 16 extra registers and the staging cost more than they save:
// retention at D 256, DV 512 0.88 against 0.78 ms)
#define AE_KV_COALESCED (AE_WAVES_PER_EU >= 2)
#define AE_KV_SCRATCH 2560
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
#define AE_KSTR (AE_D * 2)        // LDS row pitch of the K tile, bytes (no padding: swizzled)
#define AE_VSTR (AE_DV * 2)       // LDS row pitch of the V tile, bytes
#define AE_K_BYTES (AE_BN * AE_KSTR)
#define AE_V_BYTES (AE_BN * AE_VSTR)
#define AE_STAGE_BYTES (AE_K_BYTES + AE_V_BYTES)
#define AE_KCPR (AE_D / 8)        // 16-byte chunks per K row
#define AE_VCPR (AE_DV / 8)
#define AE_K_LOADS ((AE_BN * AE_KCPR) / AE_NT)   // direct loads per lane per K tile
#define AE_V_LOADS ((AE_BN * AE_VCPR) / AE_NT)
#define AE_V_RPI (64 / AE_VCPR)
#define AE_VPPR (AE_VCPR / 2)     // 32-byte pairs per V row
// the pairs of a V row are exchanged by the row's low bits: at most three of them, so that rows 8 apart (the
// two halves of a transposed fragment) share one permutation whatever the row length
#define AE_VSWM ((AE_VPPR < 8 ? AE_VPPR : 8) - 1)

static_assert(AE_D % 16 == 0, "head dim must be a multiple of 16");
static_assert(AE_DV % 32 == 0, "value head dim must be a multiple of 32");
static_assert(AE_BN % 32 == 0, "kv tile must be a multiple of 32");
static_assert((AE_BN * AE_KCPR) % AE_NT == 0, "K tile must split evenly over the workgroup");
static_assert((AE_BN * AE_VCPR) % AE_NT == 0, "V tile must split evenly over the workgroup");
static_assert(AE_K_LOADS >= 1 && AE_K_LOADS <= 8 && AE_V_LOADS >= 1 && AE_V_LOADS <= 8, "one burst per tile and wave");
static_assert(AE_KCPR == 8 || AE_KCPR == 16 || AE_KCPR == 32 || AE_KCPR % 8 == 4 || AE_KCPR % 16 == 8,
              "swizzle is written for K rows of 128, 256 or 512 bytes, or an odd multiple of 64 or 128 bytes");
static_assert(AE_VCPR == 8 || AE_VCPR == 16 || AE_VCPR == 32 || AE_VCPR == 64, "swizzle is written for 128- to 1024-byte V rows");

typedef __attribute__((address_space(3))) unsigned char ae_lds_byte;

// LDS chunk of K row `row` that holds global chunk c (and the other way round: an involution).  A fragment read
// (ds_read_b128) takes one chunk index of 16 consecutive rows; they must fall into 16 different groups of four
// banks.  Rows of a power-of-two length all start in the same group, so the chunk index is exchanged by the row
// number.  Rows of 8*odd chunks (head dim 192: 384 bytes) start in two alternating groups and rows of 4*odd
// chunks (head dims 96, 160) in four, so only the low three (two) bits of the chunk index are exchanged, by the
// row number without the bits that the row pitch already spreads.
AE_DEV int ae_k_swz(int c, int row) {
#if (AE_KCPR & (AE_KCPR - 1)) == 0
  return c ^ (row & (AE_KCPR - 1));
#elif AE_KCPR % 16 == 8
  return c ^ ((row >> 1) & 7);
#else
  return c ^ ((row >> 2) & 3);
#endif
}

// Q rows on their way in and O rows on their way out pass through LDS as whole rows (16 lanes per 256-byte row).
// A lane that loads its own row's fragments, or stores its own row's results, touches 32 rows per instruction,
// 16 bytes of each: the workgroups of a launch start and end together and queue behind each other's requests
// (measured in the pipelined kernel: 3.5 us until the first tile could be multiplied, 4.4 us to get O out).
// Q uses stage 1 of the tile ring, which is free until the loop's first prefetch, swizzled like a K tile; O the
// whole ring after the last tile.  Builds whose rows do not fit there keep the direct accesses.
#define AE_Q_LOADS ((AE_WROWS * AE_KCPR) / 64)     // direct loads per lane for the wave's Q rows
#define AE_Q_VIA_LDS (AE_BM * AE_KSTR <= AE_STAGE_BYTES)
#define AE_O_LOADS ((AE_WROWS * AE_VCPR) / 64)
#define AE_O_VIA_LDS (AE_NSPLIT == 1 && AE_NO <= 128 && AE_BM * AE_VSTR <= 2 * AE_STAGE_BYTES)

// the wave's Q rows -> qs, in bursts of up to eight loads.  qg: row q0c of this (batch, head), 4 KiB low (see
// ae_load_lds16_burst_base); row0 = first row of the wave - q0c; rows past `last` (relative to q0c) re-read it.
template <int G0>
AE_DEV void ae_q_rows_to_lds(const char* qg, ae_lds_byte* qs, int lane, int row0, int last, int stride_s) {
  if constexpr (G0 < AE_Q_LOADS) {
    constexpr int N = AE_Q_LOADS - G0 < 8 ? AE_Q_LOADS - G0 : 8;
    unsigned off[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int n = (G0 + (i < N ? i : 0)) * 64 + lane;      // chunk of the wave's rows, in LDS order
      const int row = n / AE_KCPR;
      const int c = ae_k_swz(n % AE_KCPR, row);
      int ra = row0 + row;
      ra = ra < last ? ra : last;
      off[i] = (unsigned)((ra * stride_s + c * 8) * 2 + 4096 - (i - N / 2) * 1024);
    }
    ae_load_lds16_burst_base<N>(qg, off, qs + (G0 + N / 2) * 1024);
    ae_q_rows_to_lds<G0 + 8>(qg, qs, lane, row0, last, stride_s);
  }
}

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
#if AE_NSPLIT > 1
  // split-KV ("decode" with several query tokens): consecutive ids are the splits of one q tile
  const int split = blockIdx.x % AE_NSPLIT;
  const int wg = blockIdx.x / AE_NSPLIT;
#else
  const int wg = blockIdx.x;
#endif
  const int xcd = wg & 7;
  const int slot = wg >> 3;
#if AE_MASK_MODE == 1 || (AE_MASK_MODE == 2 && AE_HEAVY_LAST)
  // causal: q tiles differ in work by up to n_qt : 1, so ids go heaviest tile first across ALL heads
  // (longest-job-first keeps the tail short); the heads of one XCD still meet in its L2.  A tile table whose
  // late q tiles are the long ones (AE_HEAVY_LAST, found on the host: causal variants, long sliding windows)
  // takes the same order: B2 H32 S4096, "kv <= q + 1": 0.40 -> 0.35 ms.
  const int n_bg = (n_bh + 7) >> 3;
  const int qt = n_qt - 1 - slot / n_bg;
  const int bh = (slot % n_bg) * 8 + xcd;
#else
  const int qt = slot % n_qt;
  const int bh = (slot / n_qt) * 8 + xcd;
#endif
  if (bh >= n_bh) return;
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
#if AE_Q_VIA_LDS
  ae_lds_byte* qs = lds + AE_STAGE_BYTES + wave * (AE_WROWS * AE_KSTR);
  {
    const int q0c = q0w < p.seqlen_q ? q0w : p.seqlen_q - 1;
    const char* qg = (const char*)((const ae_elem*)p.q + (int64_t)b * p.q_stride_b + (int64_t)q0c * p.q_stride_s +
                                   (int64_t)h * p.q_stride_h) - 4096;
    ae_q_rows_to_lds<0>(qg, qs, lane, q0w - q0c, p.seqlen_q - 1 - q0c, (int)p.q_stride_s);
  }
#else
#pragma unroll
  for (int rb = 0; rb < AE_RB; rb++) {
    const int qr = q_ok[rb] ? qrow[rb] : p.seqlen_q - 1;
    const ae_elem* qptr = (const ae_elem*)p.q + (int64_t)b * p.q_stride_b +
                          (int64_t)qr * p.q_stride_s + (int64_t)h * p.q_stride_h;
#pragma unroll
    for (int ks = 0; ks < AE_D / 16; ks++) qf[rb][ks] = *(const ae_elem8*)(qptr + ks * 16 + hf * 8);
  }
#endif

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

  // Direct HBM -> LDS tile load.  Wave w, instruction i covers the 64 consecutive 16-byte chunks
  // (w*LOADS + i)*64 ... of the tile (whole rows when the row length is a power of two); lane L lands in LDS
  // chunk c' of row r, (w*LOADS + i)*64 + L = r*CPR + c', and fetches the permuted global chunk.
  // A lane's byte offset inside a tile never changes, so it is computed once; per tile only a
  // wave-uniform base moves.  The K loads and the V loads of a wave each go out as one burst behind a
  // single write of M0 (see ae_load_lds16_burst_base: bases are passed 4 KiB low and the offsets 4 KiB
  // high, so that the offsets, which carry the compensation for the immediate offsets, stay >= 0).
  auto k_lane_off = [&](int i, int last_row) AE_LAMBDA -> unsigned {
    const int chunk = (wave * AE_K_LOADS + i) * 64 + lane;     // of the tile, in LDS order
    int row = chunk / AE_KCPR;
    const int c = ae_k_swz(chunk % AE_KCPR, row);
    row = row < last_row ? row : last_row;
    return (unsigned)((row * (int)p.k_stride_s + c * 8) * 2 + 4096 - (i - AE_K_LOADS / 2) * 1024);
  };
  auto v_lane_off = [&](int i, int last_row) AE_LAMBDA -> unsigned {
    int row = (wave * AE_V_LOADS + i) * AE_V_RPI + lane / AE_VCPR;
    const int cp = lane % AE_VCPR;
    const int c = (((cp >> 1) ^ (row & AE_VSWM)) << 1) | (cp & 1);
    row = row < last_row ? row : last_row;
    return (unsigned)((row * (int)p.v_stride_s + c * 8) * 2 + 4096 - (i - AE_V_LOADS / 2) * 1024);
  };
  unsigned koff[AE_K_LOADS], voff[AE_V_LOADS];
#pragma unroll
  for (int i = 0; i < AE_K_LOADS; i++) koff[i] = k_lane_off(i, AE_BN);
#pragma unroll
  for (int i = 0; i < AE_V_LOADS; i++) voff[i] = v_lane_off(i, AE_BN);
  auto load_tile = [&](int j, int stage) AE_LAMBDA {
    ae_lds_byte* ks = lds + stage * AE_STAGE_BYTES;
    ae_lds_byte* vs = ks + AE_K_BYTES;
    const char* gk = (const char*)kbase + (int64_t)j * AE_BN * p.k_stride_s * 2 - 4096;
    const char* gv = (const char*)vbase + (int64_t)j * AE_BN * p.v_stride_s * 2 - 4096;
    unsigned ko[8], vo[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      ko[i] = koff[i < AE_K_LOADS ? i : 0];
      vo[i] = voff[i < AE_V_LOADS ? i : 0];
#if !AE_EVEN_KV
      // rows past the end re-read the last row (masked later)
      if (j * AE_BN + AE_BN > p.seqlen_kv) {
        ko[i] = k_lane_off(i < AE_K_LOADS ? i : 0, p.seqlen_kv - 1 - j * AE_BN);
        vo[i] = v_lane_off(i < AE_V_LOADS ? i : 0, p.seqlen_kv - 1 - j * AE_BN);
      }
#endif
    }
    ae_load_lds16_burst_base<AE_K_LOADS>(gk, ko, ks + (wave * AE_K_LOADS + AE_K_LOADS / 2) * 1024);
    ae_load_lds16_burst_base<AE_V_LOADS>(gv, vo, vs + (wave * AE_V_LOADS + AE_V_LOADS / 2) * 1024);
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

  // lane-constant pieces of the swizzled LDS read addresses
  // K fragment (row l32 of a 32-row block, d chunk 2*ks+hf): chunk' = (2*ks+hf) ^ (l32 mod CPR)
  const int k_row_off = l32 * AE_KSTR;
  // V transpose read: lane i of a 16-lane group reads row 4*hf + i/4 (+8), 8 bytes at pair
  // (2*db + g) ^ (row mod PPR), g = (lane%32)/16; rows of one group differ only in their low bits
  const int v_row = 4 * hf + ((lane & 15) >> 2);
  const int v_row_off = v_row * AE_VSTR + (lane & 3) * 8;
  const int v_sw = v_row & AE_VSWM;
  const int v_g = l32 >> 4;

#if AE_NSPLIT > 1
  // this workgroup's share of the kv axis: kv_per_split positions (a multiple of the tile)
  const int j_begin = split * (p.kv_per_split / AE_BN);
  {
    const int lim = j_begin + p.kv_per_split / AE_BN;
    j_end = lim < j_end ? lim : j_end;
  }
  int j = next_tile(j_begin);
#else
  int j = next_tile(0);
#endif
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
  if (any_tile) load_tile(j, 0);
#ifdef AE_HAS_KV_PREFETCH
  if (any_tile) {
#pragma unroll
    for (int rb = 0; rb < AE_RB; rb++) ae_prefetch_custom(cust[rb], j * AE_BN + 4 * hf, q0w + rb * 32, j * AE_BN, p);
  }
#endif
  // Drain every outstanding load (Q fragments, first tile) before the loop: with loads still
  // pending at the loop header the compiler's wait-count insertion makes the QK^T MFMAs of every
  // iteration wait for that iteration's K/V prefetch, which serialises the pipeline.
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
#if AE_Q_VIA_LDS
#pragma unroll
  for (int rb = 0; rb < AE_RB; rb++)
#pragma unroll
    for (int ks = 0; ks < AE_D / 16; ks++)
      qf[rb][ks] = *(const __attribute__((address_space(3))) ae_elem8*)(
          qs + (rb * 32 + l32) * AE_KSTR + (ae_k_swz(2 * ks + hf, l32) << 4));
  __syncthreads();      // every wave has its fragments before the loop's first prefetch refills stage 1
#endif

  int stage = 0;
  while (j < j_end) {
    const int jn = next_tile(j + 1);
    int cls_n[AE_RB];
#pragma unroll
    for (int rb = 0; rb < AE_RB; rb++) cls_n[rb] = row_class(jn, rb);
    if (jn < j_end) load_tile(jn, stage ^ 1);   // streams into the other stage while this one is used

    ae_lds_byte* ks_ = lds + stage * AE_STAGE_BYTES;
    ae_lds_byte* vs_ = ks_ + AE_K_BYTES;
    const int kv0 = j * AE_BN;
#if AE_WAVES_PER_EU == 1 && (AE_RB * (AE_NO + AE_NS) <= 256 || AE_O_SCALE_ONE)
    // (builds that use both register files: naming O as accumulator-file values once per tile keeps the
    // register allocator from moving parts of it between the files around the functor code.  Not where O
    // alone fills the accumulator file and the loop also rescales it: there the hint turns into spills -
    // measured 6.2 against 0.52 ms for the softmax at D 256, DV 512, while retention, whose normalisation
    // is deferred, gains from it: 1.00 -> 0.78 ms)
#pragma unroll
    for (int rb = 0; rb < AE_RB; rb++)
#pragma unroll
      for (int db = 0; db < AE_NDB; db++) asm volatile("" : "+a"(oacc[rb][db]));
#endif

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
            ks_ + k_row_off + nb * 32 * AE_KSTR + (ae_k_swz(2 * ks + hf, l32) << 4));
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
#if defined(AE_HAS_KV_PREFETCH) && AE_KV_COALESCED
      // per-score custom inputs: from the coalesced layout they were fetched in to the lanes that own them
      ae_stage_custom(cust[rb], lds + 2 * AE_STAGE_BYTES + (wave * AE_RB + rb) * AE_KV_SCRATCH);
#endif
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
          for (int r = 0; r < 16; r++) {
#if AE_WAVES_PER_EU == 1
            // builds with one wave per SIMD keep O in the accumulator file: one register at a time through one
            // scratch register (as plain arithmetic the allocator wants all of O in ordinary registers)
            float o = oacc[rb][db][r], t;
            asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\tv_accvgpr_write_b32 %0, %1"
                         : "+a"(o), "=&v"(t) : "v"(o_scale));
            oacc[rb][db][r] = o;
#else
            oacc[rb][db][r] *= o_scale;
#endif
          }
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
        // (rb0 and +8 are multiples of 8, so they do not change the swizzle)
        ae_lds_byte* a0 = vs_ + v_row_off + rb0 * AE_VSTR + (((2 * db + v_g) ^ v_sw) << 5);
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

    // the next tile must have landed before anyone reads it: direct loads are tracked by vmcnt
    __builtin_amdgcn_s_waitcnt(0x0070 | 0x0f00 | 0x0000);  // vmcnt(0), expcnt/lgkmcnt untouched
    __syncthreads();
    stage ^= 1;
    j = jn;
#pragma unroll
    for (int rb = 0; rb < AE_RB; rb++) cls[rb] = cls_n[rb];
  }

  // ---- epilogue -------------------------------------------------------------------------------
#if AE_NO > 128 && AE_NSPLIT == 1
  // wide value heads: the epilogue functor (elementwise over the value columns) runs one 32-column block at a
  // time; a copy of all of O next to its accumulators would not fit the register file
#pragma unroll
  for (int rb = 0; rb < AE_RB; rb++) {
    float frs[AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1];
    frs[0] = 0.f;
    const bool row_seen = ae_group_max(seen[rb]) > 0.f;     // (both lanes of a row, or neither)
    ae_elem* optr = (ae_elem*)p.out + (int64_t)b * p.o_stride_b + (int64_t)qrow[rb] * p.o_stride_s +
                    (int64_t)h * p.o_stride_h;
#pragma unroll
    for (int db = 0; db < AE_NDB; db++) {
      // (read where it is used: as plain copies the accumulator reads of EVERY block move to the front, which
      // takes the whole register file and spills; a volatile asm statement stays behind the previous block's stores)
      float o[16];
#pragma unroll
      for (int r = 0; r < 16; r++) asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(o[r]) : "a"(oacc[rb][db][r]));
      if (any_tile && row_seen) {
        ae_epilogue<16>(o, st[rb], frs, ctx[rb], cust[rb]);
      } else {
#pragma unroll
        for (int r = 0; r < 16; r++) o[r] = 0.f;
#pragma unroll
        for (int i = 0; i < AE_N_ROWSCALES; i++) frs[i] = AE_NEG_INF;
      }
      if (q_ok[rb]) {
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          ae_elem4 w;
#pragma unroll
          for (int t = 0; t < 4; t++) w[t] = (ae_elem)o[rg * 4 + t];
          *(ae_elem4*)(optr + db * 32 + rg * 8 + hf * 4) = w;
        }
      }
    }
    if (q_ok[rb] && hf == 0) {
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++)
        p.rowscale_out[i][((int64_t)b * p.heads_q + h) * p.seqlen_q + qrow[rb]] = frs[i];
    }
  }
#else
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
#if AE_NSPLIT > 1
    // partial result of this split: fp32, rows ordered (batch, q position, head) so that the merge
    // kernel sees them as B x (Sq*Hq) "heads" of a one-token decode and writes out [B,Sq,Hq,DV]
    if (q_ok[rb]) {
      const int64_t prow = ((((int64_t)b * p.seqlen_q + qrow[rb]) * p.heads_q + h) * AE_NSPLIT) + split;
      float* po = p.partial_o + prow * AE_DV;
#pragma unroll
      for (int db = 0; db < AE_NDB; db++)
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          ae_f32x4 w = {o[db * 16 + rg * 4 + 0], o[db * 16 + rg * 4 + 1], o[db * 16 + rg * 4 + 2], o[db * 16 + rg * 4 + 3]};
          *(ae_f32x4*)(po + db * 32 + rg * 8 + hf * 4) = w;
        }
      if (hf == 0) {
#pragma unroll
        for (int i = 0; i < AE_N_ROWSCALES; i++)
          p.partial_rs[(int64_t)i * p.batch * p.seqlen_q * p.heads_q * AE_NSPLIT + prow] = frs[i];
      }
    }
#elif AE_O_VIA_LDS
    {
      // (addresses from a copy of the lane id that the compiler cannot trace back to the prologue's, which have
      // the same form: it would keep those in registers across the loop)
      int le = lane;
      asm volatile("" : "+v"(le));
      ae_lds_byte* orow = lds + wave * (AE_WROWS * AE_VSTR) + (rb * 32 + (le & 31)) * AE_VSTR + (le >> 5) * 8;
      const int osw = le & (AE_VCPR - 1);
#pragma unroll
      for (int db = 0; db < AE_NDB; db++)
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          ae_elem4 w;
#pragma unroll
          for (int t = 0; t < 4; t++) w[t] = (ae_elem)o[db * 16 + rg * 4 + t];
          *(__attribute__((address_space(3))) ae_elem4*)(orow + (((db * 4 + rg) ^ osw) << 4)) = w;
        }
    }
    if (q_ok[rb] && hf == 0) {
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++)
        p.rowscale_out[i][((int64_t)b * p.heads_q + h) * p.seqlen_q + qrow[rb]] = frs[i];
    }
#else
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
#endif
  }
#if AE_O_VIA_LDS
  // (the rows were written by other lanes of this wave: LDS instructions of a wave complete in order)
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  {
    ae_elem* og = (ae_elem*)p.out + (int64_t)b * p.o_stride_b + (int64_t)h * p.o_stride_h;
    const ae_lds_byte* os = lds + wave * (AE_WROWS * AE_VSTR);
    int le = lane;
    asm volatile("" : "+v"(le));
#pragma unroll
    for (int i = 0; i < AE_O_LOADS; i++) {
      const int n = i * 64 + le;
      const int row = n / AE_VCPR;
      const int c = n % AE_VCPR;
      const ae_elem8 w = *(const __attribute__((address_space(3))) ae_elem8*)(
          os + row * AE_VSTR + ((c ^ (row & (AE_VCPR - 1))) << 4));
      if (AE_EVEN_Q || q0w + row < p.seqlen_q) *(ae_elem8*)(og + (int64_t)(q0w + row) * p.o_stride_s + c * 8) = w;
    }
  }
#endif
#endif  // wide value heads
}

#if AE_NSPLIT > 1
#include "ae_combine.h"
#endif
