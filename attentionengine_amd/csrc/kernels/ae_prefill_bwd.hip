// Backward of softmax attention (prefill shapes) for gfx950 / CDNA4: dQ, dK, dV from dO.
//
// Role of the reference's backward kernels for attn_script/mha.py
// (attention_engine/core/template/tl_template/attn/attn_tl.py: flashattn_bwd_preprocess 196-221,
// flashattn_bwd 238-420, flashattn_bwd_postprocess 422-455), for the graphs the lowering has proven
// to be the online softmax of `score * constant`:
//     p = exp(s*c - lse)                      (OnlineSoftmax.forward,  mha.py:75-78)
//     dv = p^T do,  dp = do v^T
//     ds = p * (dp - rowsum(do * o)) * c      (OnlineSoftmax.backward, mha.py:80-84; d score_mod = c)
//     dq = ds k,  dk = ds^T q
// The reference accumulates dq with fp32 atomics from the kernel that owns a kv tile and converts it
// in a third kernel.  Here the work is split by OUTPUT instead, with no atomics and a fixed summation
// order: one launch owns q rows and produces dq, one owns kv rows and produces dk and dv; both
// recompute s and dp (7 tile products per tile pair instead of 5).  They are the same code with the
// operands exchanged (AE_BWD_ROLE):
//     role 0 (dq):      resident rows = q  (Q, dO in registers), streamed tiles = K, V
//     role 1 (dk, dv):  resident rows = kv (K, V in registers),  streamed tiles = Q, dO of every q head
//                       of the kv head's group, with their lse and rowsum(do * o)
// A wave owns 32 resident rows as the B operand (n = row) of v_mfma_f32_32x32x16, so a lane owns ONE
// resident row: S[streamed, resident] = X1 R1^T and dP = X2 R2^T come out with the streamed rows in
// a lane's 16 accumulator registers, which makes the packed p and ds the B operand of the second
// set of products, OUT^T[d, resident] += X^T[d, streamed] ds[streamed, resident], with X^T read from
// the same LDS tile through ds_read_b64_tr_b16.  Streamed tiles (64 rows) go HBM -> LDS directly
// (global_load_lds, 16 B per lane), three stages deep, with the pair swizzle of the forward kernels' V tile plus a flip of the two halves of
// a pair (see ae_bwd_chunk_pos): one layout serves the row reads and the transposed reads.
//
// Masks: mode 0 none; mode 1 analytic causal (tiles beyond the diagonal never visited); mode 2 two
// tile-class tables built on the host from mask_mod (0 skip, 1 test per element, 2 fully visible), one
// per launch because the two tile shapes differ: [q tiles of 32*AE_BWD_NWAVES][kv tiles of 64] for dq,
// [q tiles of 64][kv tiles of 128] for dk/dv (role of blockattn_tl.py's block mask in the backward).
// AE_EXT_BLOCK_MASK 1: the forward ran on a block mask the user supplied (blockattn_tl.py:195-470 is the
// reference's backward for it); the two tables are then made from that mask, and a tile of class 1 - one that
// straddles blocks of both kinds - looks every element up in the user's mask (ae_attn_bwd_params.block_mask).
//
// Waves per workgroup (AE_BWD_NWAVES, 32 resident rows each): dk/dv runs four, one per SIMD with the
// whole register file (two accumulators). dq has one accumulator and fits 256 registers, so it runs
// eight, two per SIMD (AE_BWD_WAVES_PER_EU 2, AE_AHEAD 2): a wave spends about half of its time waiting
// (LDS fragments, MFMA results, the p/ds arithmetic between two sets of MFMAs) and the second wave
// fills it - 0.59 -> 0.44 ms for B2 H32 S4096 D128 causal.
//
// AE_BWD_KIND 2: online functions with one final row scale of their own (retention): p and ds come from the
// generated ae_bwd_pd2, which holds the traced OnlineFunc.forward / OnlineFunc.backward
// (attention_engine/core/lower/lower.py:413-453 of the reference), the symbolic derivative of score_mod and
// the reads of its custom inputs (per score where they have a kv dimension); the `lse` argument carries
// that row scale.
// AE_BWD_KIND 1: graphs whose online function does nothing, out = sum_kv f(s) v with f = score_mod (sigmoid
// and relu attention, attn_script/sigmoidattn.py, reluattn.py): p = f(s), ds = dp * f'(s), both from the
// generated ae_bwd_pd (f' by symbolic differentiation of the traced score_mod); no row scales, scale 1.
//
// Configuration ("ae_config.h"): AE_D AE_DV AE_DTYPE_BF16 AE_MASK_MODE (0, 1, 2) AE_HAS_MASK_MOD
// AE_SM_SCALE AE_BWD_ROLE AE_BWD_KIND, optional AE_BWD_NWAVES (4 or 8) AE_BWD_WAVES_PER_EU AE_AHEAD AE_BWD_NRS (kind 2:
// final row scales of the online function, 1 .. AE_MAX_ROWSCALES).  Functors used ("ae_functors.h"): ae_mask_mod; kind 1: ae_bwd_pd,
// ae_bwd_load_custom; kind 2: ae_bwd_pd2.

#include "ae_hip.h"
#include "ae_config.h"
#include "ae_device.h"
#include "ae_functors.h"
#ifndef AE_HEAVY_LAST
#define AE_HEAVY_LAST 0
#endif
#ifndef AE_EXT_BLOCK_MASK
#define AE_EXT_BLOCK_MASK 0
#endif

#ifndef AE_BWD_NWAVES
#define AE_BWD_NWAVES 4             // waves per workgroup, 32 resident rows each
#endif
#define AE_NWAVES AE_BWD_NWAVES
#define AE_NT (AE_NWAVES * 64)
#define AE_BR (AE_NWAVES * 32)     // resident rows per workgroup
#define AE_BS 64                   // streamed rows per tile
#define AE_STR1 (AE_D * 2)         // LDS row pitch of the first streamed tensor (K or Q), bytes
#define AE_STR2 (AE_DV * 2)        // ... of the second (V or dO)
#define AE_CPR1 (AE_D / 8)         // 16-byte chunks per row
#define AE_CPR2 (AE_DV / 8)
#define AE_T1_BYTES (AE_BS * AE_STR1)
#define AE_T2_BYTES (AE_BS * AE_STR2)
// per-row values that travel with a streamed tile of the dk / dv launch: rowsum(do*o), and lse - or, kind 2, the
// AE_BWD_NRS final row scales of the online function (planes of the work buffer `delta`: 0 = rowsum(do*o), 1 + i =
// row scale i).  In LDS, behind the tile: row scale 0 first, rowsum(do*o) second, further row scales after them.
#ifndef AE_BWD_NRS
#define AE_BWD_NRS 1
#endif
#define AE_RS_PLANES (1 + AE_BWD_NRS)
#define AE_RS_SLOT(plane) ((plane) == 0 ? 1 : ((plane) == 1 ? 0 : (plane)))
#define AE_STAGE_BYTES (AE_T1_BYTES + AE_T2_BYTES + AE_RS_PLANES * AE_BS * 4)
#define AE_NKS1 (AE_D / 16)        // k-steps of S
#define AE_NKS2 (AE_DV / 16)       // k-steps of dP
#define AE_NDB1 (AE_D / 32)        // 32-wide output blocks of dQ / dK
#define AE_NDB2 (AE_DV / 32)       // ... of dV
#define AE_L1 ((AE_BS * AE_CPR1) / AE_NT)   // 1 KiB load instructions per wave and tile
#define AE_L2 ((AE_BS * AE_CPR2) / AE_NT)
#ifndef AE_NSTAGE
#define AE_NSTAGE 3                // LDS stages: a tile is requested AE_NSTAGE - 1 iterations before it is multiplied
#endif
#ifndef AE_BWD_WAVES_PER_EU
#define AE_BWD_WAVES_PER_EU 1
#endif
#define AE_RSL ((AE_RS_PLANES + AE_NWAVES - 1) / AE_NWAVES)      // row-value loads per wave and tile (dk / dv launch)
#define AE_NLOADS (AE_L1 + AE_L2 + (AE_BWD_ROLE == 1 ? AE_RSL : 0))   // load instructions per wave and tile
#define AE_VMCNT(n) (0x0F70 | ((n) & 15) | (((n) >> 4) << 14))
#ifndef AE_AHEAD
#define AE_AHEAD 4                 // LDS fragments in flight ahead of the MFMA that uses them
#endif
#define AE_RING (AE_AHEAD + 1)

static_assert(AE_D == 64 || AE_D == 128, "head dim 64 or 128");
static_assert(AE_DV == 64 || AE_DV == 128, "value head dim 64 or 128");
static_assert(AE_BWD_ROLE == 0 || AE_BWD_ROLE == 1, "role");
#ifndef AE_BWD_KIND
#define AE_BWD_KIND 0
#endif
// 1: at the top of every tile the output accumulators are named as accumulator-file values (an empty asm).
// Launches with one wave per SIMD use both register files; without the hint the register allocator keeps a
// quarter of the output accumulators in ordinary registers and moves them in and out around the p / ds
// arithmetic: 64 moves per tile.
#ifndef AE_BWD_PIN_ACC
#define AE_BWD_PIN_ACC (AE_BWD_WAVES_PER_EU == 1)
#endif
static_assert(AE_MASK_MODE >= 0 && AE_MASK_MODE <= 2, "none, causal, or tile-class tables");

typedef __attribute__((address_space(3))) unsigned char ae_lds_byte;
typedef __attribute__((address_space(3))) float ae_lds_f32;
struct ae_bwd_true { static constexpr bool value = true; };
struct ae_bwd_false { static constexpr bool value = false; };

// LDS position of 16-byte chunk c of row r: the 32-byte pairs of a row are exchanged by the row's low
// bits (transposed reads of a column group then spread over the banks), and the two chunks of a pair by
// the next row bit (so do the row reads of 16 consecutive rows, which all ask for the same chunk).
template <int CPR>
AE_DEV int ae_bwd_half_flip(int r) { return (r >> (CPR == 16 ? 3 : 2)) & 1; }
template <int CPR>
AE_DEV int ae_bwd_chunk_pos(int r, int c) {
  return ((((c >> 1) ^ (r & (CPR / 2 - 1))) << 1) | ((c ^ ae_bwd_half_flip<CPR>(r)) & 1));
}

// Resident rows on their way in and results on their way out pass through LDS as whole rows (16 lanes per
// 256-byte row), as in the forward kernels: a lane that fetches its own row's fragments, or stores its own row's
// results, touches 32 rows per instruction, 16 bytes of each, and the workgroups of a launch, which start and end
// together, queue behind each other's requests.  The resident rows use stages 1 and 2 of the tile ring before the
// loop starts (the second item is requested once every wave has its fragments), both tensors at once where they
// fit, else one after the other; the results use the ring after the last item.
#define AE_R1B (32 * AE_STR1)      // bytes of a wave's resident rows, first tensor
#define AE_R2B (32 * AE_STR2)
#define AE_RES_ONEPASS (AE_NWAVES * (AE_R1B + AE_R2B) <= 2 * AE_STAGE_BYTES)
#define AE_RES_TWOPASS (AE_NWAVES * (AE_R1B > AE_R2B ? AE_R1B : AE_R2B) <= 2 * AE_STAGE_BYTES)
#define AE_RES_VIA_LDS (AE_NSTAGE == 3 && (AE_RES_ONEPASS || AE_RES_TWOPASS))
#define AE_OUT_BYTES (AE_R1B + (AE_BWD_ROLE == 1 ? AE_R2B : 0))   // a wave's results
#define AE_OUT_VIA_LDS (AE_NWAVES * AE_OUT_BYTES <= AE_NSTAGE * AE_STAGE_BYTES)
// 1 (softmax attention, set by the host with both launches): there is no ae_bwd_delta_kernel launch.  The dq
// launch, which holds the dO rows anyway, fetches its O rows behind them, forms rowsum(dO * O) and writes both
// planes of the work buffer; the dk/dv launch runs after it.  (The separate launch read O and dO once more:
// 28 us and 138 MB of the C2 causal backward.)
#ifndef AE_BWD_FUSE_DELTA
#define AE_BWD_FUSE_DELTA 0
#endif
static_assert(!AE_BWD_FUSE_DELTA || (AE_RES_VIA_LDS && AE_BWD_KIND == 0), "the fused row sums need the staged resident rows");

// 32 rows of CPR 16-byte chunks, HBM -> dst, one burst; LDS chunk c' of row r holds global chunk c' ^ (r mod CPR).
// g: the wave's first row (clamped into the tensor), 4 KiB low (see ae_load_lds16_burst_base); row0: first row
// of the wave relative to it; rows past `last` re-read it.
template <int CPR>
AE_DEV void ae_bwd_rows_to_lds(const char* g, ae_lds_byte* dst, int lane, int row0, int last, int stride) {
  constexpr int N = CPR / 2;
  unsigned off[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int n = (i < N ? i : 0) * 64 + lane;
    const int row = n / CPR;
    const int c = (n % CPR) ^ (row & (CPR - 1));
    int ra = row0 + row;
    ra = ra < last ? ra : last;
    off[i] = (unsigned)((ra * stride + c * 8) * 2 + 4096 - (i - N / 2) * 1024);
  }
  ae_load_lds16_burst_base<N>(g, off, dst + (N / 2) * 1024);
}
// B-operand fragments of row l32 (k = 16*ks + 8*hf + j) from rows laid out by ae_bwd_rows_to_lds
template <int NKS, int CPR>
AE_DEV void ae_bwd_frags_from_lds(ae_elem8* rf, const ae_lds_byte* src, int l32, int hf) {
#pragma unroll
  for (int ks = 0; ks < NKS; ks++)
    rf[ks] = *(const __attribute__((address_space(3))) ae_elem8*)(
        src + l32 * (CPR * 16) + (((2 * ks + hf) ^ (l32 & (CPR - 1))) << 4));
}

#if AE_BWD_ROLE == 0
#define AE_BWD_KERNEL ae_bwd_dq_kernel
#else
#define AE_BWD_KERNEL ae_bwd_dkv_kernel
#endif

static_assert(AE_NSTAGE == 2 || AE_NSTAGE == 3, "two or three stages");
extern "C" __global__ __launch_bounds__(AE_NT) __attribute__((amdgpu_waves_per_eu(AE_BWD_WAVES_PER_EU, AE_BWD_WAVES_PER_EU)))
void AE_BWD_KERNEL(const ae_attn_bwd_params p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ae_smem[];
  ae_lds_byte* lds = (ae_lds_byte*)ae_smem;   // AE_NSTAGE stages of [tile 1][tile 2][lse][delta]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hf = lane >> 5;
  const int group = p.heads_q / p.heads_kv;

  // ---- which (resident tile, head, batch) --------------------------------------------------------
#if AE_BWD_ROLE == 0
  const int n_res = p.seqlen_q, n_str = p.seqlen_kv, heads = p.heads_q;
#else
  const int n_res = p.seqlen_kv, n_str = p.seqlen_q, heads = p.heads_kv;
#endif
  // ids are dealt round-robin to the 8 XCDs (each with its own L2): id = 8*slot + xcd keeps all resident
  // tiles of one (batch, head) on ONE XCD, where they share the streamed tiles, and the slots go tile by
  // tile across the heads, under a causal mask the tile with the most work first (the last q rows for
  // dq, the first kv rows for dk/dv).  The grid is padded to 8*ceil(batch*heads/8)*tiles ids.
  const int n_rt = (n_res + AE_BR - 1) / AE_BR;
  const int n_bh = p.batch * heads;
  const int n_bg = (n_bh + 7) >> 3;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int bh = (slot % n_bg) * 8 + xcd;
#if AE_BWD_ROLE == 0 && (AE_MASK_MODE == 1 || (AE_MASK_MODE == 2 && AE_HEAVY_LAST))
  // (the q tiles with the most visible keys first: the last ones under a causal mask, and under a tile table
  // that the host found to be heavier towards the end - AE_HEAVY_LAST)
  const int rt = n_rt - 1 - slot / n_bg;
#else
  const int rt = slot / n_bg;
#endif
  if (bh >= n_bh) return;
  const int h = bh % heads;            // role 0: q head; role 1: kv head
  const int b = bh / heads;
  const int r0 = rt * AE_BR;
  const int rrow = r0 + wave * 32 + l32;            // this lane's resident row
  const bool r_ok = rrow < n_res;
  const int rrow_c = r_ok ? rrow : n_res - 1;

  // ---- resident operands: B[k = 16*ks + 8*hf + j][n = row] ---------------------------------------
#if AE_BWD_ROLE == 0
  const int hk = h / group;
  const ae_elem* r1p = (const ae_elem*)p.q + (int64_t)b * p.q_stride_b + (int64_t)rrow_c * p.q_stride_s + (int64_t)h * p.q_stride_h;
  const ae_elem* r2p = (const ae_elem*)p.dout + (int64_t)b * p.do_stride_b + (int64_t)rrow_c * p.do_stride_s + (int64_t)h * p.do_stride_h;
#else
  const int hk = h;
  const ae_elem* r1p = (const ae_elem*)p.k + (int64_t)b * p.k_stride_b + (int64_t)rrow_c * p.k_stride_s + (int64_t)h * p.k_stride_h;
  const ae_elem* r2p = (const ae_elem*)p.v + (int64_t)b * p.v_stride_b + (int64_t)rrow_c * p.v_stride_s + (int64_t)h * p.v_stride_h;
#endif
#if AE_BWD_KIND == 1
  ae_custom cust;
  ae_bwd_load_custom(cust, p);
#endif
  ae_elem8 rf1[AE_NKS1], rf2[AE_NKS2];
#if !AE_RES_VIA_LDS
#pragma unroll
  for (int ks = 0; ks < AE_NKS1; ks++) rf1[ks] = *(const ae_elem8*)(r1p + ks * 16 + hf * 8);
#pragma unroll
  for (int ks = 0; ks < AE_NKS2; ks++) rf2[ks] = *(const ae_elem8*)(r2p + ks * 16 + hf * 8);
#else
  (void)r1p, (void)r2p;
#endif

#if AE_BWD_ROLE == 0
  // row scales of the lane's q row: lse in log2 units (+inf for a row without a visible key: p = 0)
  float lse2_r, delta_r;
#if AE_BWD_KIND == 2 && AE_BWD_NRS > 1
  float rs_more[AE_BWD_NRS - 1];      // the online function's further final row scales of the lane's row
#endif
  {
    const int64_t ri = ((int64_t)b * p.heads_q + h) * p.seqlen_q + rrow_c;
#if AE_BWD_FUSE_DELTA
    const float l = p.lse[ri];
    lse2_r = (l == AE_NEG_INF) ? __builtin_inff() : l * AE_LOG2E;     // +inf: a row without a visible key, p = 0
    delta_r = 0.f;                                                    // formed below, once dO and O are here
#else
    delta_r = p.delta[ri];
    lse2_r = p.delta[(int64_t)p.batch * p.heads_q * p.seqlen_q + ri];
#endif
#if AE_BWD_KIND == 2 && AE_BWD_NRS > 1
#pragma unroll
    for (int i = 1; i < AE_BWD_NRS; i++) rs_more[i - 1] = p.delta[(int64_t)(1 + i) * p.batch * p.heads_q * p.seqlen_q + ri];
#endif
  }
#endif
#if !AE_RES_VIA_LDS
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the resident operands are in registers before any tile request
#endif

  // ---- the streamed items --------------------------------------------------------------------------
  // role 0: kv tiles 0 .. (causal: up to the diagonal); role 1: for every q head of the group, q tiles
  // (causal: from the diagonal) .. last
  const int n_st = (n_str + AE_BS - 1) / AE_BS;
  int t_lo = 0, t_hi = n_st;
#if AE_MASK_MODE == 1
#if AE_BWD_ROLE == 0
  {
    const int lim = (r0 + AE_BR - 1) / AE_BS + 1;
    t_hi = lim < n_st ? lim : n_st;
  }
#else
  t_lo = r0 / AE_BS;
  t_lo = t_lo < n_st ? t_lo : n_st;
#endif
#endif
  const int n_t = t_hi - t_lo;
  // item x: tile t_lo + x % n_t of q head x / n_t of the group (role 0: one head)
#if AE_BWD_ROLE == 0
  const int n_items = n_t;
#else
  const int n_items = n_t * group;
#endif
  auto item_tile = [&](int x) AE_LAMBDA { return t_lo + (AE_BWD_ROLE == 0 ? x : x % n_t); };
  auto item_head = [&](int x) AE_LAMBDA { return AE_BWD_ROLE == 0 ? h : h * group + x / n_t; };   // q head of the item
#if AE_MASK_MODE == 2
  // Classes of the items from the tile table of this launch (0 = nothing visible, 1 = test every element,
  // 2 = all visible), 64 items at a time: lane l reads the class of item c0 + l and two ballots keep "visible"
  // and "fully visible" as 64-bit masks in scalar registers.  Reading the table item by item inside the loop
  // would cost a dependent memory access per skipped item, and, behind the tile requests' asm statements, a
  // vector load whose wait (vmcnt(0)) also waits for every tile in flight.
  int im_c0 = -64;
  unsigned long im_vis = 0, im_full = 0;
  auto item_masks = [&](int c0) AE_LAMBDA {
    const int x = c0 + lane;
    int c = 0;
    if (x < n_items) {
      const int hq = item_head(x), t = item_tile(x);
      const int64_t mbh = (int64_t)(p.mask_b == 1 ? 0 : b) * p.mask_h + (p.mask_h == 1 ? 0 : hq);
#if AE_BWD_ROLE == 0
      c = p.mask_dq[(mbh * n_rt + rt) * n_st + t];            // [q tiles of 128][kv tiles of 64]
#else
      c = p.mask_dkv[(mbh * n_st + t) * n_rt + rt];           // [q tiles of 64][kv tiles of 128]
#endif
    }
    im_vis = __builtin_amdgcn_ballot_w64(c != 0);
    im_full = __builtin_amdgcn_ballot_w64(c == 2);
    im_c0 = c0;
  };
#endif
  // first item at or after x that has anything visible (n_items if none), and its class
  auto next_item = [&](int x, int& cls) AE_LAMBDA {
    cls = 2;
#if AE_MASK_MODE == 2
    while (x < n_items) {
      if (x < im_c0 || x >= im_c0 + 64) item_masks(x & ~63);
      const unsigned long m = im_vis >> (x - im_c0);
      if (m != 0) {
        x += __builtin_ctzl(m);
        cls = ((im_full >> (x - im_c0)) & 1ul) ? 2 : 1;
        break;
      }
      x = im_c0 + 64;
    }
#endif
    return x < n_items ? x : n_items;
  };

  // Direct HBM -> LDS tile requests.  Wave w fills the 1 KiB blocks w*L .. w*L+L-1 of each tile; a lane's
  // 16 bytes land at block*1024 + lane*16, i.e. at chunk position cp of row r, so it fetches the global
  // chunk that belongs there (the swizzle is its own inverse).  A tile's loads of one tensor go out as
  // one burst behind a single write of M0 (wave-uniform base + per-lane offset + immediate, see
  // ae_load_lds16_burst_base: bases are passed 4 KiB low and offsets 4 KiB high).  Rows past the end of
  // the sequence re-read its last row (they are masked).
  auto lane_off1 = [&](int i, int last_row, int64_t st) AE_LAMBDA -> unsigned {
    const int sidx = (wave * AE_L1 + i) * 64 + lane;
    int r = sidx / AE_CPR1;
    const int c = ae_bwd_chunk_pos<AE_CPR1>(r, sidx % AE_CPR1);
    r = r < last_row ? r : last_row;
    return (unsigned)((r * (int)st + c * 8) * 2 + 4096 - (i - AE_L1 / 2) * 1024);
  };
  auto lane_off2 = [&](int i, int last_row, int64_t st) AE_LAMBDA -> unsigned {
    const int sidx = (wave * AE_L2 + i) * 64 + lane;
    int r = sidx / AE_CPR2;
    const int c = ae_bwd_chunk_pos<AE_CPR2>(r, sidx % AE_CPR2);
    r = r < last_row ? r : last_row;
    return (unsigned)((r * (int)st + c * 8) * 2 + 4096 - (i - AE_L2 / 2) * 1024);
  };
#if AE_BWD_ROLE == 0
  const int64_t st1 = p.k_stride_s, st2 = p.v_stride_s;
#else
  const int64_t st1 = p.q_stride_s, st2 = p.do_stride_s;
#endif
  unsigned off1[AE_L1], off2[AE_L2];
#pragma unroll
  for (int i = 0; i < AE_L1; i++) off1[i] = lane_off1(i, AE_BS, st1);
#pragma unroll
  for (int i = 0; i < AE_L2; i++) off2[i] = lane_off2(i, AE_BS, st2);
  // request item x (past the end: the last item again, so that every call issues AE_NLOADS loads) into `stage`
  auto request_item = [&](int x, int stage) AE_LAMBDA {
    const int itc = x < n_items ? x : n_items - 1;
    const int s0 = item_tile(itc) * AE_BS;
    ae_lds_byte* t1 = lds + stage * AE_STAGE_BYTES;
    ae_lds_byte* t2 = t1 + AE_T1_BYTES;
#if AE_BWD_ROLE == 0
    const char* x1 = (const char*)((const ae_elem*)p.k + (int64_t)b * p.k_stride_b + (int64_t)hk * p.k_stride_h + (int64_t)s0 * st1);
    const char* x2 = (const char*)((const ae_elem*)p.v + (int64_t)b * p.v_stride_b + (int64_t)hk * p.v_stride_h + (int64_t)s0 * st2);
#else
    const int hq = item_head(itc);
    const char* x1 = (const char*)((const ae_elem*)p.q + (int64_t)b * p.q_stride_b + (int64_t)hq * p.q_stride_h + (int64_t)s0 * st1);
    const char* x2 = (const char*)((const ae_elem*)p.dout + (int64_t)b * p.do_stride_b + (int64_t)hq * p.do_stride_h + (int64_t)s0 * st2);
#endif
    unsigned g1[8], g2[8];
    const bool ragged = s0 + AE_BS > n_str;           // wave-uniform
#pragma unroll
    for (int i = 0; i < 8; i++) {
      g1[i] = off1[i < AE_L1 ? i : 0];
      g2[i] = off2[i < AE_L2 ? i : 0];
    }
    if (__builtin_expect(ragged, 0)) {
      asm volatile("" ::: "memory");                   // (keeps this one branch, out of the common path)
#pragma unroll
      for (int i = 0; i < 8; i++) {
        g1[i] = lane_off1(i < AE_L1 ? i : 0, n_str - 1 - s0, st1);
        g2[i] = lane_off2(i < AE_L2 ? i : 0, n_str - 1 - s0, st2);
      }
    }
    ae_load_lds16_burst_base<AE_L1>(x1 - 4096, g1, t1 + (wave * AE_L1 + AE_L1 / 2) * 1024);
    ae_load_lds16_burst_base<AE_L2>(x2 - 4096, g2, t2 + (wave * AE_L2 + AE_L2 / 2) * 1024);
#if AE_BWD_ROLE == 1
    {
      // rowsum(do * o) and lse in log2 units (kind 2: the final row scales) of the tile's 64 q rows: the waves share
      // the planes out, every wave issuing the same number of loads (planes are fetched more than once where there
      // are fewer of them than waves)
      int row = s0 + lane;
      row = row < n_str ? row : n_str - 1;
#pragma unroll
      for (int i = 0; i < AE_RSL; i++) {
        const int plane = (wave + AE_NWAVES * i) % AE_RS_PLANES;
        const float* src = p.delta + ((int64_t)plane * p.batch * p.heads_q + (int64_t)b * p.heads_q + hq) * p.seqlen_q + row;
        ae_load_lds4(src, t2 + AE_T2_BYTES + AE_RS_SLOT(plane) * AE_BS * 4);
      }
    }
#endif
  };

  // A operands out of a staged tile.  Row fragment: A[m = row 32*nb + lane%32][k = 16*ks + 8*hf + j].
  auto row_frag1 = [&](const ae_lds_byte* t, int nb, int ks) AE_LAMBDA -> ae_elem8 {
    const int r = nb * 32 + l32;
    return *(const __attribute__((address_space(3))) ae_elem8*)(t + r * AE_STR1 + ae_bwd_chunk_pos<AE_CPR1>(r, 2 * ks + hf) * 16);
  };
  auto row_frag2 = [&](const ae_lds_byte* t, int nb, int ks) AE_LAMBDA -> ae_elem8 {
    const int r = nb * 32 + l32;
    return *(const __attribute__((address_space(3))) ae_elem8*)(t + r * AE_STR2 + ae_bwd_chunk_pos<AE_CPR2>(r, 2 * ks + hf) * 16);
  };
  // Transposed fragment: A[m = column 32*db + ..][k = the 16 rows of k-step kk], in the row order in which
  // a lane's accumulator registers hold the rows (see the forward kernels' V^T fragment).
  const int t_row = 4 * hf + ((lane & 15) >> 2);
  const int t_g = l32 >> 4;
  auto tr_frag = [&](const ae_lds_byte* t, int str, int cpr, int kk, int db) AE_LAMBDA -> ae_elem8 {
    const int rb0 = (kk >> 1) * 32 + (kk & 1) * 16;
    const int r_lo = rb0 + t_row, r_hi = r_lo + 8;
    const int sh = cpr == 16 ? 3 : 2;
    const int pair = ((2 * db + t_g) ^ (t_row & (cpr / 2 - 1))) << 5;
    const ae_lds_byte* a_lo = t + r_lo * str + pair + (((lane & 3) * 8) ^ (((r_lo >> sh) & 1) * 16));
    const ae_lds_byte* a_hi = t + r_hi * str + pair + (((lane & 3) * 8) ^ (((r_hi >> sh) & 1) * 16));
    ae_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) ae_s16x4*)a_lo);
    ae_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) ae_s16x4*)a_hi);
    return __builtin_bit_cast(ae_elem8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  ae_f32x16 acc1[AE_NDB1];            // dQ^T (role 0) / dK^T (role 1): [d][resident row]
#pragma unroll
  for (int db = 0; db < AE_NDB1; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc1[db][r] = 0.f;
#if AE_BWD_ROLE == 1
  ae_f32x16 acc2[AE_NDB2];            // dV^T
#pragma unroll
  for (int db = 0; db < AE_NDB2; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc2[db][r] = 0.f;
#endif

  // the n-th visited item is multiplied out of stage n % NSTAGE while the next two are on their way
  int cls0, cls1, cls2;                 // ... and the classes of those three items
  int x0 = next_item(0, cls0), x1 = next_item(x0 + 1, cls1), x2 = next_item(x1 + 1, cls2);
#if AE_RES_VIA_LDS
  if (x0 < n_items) request_item(x0, 0);
  {
    // the wave's 32 resident rows of both tensors travel together with the first item
    const int rw0 = r0 + wave * 32;
    const int rw0c = rw0 < n_res ? rw0 : n_res - 1;
#if AE_BWD_ROLE == 0
    const char* g1 = (const char*)((const ae_elem*)p.q + (int64_t)b * p.q_stride_b + (int64_t)rw0c * p.q_stride_s + (int64_t)h * p.q_stride_h);
    const char* g2 = (const char*)((const ae_elem*)p.dout + (int64_t)b * p.do_stride_b + (int64_t)rw0c * p.do_stride_s + (int64_t)h * p.do_stride_h);
    const int rs1 = (int)p.q_stride_s, rs2 = (int)p.do_stride_s;
#else
    const char* g1 = (const char*)((const ae_elem*)p.k + (int64_t)b * p.k_stride_b + (int64_t)rw0c * p.k_stride_s + (int64_t)h * p.k_stride_h);
    const char* g2 = (const char*)((const ae_elem*)p.v + (int64_t)b * p.v_stride_b + (int64_t)rw0c * p.v_stride_s + (int64_t)h * p.v_stride_h);
    const int rs1 = (int)p.k_stride_s, rs2 = (int)p.v_stride_s;
#endif
#if AE_RES_ONEPASS
    ae_lds_byte* rs = lds + AE_STAGE_BYTES + wave * (AE_R1B + AE_R2B);
    ae_bwd_rows_to_lds<AE_CPR1>(g1 - 4096, rs, lane, rw0 - rw0c, n_res - 1 - rw0c, rs1);
    ae_bwd_rows_to_lds<AE_CPR2>(g2 - 4096, rs + AE_R1B, lane, rw0 - rw0c, n_res - 1 - rw0c, rs2);
    __builtin_amdgcn_s_waitcnt(AE_VMCNT(0));
    ae_bwd_frags_from_lds<AE_NKS1, AE_CPR1>(rf1, rs, l32, hf);
    ae_bwd_frags_from_lds<AE_NKS2, AE_CPR2>(rf2, rs + AE_R1B, l32, hf);
#else
    ae_lds_byte* rs = lds + AE_STAGE_BYTES + wave * (AE_R1B > AE_R2B ? AE_R1B : AE_R2B);
    ae_bwd_rows_to_lds<AE_CPR1>(g1 - 4096, rs, lane, rw0 - rw0c, n_res - 1 - rw0c, rs1);
    __builtin_amdgcn_s_waitcnt(AE_VMCNT(0));
    ae_bwd_frags_from_lds<AE_NKS1, AE_CPR1>(rf1, rs, l32, hf);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     // the fragments are out before the rows are replaced
    ae_bwd_rows_to_lds<AE_CPR2>(g2 - 4096, rs, lane, rw0 - rw0c, n_res - 1 - rw0c, rs2);
    __builtin_amdgcn_s_waitcnt(AE_VMCNT(0));
    ae_bwd_frags_from_lds<AE_NKS2, AE_CPR2>(rf2, rs, l32, hf);
#endif
#if AE_BWD_ROLE == 0 && AE_BWD_FUSE_DELTA
    {
      // rowsum(dO * O) of the lane's row: the O rows follow the dO rows through the staging region, are read in
      // the same fragment layout, and the two lanes that share a row add their halves
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      const char* g3 = (const char*)((const ae_elem*)p.out + (int64_t)b * p.o_stride_b + (int64_t)rw0c * p.o_stride_s + (int64_t)h * p.o_stride_h);
      ae_bwd_rows_to_lds<AE_CPR2>(g3 - 4096, rs, lane, rw0 - rw0c, n_res - 1 - rw0c, (int)p.o_stride_s);
      __builtin_amdgcn_s_waitcnt(AE_VMCNT(0));
      ae_elem8 of[AE_NKS2];
      ae_bwd_frags_from_lds<AE_NKS2, AE_CPR2>(of, rs, l32, hf);
      float acc = 0.f;
#pragma unroll
      for (int ks = 0; ks < AE_NKS2; ks++)
#pragma unroll
        for (int j = 0; j < 8; j++) acc += (float)of[ks][j] * (float)rf2[ks][j];
      delta_r = acc + __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, acc)));
      if (r_ok && hf == 0) {
        const int64_t ri = ((int64_t)b * p.heads_q + h) * p.seqlen_q + rrow;
        p.delta[ri] = delta_r;
        p.delta[(int64_t)p.batch * p.heads_q * p.seqlen_q + ri] = lse2_r;
      }
    }
#endif
#if AE_BWD_ROLE == 0
    // (the row scales were loaded as ordinary loads: used here, their wait falls before the loop and not into it)
    asm volatile("" :: "v"(lse2_r), "v"(delta_r));
#endif
  }
  __syncthreads();       // every wave has its fragments: stages 1 and 2 go back to the ring
  if (x0 < n_items) request_item(x1, 1);
#else
  if (x0 < n_items) {
    request_item(x0, 0);
    if (AE_NSTAGE == 3) request_item(x1, 1);
    __builtin_amdgcn_s_waitcnt(AE_VMCNT((AE_NSTAGE - 2) * AE_NLOADS));   // the first item has landed
  }
  __syncthreads();
#endif

  for (int n = 0; x0 < n_items; n++) {
    const int it = x0;
    // into the stage everyone left at the last barrier
    request_item(AE_NSTAGE == 3 ? x2 : x1, (n + AE_NSTAGE - 1) % AE_NSTAGE);
    const ae_lds_byte* t1 = lds + (n % AE_NSTAGE) * AE_STAGE_BYTES;
    const ae_lds_byte* t2 = t1 + AE_T1_BYTES;
    const int s0 = item_tile(it) * AE_BS;
#if AE_BWD_PIN_ACC
#pragma unroll
    for (int db = 0; db < AE_NDB1; db++) asm volatile("" : "+a"(acc1[db]));
#if AE_BWD_ROLE == 1
#pragma unroll
    for (int db = 0; db < AE_NDB2; db++) asm volatile("" : "+a"(acc2[db]));
#endif
#endif

    // S = X1 R1^T and dP = X2 R2^T, [streamed row][resident row], one 32-row block of the tile at a
    // time; p and ds are packed as B operands: k-step kk holds the lane's elements 8*kk .. 8*kk+7
    ae_u32x4 pf[4], dsf[4];       // as packed pairs: two scores are converted by ONE packed conversion
#if AE_BWD_ROLE == 1
    const ae_lds_f32* rs_l = (const ae_lds_f32*)(t2 + AE_T2_BYTES);
    const int hq = item_head(it);
#else
    const int hq = h;
#endif
    (void)hq;
    // only tiles that touch the diagonal, the end of a sequence or an elementwise mask test visibility
    const int r0w = r0 + wave * 32;
#if AE_MASK_MODE == 2
    bool need_vis = cls0 != 2 || s0 + AE_BS > n_str || r0w + 32 > n_res;
#else
    bool need_vis = (AE_HAS_MASK_MOD != 0) || (AE_EXT_BLOCK_MASK != 0) || s0 + AE_BS > n_str || r0w + 32 > n_res;
#endif
#if AE_MASK_MODE == 1
    need_vis = need_vis || (AE_BWD_ROLE == 0 ? s0 + AE_BS - 1 > r0w : s0 < r0w + 31);
#endif
    auto block = [&](int nb, auto masked) AE_LAMBDA {
      ae_f32x16 sacc, pacc;
#pragma unroll
      for (int r = 0; r < 16; r++) sacc[r] = pacc[r] = 0.f;
      // fragment stream of the block: S and dP k-steps alternate (two independent accumulation chains);
      // fragments are read AE_AHEAD MFMAs ahead of their use into a small ring, one fence per MFMA (left to
      // itself the scheduler either exposes the LDS latency or hoists every read and spills)
      constexpr int NF = AE_NKS1 + AE_NKS2;
      auto frag = [&](int f) AE_LAMBDA -> ae_elem8 {
        // f even and S still has k-steps: S; else dP (the dims may differ)
        const int pairs = AE_NKS1 < AE_NKS2 ? AE_NKS1 : AE_NKS2;
        if (f < 2 * pairs) return (f & 1) ? row_frag2(t2, nb, f >> 1) : row_frag1(t1, nb, f >> 1);
        return AE_NKS1 > AE_NKS2 ? row_frag1(t1, nb, f - pairs) : row_frag2(t2, nb, f - pairs);
      };
      ae_elem8 ring[AE_RING];
#pragma unroll
      for (int f = 0; f < AE_AHEAD && f < NF; f++) ring[f] = frag(f);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int f = 0; f < NF; f++) {
        if (f + AE_AHEAD < NF) ring[(f + AE_AHEAD) % AE_RING] = frag(f + AE_AHEAD);
        const int pairs = AE_NKS1 < AE_NKS2 ? AE_NKS1 : AE_NKS2;
        const bool is_s = f < 2 * pairs ? !(f & 1) : AE_NKS1 > AE_NKS2;
        const int ks = f < 2 * pairs ? f >> 1 : f - pairs;
        if (is_s) sacc = ae_mfma32(ring[f % AE_RING], rf1[ks], sacc);
        else pacc = ae_mfma32(ring[f % AE_RING], rf2[ks], pacc);
        __builtin_amdgcn_sched_barrier(0);
      }
      float pvs[16], dss[16];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int sl = nb * 32 + 8 * (r >> 2) + 4 * hf + (r & 3);     // streamed row inside the tile
        const int srow = s0 + sl;
#if AE_BWD_ROLE == 0
        const int qi = rrow, ki = srow;
        const float l2 = lse2_r, dl = delta_r;
#else
        const int qi = srow, ki = rrow;
        const float l2 = rs_l[sl], dl = rs_l[AE_BS + sl];
#endif
#if AE_BWD_KIND == 0
        float pv = ae_exp2(__builtin_fmaf(sacc[r], AE_SM_SCALE * AE_LOG2E, -l2));
        const float dfac = pacc[r] - dl;
#elif AE_BWD_KIND == 1
        float pv, dfac;
        ae_bwd_pd(sacc[r], (float)b, (float)hq, (float)qi, (float)ki, cust, pv, dfac);
        dfac *= pacc[r];
        (void)l2; (void)dl;
#else
        // traced OnlineFunc.forward / backward: l2 is the row's (first) final row scale as the forward wrote it
        float pv, dfac;
        float rsv[AE_BWD_NRS];
        rsv[0] = l2;
#if AE_BWD_NRS > 1
#pragma unroll
        for (int i = 1; i < AE_BWD_NRS; i++)
#if AE_BWD_ROLE == 0
          rsv[i] = rs_more[i - 1];
#else
          rsv[i] = rs_l[(1 + i) * AE_BS + sl];
#endif
#endif
        ae_bwd_pd2(sacc[r], pacc[r], rsv, dl, b, hq, qi, ki, p, pv, dfac);
#endif
        bool vis = true;
        if (decltype(masked)::value) {
          vis = r_ok && srow < n_str;
#if AE_MASK_MODE == 1
          vis = vis && qi >= ki;
#endif
#if AE_HAS_MASK_MOD
          vis = vis && ae_mask_mod(b, hq, qi, ki);
#endif
#if AE_EXT_BLOCK_MASK
          {
            // the user's block of this (q, kv) position (positions past the end are invisible anyway: clamped)
            int mr = qi / p.mask_block_m, mc = ki / p.mask_block_n;
            mr = mr < p.mask_nq ? mr : p.mask_nq - 1;
            mc = mc < p.mask_nkv ? mc : p.mask_nkv - 1;
            const int64_t mbh = (int64_t)(p.mask_b == 1 ? 0 : b) * p.mask_h + (p.mask_h == 1 ? 0 : hq);
            vis = vis && p.block_mask[(mbh * p.mask_nq + mr) * p.mask_nkv + mc] != 0;
          }
#endif
          pv = vis ? pv : 0.f;
        }
        (void)qi; (void)ki;
#if AE_BWD_KIND == 0
        const float dsv = pv * dfac;                           // score_mod's derivative (the scale) is applied to the sums
#else
        const float dsv = vis ? dfac : 0.f;                    // an invisible score contributes nothing and moves nothing
#endif
        pvs[r] = pv;
        dss[r] = dsv;
      }
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        typedef float ae_f32x2 __attribute__((ext_vector_type(2)));
        const int e = nb * 16 + r;
        const ae_f32x2 p2 = {pvs[r], pvs[r + 1]}, d2 = {dss[r], dss[r + 1]};
        pf[e >> 3][(e & 7) >> 1] = __builtin_bit_cast(unsigned, __builtin_convertvector(p2, ae_elem2));
        dsf[e >> 3][(e & 7) >> 1] = __builtin_bit_cast(unsigned, __builtin_convertvector(d2, ae_elem2));
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    if (need_vis) {
      block(0, ae_bwd_true{});
      block(1, ae_bwd_true{});
    } else {
      block(0, ae_bwd_false{});
      block(1, ae_bwd_false{});
    }

    // OUT^T[d][resident] += X^T[d][streamed] ds[streamed][resident]: fragment f = (k-step kk, output block
    // j of dQ/dK, then of dV), read ahead through the same kind of ring
    {
      constexpr int NB_OUT = AE_NDB1 + (AE_BWD_ROLE == 1 ? AE_NDB2 : 0);
      constexpr int NF = 4 * NB_OUT;
      auto frag = [&](int f) AE_LAMBDA -> ae_elem8 {
        const int kk = f / NB_OUT, j = f % NB_OUT;
        return j < AE_NDB1 ? tr_frag(t1, AE_STR1, AE_CPR1, kk, j) : tr_frag(t2, AE_STR2, AE_CPR2, kk, j - AE_NDB1);
      };
      ae_elem8 ring[AE_RING];
#pragma unroll
      for (int f = 0; f < AE_AHEAD && f < NF; f++) ring[f] = frag(f);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int f = 0; f < NF; f++) {
        if (f + AE_AHEAD < NF) ring[(f + AE_AHEAD) % AE_RING] = frag(f + AE_AHEAD);
        const int kk = f / NB_OUT, j = f % NB_OUT;
        if (j < AE_NDB1) {
          acc1[j] = ae_mfma32(ring[f % AE_RING], __builtin_bit_cast(ae_elem8, dsf[kk]), acc1[j]);
        } else {
#if AE_BWD_ROLE == 1
          acc2[j - AE_NDB1] = ae_mfma32(ring[f % AE_RING], __builtin_bit_cast(ae_elem8, pf[kk]), acc2[j - AE_NDB1]);
#endif
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    (void)pf;

    // the next item has landed (with three stages the one after it is still outstanding)
    __builtin_amdgcn_s_waitcnt(AE_VMCNT((AE_NSTAGE - 2) * AE_NLOADS));
    __syncthreads();
    x0 = x1, cls0 = cls1;
    x1 = x2, cls1 = cls2;
    x2 = next_item(x2 + 1, cls2);
  }
  __builtin_amdgcn_s_waitcnt(AE_VMCNT(0));             // nothing may land in LDS after the workgroup has gone

  // ---- results: lane owns its resident row, columns 32*db + 8*(r/4) + 4*hf + r%4 ------------------
#if AE_OUT_VIA_LDS
  __syncthreads();       // ... of any wave: the ring becomes the staging area of the results
  {
    // (addresses from a copy of the lane id that the compiler cannot trace back to the prologue's)
    int le = lane;
    asm volatile("" : "+v"(le));
    ae_lds_byte* os1 = lds + wave * AE_OUT_BYTES;
    {
      ae_lds_byte* orow = os1 + (le & 31) * AE_STR1 + (le >> 5) * 8;
      const int osw = le & (AE_CPR1 - 1);
#pragma unroll
      for (int db = 0; db < AE_NDB1; db++)
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          ae_elem4 w;
#pragma unroll
          for (int t = 0; t < 4; t++) w[t] = (ae_elem)(acc1[db][rg * 4 + t] * AE_SM_SCALE);
          *(__attribute__((address_space(3))) ae_elem4*)(orow + (((db * 4 + rg) ^ osw) << 4)) = w;
        }
    }
#if AE_BWD_ROLE == 1
    {
      ae_lds_byte* orow = os1 + AE_R1B + (le & 31) * AE_STR2 + (le >> 5) * 8;
      const int osw = le & (AE_CPR2 - 1);
#pragma unroll
      for (int db = 0; db < AE_NDB2; db++)
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          ae_elem4 w;
#pragma unroll
          for (int t = 0; t < 4; t++) w[t] = (ae_elem)acc2[db][rg * 4 + t];
          *(__attribute__((address_space(3))) ae_elem4*)(orow + (((db * 4 + rg) ^ osw) << 4)) = w;
        }
    }
#endif
    // (the rows were written by other lanes of this wave: LDS instructions of a wave complete in order)
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const int rw0 = r0 + wave * 32;
#if AE_BWD_ROLE == 0
    ae_elem* o1 = (ae_elem*)p.dq + (int64_t)b * p.dq_stride_b + (int64_t)h * p.dq_stride_h;
    const int64_t os1s = p.dq_stride_s;
#else
    ae_elem* o1 = (ae_elem*)p.dk + (int64_t)b * p.dk_stride_b + (int64_t)h * p.dk_stride_h;
    ae_elem* o2 = (ae_elem*)p.dv + (int64_t)b * p.dv_stride_b + (int64_t)h * p.dv_stride_h;
    const int64_t os1s = p.dk_stride_s, os2s = p.dv_stride_s;
#endif
#pragma unroll
    for (int i = 0; i < AE_CPR1 / 2; i++) {
      const int n = i * 64 + le;
      const int row = n / AE_CPR1, c = n % AE_CPR1;
      const ae_elem8 w = *(const __attribute__((address_space(3))) ae_elem8*)(
          os1 + row * AE_STR1 + ((c ^ (row & (AE_CPR1 - 1))) << 4));
      if (rw0 + row < n_res) *(ae_elem8*)(o1 + (int64_t)(rw0 + row) * os1s + c * 8) = w;
    }
#if AE_BWD_ROLE == 1
#pragma unroll
    for (int i = 0; i < AE_CPR2 / 2; i++) {
      const int n = i * 64 + le;
      const int row = n / AE_CPR2, c = n % AE_CPR2;
      const ae_elem8 w = *(const __attribute__((address_space(3))) ae_elem8*)(
          os1 + AE_R1B + row * AE_STR2 + ((c ^ (row & (AE_CPR2 - 1))) << 4));
      if (rw0 + row < n_res) *(ae_elem8*)(o2 + (int64_t)(rw0 + row) * os2s + c * 8) = w;
    }
#endif
  }
  (void)r_ok;
#else
  if (r_ok) {
#if AE_BWD_ROLE == 0
    ae_elem* o1 = (ae_elem*)p.dq + (int64_t)b * p.dq_stride_b + (int64_t)rrow * p.dq_stride_s + (int64_t)h * p.dq_stride_h;
#else
    ae_elem* o1 = (ae_elem*)p.dk + (int64_t)b * p.dk_stride_b + (int64_t)rrow * p.dk_stride_s + (int64_t)h * p.dk_stride_h;
    ae_elem* o2 = (ae_elem*)p.dv + (int64_t)b * p.dv_stride_b + (int64_t)rrow * p.dv_stride_s + (int64_t)h * p.dv_stride_h;
#endif
#pragma unroll
    for (int db = 0; db < AE_NDB1; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        ae_elem4 w;
#pragma unroll
        for (int t = 0; t < 4; t++) w[t] = (ae_elem)(acc1[db][rg * 4 + t] * AE_SM_SCALE);
        *(ae_elem4*)(o1 + db * 32 + rg * 8 + hf * 4) = w;
      }
#if AE_BWD_ROLE == 1
#pragma unroll
    for (int db = 0; db < AE_NDB2; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        ae_elem4 w;
#pragma unroll
        for (int t = 0; t < 4; t++) w[t] = (ae_elem)acc2[db][rg * 4 + t];
        *(ae_elem4*)(o2 + db * 32 + rg * 8 + hf * 4) = w;
      }
#endif
  }
#endif  // results through LDS
}

#if AE_BWD_ROLE == 0
// Work buffer fp32 [2,B,Hq,Sq]: plane 0 = rowsum(do * o), the `doosum` row scale of the reference's
// backward (flashattn_bwd_preprocess, attn_tl.py:196-221); plane 1 = lse in log2 units, the form the two
// other launches subtract inside exp2.  DV/8 lanes share a row, 16 bytes each.
extern "C" __global__ __launch_bounds__(256)
void ae_bwd_delta_kernel(const ae_attn_bwd_params p) {
  constexpr int LPR = AE_DV / 8;                   // lanes per row
  constexpr int RPB = 256 / LPR;                   // rows per workgroup
  const int tid = threadIdx.x;
  const int64_t n_rows = (int64_t)p.batch * p.seqlen_q * p.heads_q;
  const int64_t row = (int64_t)blockIdx.x * RPB + tid / LPR;
  const int c = tid % LPR;
  float acc = 0.f;
  int b = 0, s = 0, h = 0;
  if (row < n_rows) {
    h = (int)(row % p.heads_q);
    s = (int)((row / p.heads_q) % p.seqlen_q);
    b = (int)(row / ((int64_t)p.heads_q * p.seqlen_q));
    const ae_elem8 o = *(const ae_elem8*)((const ae_elem*)p.out + (int64_t)b * p.o_stride_b + (int64_t)s * p.o_stride_s + (int64_t)h * p.o_stride_h + c * 8);
    const ae_elem8 d = *(const ae_elem8*)((const ae_elem*)p.dout + (int64_t)b * p.do_stride_b + (int64_t)s * p.do_stride_s + (int64_t)h * p.do_stride_h + c * 8);
#pragma unroll
    for (int j = 0; j < 8; j++) acc += (float)o[j] * (float)d[j];
  }
  // the LPR lanes of a row are consecutive and aligned: butterfly inside the group
#pragma unroll
  for (int m = 1; m < LPR; m <<= 1) {
    const int lane = tid & 63;
    acc += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ m) << 2, __builtin_bit_cast(int, acc)));
  }
  if (row < n_rows && c == 0) {
    const int64_t ri = ((int64_t)b * p.heads_q + h) * p.seqlen_q + s;
    const float l = p.lse ? p.lse[ri] : 0.f;
    p.delta[ri] = acc;
#if AE_BWD_KIND == 2
    // further planes: the online function's final row scales, as the forward wrote them
    p.delta[(int64_t)p.batch * p.heads_q * p.seqlen_q + ri] = l;
#pragma unroll
    for (int i = 1; i < AE_BWD_NRS; i++)
      p.delta[(int64_t)(1 + i) * p.batch * p.heads_q * p.seqlen_q + ri] = p.more_rowscales[i - 1][ri];
#else
    // second plane: lse in log2 units, +inf for a row without a visible key (its p is 0 everywhere)
    p.delta[(int64_t)p.batch * p.heads_q * p.seqlen_q + ri] = (l == AE_NEG_INF) ? __builtin_inff() : l * AE_LOG2E;
#endif
  }
}
#endif
