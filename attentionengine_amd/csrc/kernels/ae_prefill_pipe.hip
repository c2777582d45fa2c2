// Software-pipelined flash attention forward (prefill) for gfx950 / CDNA4: the online softmax, or (AE_PIPE_KIND 1)
// any elementwise graph out = sum_kv f(s) v through its generated functor.
//
// Same role and operation order as ae_prefill.hip (the reference's TileLang prefill template,
// attention_engine/core/template/tl_template/attn/attn_tl.py:76-174, and its block-sparse sibling
// blockattn_tl.py:49-160), specialised for the case the lowering has PROVEN to be the online
// softmax of attn_script/mha.py:47-72 applied to `score * constant`:
//     m' = max(m, rowmax(s*c)), p = exp(s*c - m'), r' = r*exp(m - m') + rowsum(p), O' = O*exp(m - m') + pV
// Graphs with other row state use ae_prefill.hip, which runs the generated functors on whole tiles.
//
// Why a second kernel: with 32 query rows per wave every 32x32x16 MFMA needs a fresh 1 KiB A
// fragment (K or V^T) from LDS, and four SIMDs issuing MFMAs back to back then ask LDS for exactly
// its peak bandwidth.  Here a wave owns 64 query rows, so every fragment feeds two MFMAs and LDS
// traffic per flop halves.  The price is 128 (O) + 64 (S) accumulator registers + 64 for Q: one wave
// per SIMD, so no second wave hides the softmax arithmetic.  It is hidden by software pipelining
// inside the wave instead.  Measured on MI355X: a wave issues one instruction per 4 cycles, a
// 32x32x16 MFMA keeps the matrix pipe busy for 32 cycles but the wave's issue port for only about 16,
// v_exp_f32 costs 8; so the rest of an MFMA's time is free for independent VALU work.  One loop
// iteration therefore interleaves, MFMA by MFMA,
//     phase 1:  x(j+1) = K(j+1) Q'^T - m2   with   p(j) = exp2(x(j)), row sums, fp16 cast
//     phase 2:  O += V(j)^T p(j)^T          with   reading x(j+1) out of its accumulators, row maxima
// with `sched_barrier` fences pinning the interleaving, the exponentiation split into stages (exp2,
// pack + sum) that run in different MFMA slots so no instruction waits for the one just issued, A
// fragments read from LDS a few MFMAs ahead of their use into a small register ring, and the tile
// loads (HBM -> LDS direct) issued as two bursts from phase-1 slots.
// The loop is bound by the number of instructions a wave issues per tile, so what can leave the loop
// has left it: for fp16 the Q fragments are multiplied by c*log2e once (Q' above; the rounding of the
// product to fp16 moves a score by about 2^-12 of its size, inside the 1e-3 bar on lse for scores up
// to a few tens) and the row's reference -m2 enters as the C operand of the first k-step, so the MFMA
// result IS the exponent; bf16 (8 significant bits) keeps one fma per score instead.  The reference is
// lazy: it moves only when a tile exceeds it by more than 8 (p < 256), and then a cold path shifts the
// tile, rescales the running sum and leaves the loop so that O is rescaled outside it.
//
// Configuration ("ae_config.h"): AE_D AE_DV AE_BN(=64) AE_NWAVES AE_DTYPE_BF16 AE_MASK_MODE
// AE_HAS_MASK_MOD AE_N_ROWSCALES AE_EVEN_Q AE_EVEN_KV, plus AE_SM_SCALE (the constant c > 0) and
// AE_SM_M / AE_SM_R (names of the running-max and running-sum fields of ae_rowstate, which the
// lowering has checked to start at -inf and 0).
// Functors used ("ae_functors.h"): ae_rowstate, ae_rowstate_init, ae_mask_mod, ae_epilogue,
// ae_load_custom.

#include "ae_hip.h"
#include "ae_config.h"
#include "ae_device.h"
#include "ae_functors.h"
#include "ae_tile_table.h"
#ifndef AE_HEAVY_LAST
#define AE_HEAVY_LAST 0      // 1: the tile table gives late q tiles more work than early ones
#endif

#define AE_WROWS 64                // query rows per wave (two 32-row blocks)
#define AE_BM (AE_NWAVES * AE_WROWS)
#define AE_NT (AE_NWAVES * 64)
#define AE_NKS (AE_D / 16)         // k-steps of S^T = K Q^T
#define AE_NKF (AE_NKS * 2)        // K fragments per tile (two 32-row kv blocks per k-step)
#define AE_NDB (AE_DV / 32)        // 32-wide dv blocks
#define AE_NVF (4 * AE_NDB)        // V^T fragments per tile (four 16-deep k-steps)
#define AE_NO (AE_NDB * 16)
#define AE_KSTR (AE_D * 2)
#define AE_VSTR (AE_DV * 2)
#define AE_K_BYTES (AE_BN * AE_KSTR)
#define AE_V_BYTES (AE_BN * AE_VSTR)
#define AE_KCPR (AE_D / 8)
#define AE_VCPR (AE_DV / 8)
#define AE_K_LOADS ((AE_BN * AE_KCPR) / AE_NT)
#define AE_V_LOADS ((AE_BN * AE_VCPR) / AE_NT)
#define AE_K_RPI (64 / AE_KCPR)
#define AE_V_RPI (64 / AE_VCPR)
#define AE_VPPR (AE_VCPR / 2)
#define AE_QO_BYTES (AE_WROWS * (AE_KSTR > AE_VSTR ? AE_KSTR : AE_VSTR))   // a wave's Q rows, later its O rows
#define AE_VPS1 (32 / AE_NKF)      // scores per row handled next to one phase-1 MFMA
#define AE_VPS2 (32 / AE_NVF)      // scores per row read back next to one phase-2 MFMA
#ifndef AE_AHEAD
#define AE_AHEAD 3                 // fragments in flight ahead of the MFMA that uses them
#endif
#define AE_RING (AE_AHEAD + 1)
#ifndef AE_EXP_SPAN
#define AE_EXP_SPAN (2 * AE_NKF + 8)   // MFMA slots over which the 32 exponentiation units of a tile start
#endif
// K / V tile stages in LDS.  2: a tile is requested in the iteration before the one that multiplies it and waited
// for (vmcnt(0)) at that iteration's end, i.e. it has about three quarters of an iteration to arrive.  3: it is
// requested one iteration earlier still, and an iteration ends by waiting only until its OWN requests are the
// ones outstanding - the tile it waits for has had a whole further iteration.
#ifndef AE_KV_STAGES
#define AE_KV_STAGES 2
#endif
// order of a causal launch's workgroups: 0 = heaviest q tile first across ALL heads (longest job first),
// 1 = head by head (see below)
#ifndef AE_CAUSAL_ORDER
#define AE_CAUSAL_ORDER 0
#endif
static_assert(AE_KV_STAGES == 2 || AE_KV_STAGES == 3, "two or three K / V stages");
// s_waitcnt with vmcnt(n) and the other counters left alone (vmcnt is six bits wide: 3:0 and 15:14)
#define AE_VMCNT(n) (0x0F70 | ((n) & 15) | (((n) >> 4) << 14))
// tile loads a wave may leave in flight across the end of an iteration: its own requests of that iteration
#define AE_INFLIGHT (AE_KV_STAGES == 3 ? AE_K_LOADS + AE_V_LOADS : 0)
#ifndef AE_KLOAD_SLOT
#define AE_KLOAD_SLOT 7            // phase-1 MFMA slots after which the K and the V tile loads go out
#define AE_VLOAD_SLOT (AE_NKF + 7)
#endif
#define AE_TAU 5.545177444479562f  // 8 ln 2: the running maximum is refreshed only when it moved by more
// 1: an iteration ends by requesting the next one's first LDS fragments and compares the new tile's maxima
// with the reference while they travel; 0: it starts with the requests.  Measured on B2 H32 S4096 D128:
// 1 is 3.5 % faster without a mask, 0 is 2 % faster under a causal mask (set by the lowering).
#ifndef AE_TOP_PREFETCH
#define AE_TOP_PREFETCH (AE_MASK_MODE == 0)
#endif
// What turns a score into p.  0: the online softmax described above.  1: the generated functor
// ae_online_fwd itself, two scores at a time, for graphs the lowering has shown to be ELEMENTWISE
// (out = sum_kv f(s) v, attn_script/sigmoidattn.py, reluattn.py: no row state, no row reduction, no use of
// the kv index, o_scale = 1): the same pipeline without maxima, sums and the lazy reference.
#ifndef AE_PIPE_KIND
#define AE_PIPE_KIND 0
#endif
// 1: every workgroup reports the shader-clock cycles (s_memtime) and the constant-rate 100 MHz ticks
// (s_memrealtime) between its entry and its last store, as two 64-bit values at
// ((unsigned long long*)p.partial_o)[2 * blockIdx.x] - a buffer the prefill launch does not otherwise use.
// Their ratio is the shader clock the chip granted while the workgroup ran (a measurement build: bench.py
// --mfma-probe).
#ifndef AE_CLOCK_STAMPS
#define AE_CLOCK_STAMPS 0
#endif
// 1: Q carries c*log2e and the reference is the C operand of the first k-step (see above)
#ifndef AE_PRESCALE
#define AE_PRESCALE (!AE_DTYPE_BF16 && AE_PIPE_KIND == 0)
#endif

typedef __attribute__((address_space(3))) unsigned char ae_lds_byte;
#define AE_SB() __builtin_amdgcn_sched_barrier(0)
// C operand of a tile's first k-step for q block qb
#if AE_PRESCALE
#define AE_C0(qb) negc[qb]
#else
#define AE_C0(qb) zero16
#endif

struct ae_tag_true { static constexpr bool value = true; };
struct ae_tag_false { static constexpr bool value = false; };

extern "C" __global__ __launch_bounds__(AE_NT) __attribute__((amdgpu_waves_per_eu(1, 1)))
void ae_prefill_kernel(const ae_attn_params p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ae_smem[];
  ae_lds_byte* lds = (ae_lds_byte*)ae_smem;   // [AE_KV_STAGES][K tile], [AE_KV_STAGES][V tile], then AE_QO_BYTES per wave (its Q rows, later its O rows)

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hf = lane >> 5;
#if AE_CLOCK_STAMPS
  const unsigned long long ae_t0 = __builtin_amdgcn_s_memtime();
  const unsigned long long ae_w0 = __builtin_amdgcn_s_memrealtime();
#endif

  // ---- which (q-tile, head, batch): ids dealt so that the heads sharing K/V meet in one XCD's L2,
  // heavy causal q-tiles first (see ae_prefill.hip) -------------------------------------------
  const int n_qt = (p.seqlen_q + AE_BM - 1) / AE_BM;
  const int n_bh = p.batch * p.heads_q;
  const int wg = blockIdx.x;
  const int xcd = wg & 7;
  const int slot = wg >> 3;
#if AE_MASK_MODE == 1 || (AE_MASK_MODE == 2 && AE_HEAVY_LAST)
  // causal: q tiles differ in work by up to n_qt : 1, so ids go heaviest tile first across ALL heads
  // (longest-job-first keeps the tail short); the heads of one XCD still meet in its L2.  A tile table whose
  // late q tiles are the long ones (AE_HEAVY_LAST, found on the host: causal variants, long sliding windows)
  // takes the same order: B2 H32 S4096, "kv <= q + 1": 0.40 -> 0.35 ms.
  const int n_bg = (n_bh + 7) >> 3;
#if AE_CAUSAL_ORDER == 0
  const int qt = n_qt - 1 - slot / n_bg;
  const int bh = (slot % n_bg) * 8 + xcd;
#else
  // (measurement switch) head by head: the q tiles of one (batch, head) are adjacent in time, heaviest first, so
  // that its K / V stay in the XCD's L2 while they are used - at the price of a longer tail
  const int qt = n_qt - 1 - slot % n_qt;
  const int bh = (slot / n_qt) * 8 + xcd;
  (void)n_bg;
#endif
#else
  const int qt = slot % n_qt;
  const int bh = (slot / n_qt) * 8 + xcd;
#endif
  if (bh >= n_bh) return;
  const int h = bh % p.heads_q;
  const int b = bh / p.heads_q;
  const int hk = h / (p.heads_q / p.heads_kv);
  const int q0 = qt * AE_BM;
  const int q0w = q0 + wave * AE_WROWS;
  int qrow[2];
  bool q_ok[2];
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    qrow[qb] = q0w + qb * 32 + l32;
#if AE_EVEN_Q
    q_ok[qb] = true;
#else
    q_ok[qb] = qrow[qb] < p.seqlen_q;
#endif
  }

  // ---- Q fragments (B operand of S^T = K Q^T), resident ------------------------------------
  // The wave's 64 rows travel HBM -> LDS as whole rows (16 lanes per 256-byte row: a lane that fetched its own
  // row's fragments straight into registers asked for 32 rows per instruction, 16 bytes of each, and the
  // workgroups of a launch, which start and end together, then queue behind each other's requests: 3.5 us
  // until the first tile could be multiplied), swizzled like a K tile, into a region of the wave's own behind
  // the tile stages; the fragments are read from there once the first tiles have landed too.
  ae_elem8 qf[2][AE_NKS];
  ae_lds_byte* qo = lds + AE_KV_STAGES * (AE_K_BYTES + AE_V_BYTES) + wave * AE_QO_BYTES;
  {
    const int q0c = q0w < p.seqlen_q ? q0w : p.seqlen_q - 1;
    const char* qg = (const char*)((const ae_elem*)p.q + (int64_t)b * p.q_stride_b + (int64_t)q0c * p.q_stride_s +
                                   (int64_t)h * p.q_stride_h) - 4096;
#pragma unroll
    for (int g = 0; g < AE_KCPR / 8; g++) {
      unsigned off[8];
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const int row = (g * 8 + i) * AE_K_RPI + lane / AE_KCPR;
        const int c = (lane % AE_KCPR) ^ (row & (AE_KCPR - 1));
        int ra = q0w + row;                      // rows past the end re-read the last row
        ra = ra < p.seqlen_q ? ra : p.seqlen_q - 1;
        off[i] = (unsigned)(((ra - q0c) * (int)p.q_stride_s + c * 8) * 2 + 4096 - (i - 4) * 1024);
      }
      ae_load_lds16_burst_base<8>(qg, off, qo + (g * 8 + 4) * 1024);
    }
  }

  // ---- KV tile range and tile classes --------------------------------------------------------
  const int n_kvt = (p.seqlen_kv + AE_BN - 1) / AE_BN;
  int j_end = n_kvt;
#if AE_MASK_MODE == 1
  {
    int lim = (q0 + AE_BM + AE_BN - 1) / AE_BN;   // attn_tl.py:113-115
    j_end = lim < n_kvt ? lim : n_kvt;
  }
#endif
  // Under the causal mask a wave's own rows end before the workgroup's: the kv tiles past its diagonal are
  // invisible to all of its rows.  It does not multiply them (for 256-row q tiles six of the sixteen
  // (wave, tile) pairs on the diagonal), but keeps requesting its share of every tile and keeps meeting
  // the others at the barriers.
  int j_end_w = j_end;
#if AE_MASK_MODE == 1
  {
    int lim = (q0w + AE_WROWS + AE_BN - 1) / AE_BN;
    j_end_w = lim < j_end ? lim : j_end;
  }
#endif
#if AE_MASK_MODE == 2
  // tile classes from the block table, 64 kv tiles at a time (ae_tile_table.h): 0 skip, 1 elementwise mask,
  // 2 fully visible
  ae_tile_table tt;
  ae_tt_init(tt, p, b, h, q0, AE_BM);
#endif
  auto next_tile = [&](int j) AE_LAMBDA {
#if AE_MASK_MODE == 2
    j = ae_tt_next(tt, p, j, j_end, AE_BN, n_kvt);
#endif
    return j < j_end ? j : j_end;
  };
  // What tile j (just found by next_tile) means to this wave: the class of each lane's two rows (the table may
  // be finer than the 256-row q tile - user block masks -, so rows of one workgroup, even of one wave, can
  // differ), and whether the wave takes the masked path for it: anything but "every row of this wave sees the
  // whole tile".
  auto tile_info = [&](int j, int (&c)[2], bool& nm) AE_LAMBDA {
    nm = false;
    c[0] = c[1] = 2;
    if (j >= j_end) return;
#if AE_MASK_MODE == 1
    nm = j * AE_BN + AE_BN - 1 > q0w;
#elif AE_MASK_MODE == 2
    c[0] = ae_tt_class(tt, p, j, qrow[0]);
    c[1] = ae_tt_class(tt, p, j, qrow[1]);
    nm = __builtin_amdgcn_ballot_w64(c[0] != 2 || c[1] != 2) != 0;
#elif AE_HAS_MASK_MOD
    nm = true;
#endif
#if !AE_EVEN_KV
    nm = nm || (j * AE_BN + AE_BN > p.seqlen_kv);
#endif
  };

  const ae_elem* kbase = (const ae_elem*)p.k + (int64_t)b * p.k_stride_b + (int64_t)hk * p.k_stride_h;
  const ae_elem* vbase = (const ae_elem*)p.v + (int64_t)b * p.v_stride_b + (int64_t)hk * p.v_stride_h;

  // Direct HBM -> LDS tile loads with the chunk swizzles of ae_prefill.hip: wave w fills the AE_K_LOADS
  // (AE_V_LOADS) consecutive 1 KiB blocks starting at block w*AE_K_LOADS of a K (V) tile.  A lane's byte
  // offset inside a tile never changes, so it is computed once; per tile only a wave-uniform base moves.
  // A tile's loads go out as one burst behind a single write of M0 (see ae_load_lds16_burst; the offsets
  // carry the compensation for its immediate offsets).
  // (bases are passed 4 KiB low and the offsets 4 KiB high, so that the compensated offsets stay >= 0)
  auto k_lane_off = [&](int i, int last_row) AE_LAMBDA -> unsigned {
    int row = (wave * AE_K_LOADS + i) * AE_K_RPI + lane / AE_KCPR;
    const int c = (lane % AE_KCPR) ^ (row & (AE_KCPR - 1));
    row = row < last_row ? row : last_row;
    return (unsigned)((row * (int)p.k_stride_s + c * 8) * 2 + 4096 - (i - AE_K_LOADS / 2) * 1024);
  };
  auto v_lane_off = [&](int i, int last_row) AE_LAMBDA -> unsigned {
    int row = (wave * AE_V_LOADS + i) * AE_V_RPI + lane / AE_VCPR;
    const int cp = lane % AE_VCPR;
    const int c = (((cp >> 1) ^ (row & (AE_VPPR - 1))) << 1) | (cp & 1);
    row = row < last_row ? row : last_row;
    return (unsigned)((row * (int)p.v_stride_s + c * 8) * 2 + 4096 - (i - AE_V_LOADS / 2) * 1024);
  };
  unsigned koff[AE_K_LOADS], voff[AE_V_LOADS];
#pragma unroll
  for (int i = 0; i < AE_K_LOADS; i++) koff[i] = k_lane_off(i, AE_BN);
#pragma unroll
  for (int i = 0; i < AE_V_LOADS; i++) voff[i] = v_lane_off(i, AE_BN);
  auto load_k = [&](int j, int stage) AE_LAMBDA {
    const char* g = (const char*)kbase + (int64_t)j * AE_BN * p.k_stride_s * 2 - 4096;
    unsigned gp[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int ii = i < AE_K_LOADS ? i : 0;
      unsigned off = koff[ii];
#if !AE_EVEN_KV
      // rows past the end re-read the last row (masked later)
      if (j * AE_BN + AE_BN > p.seqlen_kv) off = k_lane_off(ii, p.seqlen_kv - 1 - j * AE_BN);
#endif
      gp[i] = off;
    }
    ae_load_lds16_burst_base<AE_K_LOADS>(g, gp, lds + stage * AE_K_BYTES + (wave * AE_K_LOADS + AE_K_LOADS / 2) * 1024);
  };
  auto load_v = [&](int j, int stage) AE_LAMBDA {
    const char* g = (const char*)vbase + (int64_t)j * AE_BN * p.v_stride_s * 2 - 4096;
    unsigned gp[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int ii = i < AE_V_LOADS ? i : 0;
      unsigned off = voff[ii];
#if !AE_EVEN_KV
      if (j * AE_BN + AE_BN > p.seqlen_kv) off = v_lane_off(ii, p.seqlen_kv - 1 - j * AE_BN);
#endif
      gp[i] = off;
    }
    ae_load_lds16_burst_base<AE_V_LOADS>(
        g, gp, lds + AE_KV_STAGES * AE_K_BYTES + stage * AE_V_BYTES + (wave * AE_V_LOADS + AE_V_LOADS / 2) * 1024);
  };

  // ---- the first tiles are requested before anything else is set up: the zeroing of the accumulators, the
  // constants and the address arithmetic below (about a thousand instructions of one wave per SIMD) then run
  // while they and the Q rows travel ----
  int j0 = next_tile(0);                  // tile whose scores are in sv (exp + PV next)
  int tc0[2], tc1[2], tc2[2], tcn[2];     // ... and what tiles j0, j1, j2, jn mean to this wave (tile_info)
  bool tnm0, tnm1, tnm2 = false, tnmn = false;
  tile_info(j0, tc0, tnm0);
  tc2[0] = tc2[1] = tcn[0] = tcn[1] = 2;
  const bool any_tile = j0 < j_end;
  int j1 = any_tile ? next_tile(j0 + 1) : j_end;   // tile multiplied by Q next
  tile_info(j1, tc1, tnm1);
#if AE_KV_STAGES == 3
  int j2 = j1 < j_end ? next_tile(j1 + 1) : j_end;  // with three stages the tile after it is on its way as well
  tile_info(j2, tc2, tnm2);
#endif
  if (any_tile) {
    load_k(j0, 0);
    load_v(j0, 0);
#if AE_KV_STAGES == 2
    if (j1 < j_end) load_k(j1, 1);
#else
    // (tiles past the end: the last tile again, so that every wave's requests can be counted)
    load_k(j1 < j_end ? j1 : j_end - 1, 1);
    load_v(j1 < j_end ? j1 : j_end - 1, 1);
    load_k(j2 < j_end ? j2 : j_end - 1, 2);
#endif
  }

  // ---- state ------------------------------------------------------------------------------
  ae_ctx ctx[2];
  ae_custom cust[2];
  ae_rowstate st[2];
  ae_f32x16 oacc[2][AE_NDB];
  // Scores leave the MFMAs already as the exponent of p:  x = s*c*log2e - m2.  With AE_PRESCALE the Q
  // fragments carry the factor c*log2e and -m2 is the C operand of the first k-step (16 equal registers
  // per q block, `negc`, kept in the accumulator file and rewritten only when the reference moves), so no
  // instruction touches a score between the MFMA and v_exp.  m2 is the row's reference in log2 units;
  // thr is what a tile maximum (relative to the reference) must exceed before the reference moves: 8
  // (p stays below 256), or -inf while the row has not seen a visible key and its reference is unset.
  float m2[2], r_run[2], thr[2];
#if AE_PRESCALE
  ae_f32x16 negc[2];
#else
  // (the first k-step starts from the constant 0, an operand the MFMA encodes itself: sixteen registers of
  // zeros per q block in the accumulator file, and the copies out of them, are what made the bf16 builds spill)
  ae_f32x16 zero16;
#pragma unroll
  for (int r = 0; r < 16; r++) zero16[r] = 0.f;
#endif
  ae_elem8 zero8;
#pragma unroll
  for (int i = 0; i < 8; i++) zero8[i] = (ae_elem)0.f;
  // a value DEFINED by an MFMA lives in the accumulator file: splat(v) + 0*0
  auto acc_splat = [&](float v) AE_LAMBDA -> ae_f32x16 {
    ae_f32x16 t;
#pragma unroll
    for (int r = 0; r < 16; r++) t[r] = v;
    return ae_mfma32(zero8, zero8, t);
  };
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    ctx[qb].b = b;
    ctx[qb].h = h;
    ctx[qb].q_idx = qrow[qb];
    ctx[qb].kv_base = 0;
    ae_load_custom(cust[qb], p, ctx[qb]);
    ae_rowstate_init(st[qb]);
    m2[qb] = 0.f;
    thr[qb] = AE_NEG_INF;
    r_run[qb] = 0.f;                  // per-lane partial sum; the two halves of a row meet in the epilogue
#if AE_PRESCALE
    negc[qb] = acc_splat(0.f);
#endif
#pragma unroll
    for (int db = 0; db < AE_NDB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[qb][db][r] = 0.f;
  }
  // (the zeroes are written now, while the first tiles travel: left alone, the compiler writes them after the wait)
#pragma unroll
  for (int qb = 0; qb < 2; qb++)
#pragma unroll
    for (int db = 0; db < AE_NDB; db++) asm volatile("" : "+a"(oacc[qb][db]));

  // lane-constant pieces of the swizzled LDS fragment addresses (see ae_prefill.hip)
  const int k_row_off = l32 * AE_KSTR;
  const int k_sw = l32 & (AE_KCPR - 1);
  const int v_row = 4 * hf + ((lane & 15) >> 2);
  const int v_row_off = v_row * AE_VSTR + (lane & 3) * 8;
  const int v_sw = v_row & (AE_VPPR - 1);
  const int v_g = l32 >> 4;

  // K fragment f = (k-step f/2, kv block f%2); V^T fragment f = (k-step f/NDB, dv block f%NDB)
  auto read_kfrag = [&](int f, const ae_lds_byte* kt) AE_LAMBDA -> ae_elem8 {
    const int ks = f >> 1, nb = f & 1;
    return *(const __attribute__((address_space(3))) ae_elem8*)(
        kt + k_row_off + nb * 32 * AE_KSTR + (((2 * ks + hf) ^ k_sw) << 4));
  };
  auto read_vfrag = [&](int f, const ae_lds_byte* vt) AE_LAMBDA -> ae_elem8 {
    const int kk = f / AE_NDB, db = f % AE_NDB;
    const int rb0 = (kk >> 1) * 32 + (kk & 1) * 16;
    const ae_lds_byte* a0 = vt + v_row_off + rb0 * AE_VSTR + (((2 * db + v_g) ^ v_sw) << 5);
    ae_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) ae_s16x4*)a0);
    ae_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) ae_s16x4*)(a0 + 8 * AE_VSTR));
    return __builtin_bit_cast(ae_elem8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  ae_f32x16 sacc[2][2];     // [kv block][q block] accumulators of the tile being multiplied
  float sv[2][32];          // [q block][score]: exponents x of the tile being exponentiated (masked)
  float mx[2];              // lane-local maxima of the tile being multiplied
  ae_u32x4 pf[2][4];        // [q block][k-step] P^T fragments (B operand of O^T += V^T P^T), as packed pairs
  ae_elem8 ring[AE_RING];
  bool rescale = false;
  float osc[2];             // factors of a pending rescale of O

  // read x out of its accumulators (q block qb, scores e0 .. e0+n-1) and track the maximum
  auto read_scores = [&](int qb, int e0, int n) AE_LAMBDA {
#pragma unroll
    for (int e = e0; e < e0 + n; e++) {
      float x = sacc[e >> 4][qb][e & 15];
      // pin the copy into an ordinary VGPR here, in the MFMA shadow; otherwise the register
      // allocator keeps the value in the accumulator file and re-reads it at the top of the loop
      asm volatile("" : "+v"(x));
      sv[qb][e] = x;
#if AE_PIPE_KIND == 0
      mx[qb] = __builtin_fmaxf(mx[qb], x);
#endif
    }
  };
  // p = exp2(x), two scores at a time ("unit" u: q block u%2, k-step u/8, pair (u/2)%4 of that k-step's 8
  // scores), in stages that run in DIFFERENT MFMA slots so that no instruction waits for the one just
  // issued: A = (without AE_PRESCALE) the fma that turns a raw score into x, B = exp2, C = convert + row
  // sum.  Unit u starts in slot (u * AE_EXP_SPAN) / 32; units are ordered by k-step, the order
  // O^T += V^T P^T needs them.
  float rsum[2];
  int kv_lim = 0;       // elementwise kind, ragged kv: keys of the tile in sv at offsets >= kv_lim (lane-relative) are past the end
  float xa[32][2];
  float negm2[2] = {0.f, 0.f};
  auto stage_a = [&](int u) AE_LAMBDA {
    const int qb = u & 1, e = (u >> 3) * 8 + ((u >> 1) & 3) * 2;
#if AE_PRESCALE || AE_PIPE_KIND == 1
    xa[u][0] = sv[qb][e];
    xa[u][1] = sv[qb][e + 1];
#else
    xa[u][0] = __builtin_fmaf(sv[qb][e], AE_SM_SCALE * AE_LOG2E, negm2[qb]);
    xa[u][1] = __builtin_fmaf(sv[qb][e + 1], AE_SM_SCALE * AE_LOG2E, negm2[qb]);
#endif
  };
  auto stage_b = [&](int u) AE_LAMBDA {
#if AE_PIPE_KIND == 1
    // (score_mod is fused into ae_online_fwd; the graph has neither row state nor an o_scale)
    ae_online_fwd<2>(xa[u], st[u & 1], ctx[u & 1], cust[u & 1]);
#else
    xa[u][0] = ae_exp2(xa[u][0]);
    xa[u][1] = ae_exp2(xa[u][1]);
#endif
  };
  auto stage_c = [&](int u) AE_LAMBDA {
    const int qb = u & 1, e = (u >> 3) * 8 + ((u >> 1) & 3) * 2;
    typedef float ae_f32x2 __attribute__((ext_vector_type(2)));
    const ae_f32x2 x2 = {xa[u][0], xa[u][1]};
    const ae_elem2 hv = __builtin_convertvector(x2, ae_elem2);   // one packed conversion, round to nearest
    pf[qb][e >> 3][(e & 7) >> 1] = __builtin_bit_cast(unsigned, hv);
#if AE_PIPE_KIND == 1
    (void)rsum;
#if !AE_EVEN_KV
    // keys past the end: f(-inf) need not be zero
    if (ae_kv_off(e) >= kv_lim) pf[qb][e >> 3][(e & 7) >> 1] = 0u;
    else if (ae_kv_off(e + 1) >= kv_lim) pf[qb][e >> 3][(e & 7) >> 1] &= 0xffffu;
#endif
#elif AE_DTYPE_BF16
    // bf16 keeps 8 significant bits: summing the rounded values would put ~1e-3 into lse for rows
    // with few visible keys, so the fp32 values are summed (fp16 sums the rounded pairs in one v_dot2)
    rsum[qb] += xa[u][0] + xa[u][1];
#else
    const ae_elem2 one = {(_Float16)1.0f, (_Float16)1.0f};
    rsum[qb] = __builtin_amdgcn_fdot2(hv, one, rsum[qb], false);
#endif
  };
  auto exp_slot = [&](int g) AE_LAMBDA {      // the stages that belong to MFMA slot g of an iteration
#pragma unroll
    for (int u = 0; u < 32; u++) {
      const int a = (u * AE_EXP_SPAN) / 32;
      if (a + 2 == g) stage_c(u);
      if (a + 1 == g) stage_b(u);
      if (a == g) stage_a(u);
    }
  };
  auto exp_all = [&]() AE_LAMBDA {            // all stages back to back (no MFMA to hide behind)
#pragma unroll
    for (int u = 0; u < 32; u++) stage_a(u);
#pragma unroll
    for (int u = 0; u < 32; u++) stage_b(u);
#pragma unroll
    for (int u = 0; u < 32; u++) stage_c(u);
  };
  // Tile j sits in sv, its lane-local maxima in mx: mask fix-up where the tile needs it, then the
  // row maxima against the (lazy) reference.  The common case ends after two exchanges and a ballot; a
  // row whose maximum exceeds its threshold moves its reference (cold path): sv is shifted, the
  // running sum rescaled here, O before the next iteration (rescale_o, outside the hot loop).
  auto finish_scores = [&](int j, const int (&tcls)[2], bool masked) AE_LAMBDA {
    const int kvb = j * AE_BN + 4 * hf;
    if (masked) {
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        mx[qb] = AE_NEG_INF;
#if AE_MASK_MODE == 2
        const int cls = tcls[qb];   // this row's class
#endif
#pragma unroll
        for (int e = 0; e < 32; e++) {
          const int kv = kvb + ae_kv_off(e);
          bool vis = true;
#if AE_MASK_MODE == 1
          vis = qrow[qb] >= kv;
#elif AE_MASK_MODE == 2
#if AE_HAS_MASK_MOD
          vis = cls == 2 || (cls == 1 && ae_mask_mod(b, h, qrow[qb], kv));
#else
          vis = cls != 0;
#endif
#elif AE_HAS_MASK_MOD
          vis = ae_mask_mod(b, h, qrow[qb], kv);
#endif
#if !AE_EVEN_KV
          vis = vis && (kv < p.seqlen_kv);
#endif
          const float x = vis ? sv[qb][e] : AE_NEG_INF;
          sv[qb][e] = x;
          mx[qb] = __builtin_fmaxf(mx[qb], x);
        }
      }
    }
#if AE_PIPE_KIND == 0
    float tmax[2];
    bool any_need = false;
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      float hi;
      const float lo = ae_swap32_lo_hi(mx[qb], hi);
#if AE_PRESCALE
      tmax[qb] = __builtin_fmaxf(lo, hi);                              // relative to the reference, log2 units
#else
      tmax[qb] = __builtin_fmaf(__builtin_fmaxf(lo, hi), AE_SM_SCALE * AE_LOG2E, negm2[qb]);
#endif
      any_need = any_need || (tmax[qb] > thr[qb]);
    }
    rescale = __builtin_amdgcn_ballot_w64(any_need) != 0;
    if (__builtin_expect(rescale, 0)) {
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        const bool need = tmax[qb] > thr[qb];
        const float d = need ? tmax[qb] : 0.f;
        // a row whose reference was unset has O = 0 and r = 0: any finite factor will do
        osc[qb] = (need && thr[qb] > AE_NEG_INF) ? ae_exp2(-d) : 1.0f;
        thr[qb] = need ? AE_TAU * AE_LOG2E : thr[qb];
        m2[qb] += d;
        r_run[qb] *= osc[qb];
#if AE_PRESCALE
#pragma unroll
        for (int e = 0; e < 32; e++) sv[qb][e] -= d;
        negc[qb] = acc_splat(-m2[qb]);
#else
        negm2[qb] = -m2[qb];
#endif
      }
    }
#endif  // AE_PIPE_KIND == 0
  };

  // ---- prologue: first tile's scores ------------------------------------------------------------
  // (three stages: V of the second tile and K of the third, requested last, may still be travelling)
  if (AE_KV_STAGES == 3 && any_tile) __builtin_amdgcn_s_waitcnt(AE_VMCNT(AE_INFLIGHT) & 0xF0FF);   // ... and lgkmcnt(0)
  else __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
#pragma unroll
  for (int qb = 0; qb < 2; qb++)
#pragma unroll
    for (int ks = 0; ks < AE_NKS; ks++) {
      ae_elem8 t = *(const __attribute__((address_space(3))) ae_elem8*)(
          qo + (qb * 32 + l32) * AE_KSTR + (((2 * ks + hf) ^ k_sw) << 4));
#if AE_PRESCALE
      // q * (c log2e), the product in fp32 rounded once to fp16: one mixed-precision fma per value (written as
      // conversions and a multiplication the compiler issues five instructions per pair)
      ae_u32x4 tp = __builtin_bit_cast(ae_u32x4, t);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        unsigned d;
        asm("v_fma_mixlo_f16 %0, %1, %2, 0 op_sel_hi:[1,0,0]" : "=&v"(d) : "v"(tp[i]), "s"(AE_SM_SCALE * AE_LOG2E));
        asm("v_fma_mixhi_f16 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]"
            : "+&v"(d) : "v"(tp[i]), "s"(AE_SM_SCALE * AE_LOG2E));
        tp[i] = d;
      }
      t = __builtin_bit_cast(ae_elem8, tp);
#endif
      qf[qb][ks] = t;
    }
  if (any_tile) {
#pragma unroll
    for (int f = 0; f < AE_NKF; f++) {
      const ae_elem8 kf = read_kfrag(f, lds);
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        sacc[f & 1][qb] = ae_mfma32(kf, qf[qb][f >> 1], f < 2 ? AE_C0(qb) : sacc[f & 1][qb]);
      }
    }
    mx[0] = mx[1] = AE_NEG_INF;
    read_scores(0, 0, 32);
    read_scores(1, 0, 32);
    finish_scores(j0, tc0, tnm0);
    rescale = false;                       // O is still zero
  }
  __syncthreads();                         // everyone is done with K stage 0 before it is refilled

  // ---- main loop ----------------------------------------------------------------------------------
  // iteration n (two stages): loads K(n+2) -> K stage n%2, V(n+1) -> V stage (n+1)%2;
  //              phase 1 multiplies K(n+1) (K stage (n+1)%2), phase 2 multiplies V(n) (V stage n%2).
  // With three stages the loads are K(n+3) -> K stage n%3 and V(n+2) -> V stage (n+2)%3.
  int n = 0;
  int sg = 0;     // n % AE_KV_STAGES: the stage of V(j0); K(j1) sits in the next one
  // first AE_AHEAD fragments of iteration n's stream: K(j1) if it has a next tile, else V(j0)
  auto prefetch_ring = [&]() AE_LAMBDA {
    if (j1 < j_end) {
      const ae_lds_byte* kt = lds + (sg + 1 == AE_KV_STAGES ? 0 : sg + 1) * AE_K_BYTES;
#pragma unroll
      for (int f = 0; f < AE_AHEAD; f++) ring[f] = read_kfrag(f, kt);
    } else {
      const ae_lds_byte* vt = lds + AE_KV_STAGES * AE_K_BYTES + sg * AE_V_BYTES;
#pragma unroll
      for (int f = 0; f < AE_AHEAD; f++) ring[f] = read_vfrag(f, vt);
    }
  };
#if AE_TOP_PREFETCH
  if (any_tile) prefetch_ring();
#endif
  // HN: the wave multiplies a next tile of its own.  TL (only without HN): it has none, but the other waves
  // have, so it still requests its share of the tiles they need.
  auto iteration = [&](auto has_next_tag, auto tail_loads_tag) AE_LAMBDA {
    constexpr bool HN = decltype(has_next_tag)::value;
    constexpr bool TL = decltype(tail_loads_tag)::value;
    const int sg1 = sg + 1 == AE_KV_STAGES ? 0 : sg + 1;              // stage of K(j1), V(j1)
    const int sgv = AE_KV_STAGES == 2 ? sg1 : (sg1 + 1 == 3 ? 0 : sg1 + 1);   // stage of the V tile requested now
    const ae_lds_byte* kt = lds + sg1 * AE_K_BYTES;
    const ae_lds_byte* vt = lds + AE_KV_STAGES * AE_K_BYTES + sg * AE_V_BYTES;
#if AE_KV_STAGES == 2
    const int jlast = j1;
#else
    const int jlast = j2;
#endif
    const int jn = (HN || TL) ? next_tile(jlast + 1) : j_end;        // the tile whose K is requested now
    tile_info(jn, tcn, tnmn);
    // Only this wave's requests of the previous iteration (none with two stages) are in flight here on the back
    // edge; saying so also clears loads still pending on loop ENTRY (Q fragments, spill reloads), which the
    // compiler's wait-count insertion would otherwise wait for after this iteration's tile loads
    // have been issued, i.e. with a vmcnt(0) that serialises them.
    __builtin_amdgcn_s_waitcnt(AE_VMCNT(AE_INFLIGHT));
    // The tile loads of this iteration, K(jn) and V(jlast), are issued as two bursts from phase-1 slots
    // below.  When there is no such tile the stage is refilled with the last tile, which nobody reads.
    const int j2l = jn < j_end ? jn : j_end - 1;
    const int jvl = jlast < j_end ? jlast : j_end - 1;
    // fragment stream of this iteration: K fragments 0..NKF-1 (if HN) then V fragments
    constexpr int NF1 = HN ? AE_NKF : 0;
    constexpr int NF = NF1 + AE_NVF;
    auto read_frag = [&](int f) AE_LAMBDA -> ae_elem8 {
      return f < NF1 ? read_kfrag(f, kt) : read_vfrag(f - NF1, vt);
    };
#if !AE_TOP_PREFETCH
#pragma unroll
    for (int f = 0; f < AE_AHEAD && f < NF; f++) ring[f % AE_RING] = read_frag(f);
#endif
    // (with AE_TOP_PREFETCH the first AE_AHEAD fragments are already on their way: prefetch_ring at the
    // end of the previous iteration, or of the prologue)
    rsum[0] = rsum[1] = 0.f;
    kv_lim = p.seqlen_kv - j0 * AE_BN - 4 * hf;
    AE_SB();

    // ---- phase 1: x(j1)^T = K Q^T - m2  ||  p(j0) ------------------------------------------------
    if (HN) {
#pragma unroll
      for (int f = 0; f < AE_NKF; f++) {
        if (f + AE_AHEAD < NF) ring[(f + AE_AHEAD) % AE_RING] = read_frag(f + AE_AHEAD);
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
          sacc[f & 1][qb] = ae_mfma32(ring[f % AE_RING], qf[qb][f >> 1], f < 2 ? AE_C0(qb) : sacc[f & 1][qb]);
          exp_slot(2 * f + qb);
          if (2 * f + qb == AE_KLOAD_SLOT) load_k(j2l, sg);
          if (2 * f + qb == AE_VLOAD_SLOT) load_v(jvl, sgv);
          AE_SB();
        }
      }
    } else {
      if (TL) {
        load_k(j2l, sg);
        load_v(jvl, sgv);
      }
      exp_all();
    }
    if (HN) mx[0] = mx[1] = AE_NEG_INF;
    AE_SB();
    // ---- phase 2: O^T += V(j0)^T P^T  ||  maxima of x(j1) -------------------------------------------
#pragma unroll
    for (int f = 0; f < AE_NVF; f++) {
      const int fs = NF1 + f;
      if (fs + AE_AHEAD < NF) ring[(fs + AE_AHEAD) % AE_RING] = read_frag(fs + AE_AHEAD);
#pragma unroll
      for (int qb = 0; qb < 2; qb++) {
        oacc[qb][f % AE_NDB] = ae_mfma32(ring[fs % AE_RING], __builtin_bit_cast(ae_elem8, pf[qb][f / AE_NDB]),
                                         oacc[qb][f % AE_NDB]);
        if (HN) {
          exp_slot(2 * AE_NKF + 2 * f + qb);
          read_scores(qb, f * AE_VPS2, AE_VPS2);
        }
        AE_SB();
      }
    }
#pragma unroll
    for (int qb = 0; qb < 2; qb++) r_run[qb] += rsum[qb];
#if !AE_TOP_PREFETCH
    if (HN) finish_scores(j1, tc1, tnm1);
#endif
    // tiles for the next iteration must have landed (with three stages they were requested an iteration ago: only
    // this iteration's own requests may still travel), and everyone must be done with this one's
    __builtin_amdgcn_s_waitcnt(AE_VMCNT((HN || TL) ? AE_INFLIGHT : 0));
    __syncthreads();
    j0 = j1;
    tc0[0] = tc1[0], tc0[1] = tc1[1], tnm0 = tnm1;
#if AE_KV_STAGES == 2
    j1 = jn;
    tc1[0] = tcn[0], tc1[1] = tcn[1], tnm1 = tnmn;
#else
    j1 = j2;
    tc1[0] = tc2[0], tc1[1] = tc2[1], tnm1 = tnm2;
    j2 = jn;
    tc2[0] = tcn[0], tc2[1] = tcn[1], tnm2 = tnmn;
#endif
    sg = sg1;
    n++;
#if AE_TOP_PREFETCH
    if (HN) {
      // the next iteration's first fragments go out now, and the new tile's maxima are compared with the
      // reference while they travel (an iteration that started with the reads would wait for them)
      prefetch_ring();
      finish_scores(j0, tc0, tnm0);
    }
#endif
  };

  // The rescale of O (rare once the reference has settled) stays OUTSIDE the hot loop: inside it, O
  // would have to be reachable by VALU instructions on every iteration and the register allocator
  // then shuttles all 128 accumulator registers between the two register files per tile.
  auto rescale_o = [&]() AE_LAMBDA {
#pragma unroll
    for (int qb = 0; qb < 2; qb++)
#pragma unroll
      for (int db = 0; db < AE_NDB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          // one accumulator register at a time through one scratch register: written as plain arithmetic,
          // the register allocator makes room for all of O in ordinary registers and pays for it with
          // ~70 registers stored to and reloaded from scratch memory in every workgroup's prologue
          float o = oacc[qb][db][r], t;
          asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\tv_accvgpr_write_b32 %0, %1"
                       : "+a"(o), "=&v"(t) : "v"(osc[qb]));
          oacc[qb][db][r] = o;
        }
    rescale = false;
  };
#if AE_MASK_MODE == 1
  // an iteration of a wave that is done with its own tiles: its share of the tile loads, and the barrier
  auto drain = [&]() AE_LAMBDA {
    const int sg1 = sg + 1 == AE_KV_STAGES ? 0 : sg + 1;
    const int sgv = AE_KV_STAGES == 2 ? sg1 : (sg1 + 1 == 3 ? 0 : sg1 + 1);
#if AE_KV_STAGES == 2
    const int jlast = j1;
#else
    const int jlast = j2;
#endif
    const int jn = next_tile(jlast + 1);
    load_k(jn < j_end ? jn : j_end - 1, sg);
    load_v(jlast < j_end ? jlast : j_end - 1, sgv);
    __builtin_amdgcn_s_waitcnt(AE_VMCNT(AE_INFLIGHT));
    __syncthreads();
    j0 = j1;
#if AE_KV_STAGES == 2
    j1 = jn;
#else
    j1 = j2;
    j2 = jn;
#endif
    sg = sg1;
    n++;      // (a wave that only requests tiles no longer looks at their classes)
  };
  if (any_tile) {
    while (true) {
      while (j1 < j_end_w && !rescale) iteration(ae_tag_true{}, ae_tag_false{});
      if (rescale) {
        rescale_o();
        continue;
      }
      break;
    }
    if (j1 < j_end) {              // the other waves go on: last product of this wave, then only loads
      iteration(ae_tag_false{}, ae_tag_true{});
      while (j1 < j_end) drain();
      __builtin_amdgcn_s_waitcnt(0x0070 | 0x0f00);
      __syncthreads();             // the barrier of the other waves' last iteration
    } else {
      iteration(ae_tag_false{}, ae_tag_false{});
    }
  }
#else
  if (any_tile) {
    while (true) {
      while (j1 < j_end && !rescale) iteration(ae_tag_true{}, ae_tag_false{});
      if (rescale) {
        rescale_o();
        continue;
      }
      break;
    }
    iteration(ae_tag_false{}, ae_tag_false{});
  }
#endif

  // ---- epilogue -------------------------------------------------------------------------------
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    float o[AE_NO];
#pragma unroll
    for (int db = 0; db < AE_NDB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[db * 16 + r] = oacc[qb][db][r];
    float frs[AE_N_ROWSCALES > 0 ? AE_N_ROWSCALES : 1];
    frs[0] = 0.f;
    if (any_tile) {
#if AE_PIPE_KIND == 0
      st[qb].AE_SM_M = m2[qb] * AE_LN2;
      st[qb].AE_SM_R = ae_group_sum(r_run[qb]);
      ae_epilogue<AE_NO>(o, st[qb], frs, ctx[qb], cust[qb]);
      // a row that saw tiles but no visible key: out = 0 (as for a q tile without any tile), not 0/0
      if (st[qb].AE_SM_R == 0.f) {
#pragma unroll
        for (int e = 0; e < AE_NO; e++) o[e] = 0.f;
      }
#else
      ae_epilogue<AE_NO>(o, st[qb], frs, ctx[qb], cust[qb]);
#endif
    } else {
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++) frs[i] = AE_NEG_INF;
    }
    // O leaves through the wave's LDS region (the Q rows are long in registers): a lane holds four adjacent
    // values of its own row per accumulator group, so stores straight from the registers would touch 32 rows
    // per instruction, 16 bytes of each
    {
      // (the addresses are derived from a copy of the lane id that the compiler cannot trace back: it would
      // otherwise keep the prologue's Q fragment addresses, which have the same form, in registers across the
      // whole loop and spill for it)
      int le = lane;
      asm volatile("" : "+v"(le));
      ae_lds_byte* orow = qo + (qb * 32 + (le & 31)) * AE_VSTR + (le >> 5) * 8;
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
    if (q_ok[qb] && hf == 0) {
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++)
        p.rowscale_out[i][((int64_t)b * p.heads_q + h) * p.seqlen_q + qrow[qb]] = frs[i];
    }
  }
  // (the rows were written by other lanes of this wave: LDS instructions of a wave complete in order)
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  {
    ae_elem* og = (ae_elem*)p.out + (int64_t)b * p.o_stride_b + (int64_t)h * p.o_stride_h;
    int le = lane;
    asm volatile("" : "+v"(le));
#pragma unroll
    for (int i = 0; i < AE_VCPR; i++) {
      const int row = i * AE_V_RPI + le / AE_VCPR;
      const int c = le % AE_VCPR;
      const ae_elem8 w = *(const __attribute__((address_space(3))) ae_elem8*)(
          qo + row * AE_VSTR + ((c ^ (row & (AE_VCPR - 1))) << 4));
      if (AE_EVEN_Q || q0w + row < p.seqlen_q) *(ae_elem8*)(og + (int64_t)(q0w + row) * p.o_stride_s + c * 8) = w;
    }
  }
#if AE_CLOCK_STAMPS
  __builtin_amdgcn_s_waitcnt(0);          // the stores have been acknowledged
  {
    const unsigned long long t1 = __builtin_amdgcn_s_memtime();
    const unsigned long long w1 = __builtin_amdgcn_s_memrealtime();
    if (tid == 0) {
      unsigned long long* st = (unsigned long long*)p.partial_o + 2 * (unsigned long long)blockIdx.x;
      st[0] = t1 - ae_t0;
      st[1] = w1 - ae_w0;
    }
  }
#endif
}
