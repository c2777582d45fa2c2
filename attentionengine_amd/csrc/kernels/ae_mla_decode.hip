// MLA (shared latent KV) split-KV decode for gfx950 / CDNA4.
//
// Takes the place of the reference's TileLang MLA decode template
// (attention_engine/core/template/tl_template/attn/mla_decode_tl.py: flash_attn_split 104-179) and of
// the CuTe/FlashMLA split kernel (core/template/cute_template_kvshared/kernels/splitkv_mla.cu:
// 1061-1393).  K = [latent | rope] (AE_D = AE_D1 + AE_D2 wide), V = the first AE_DV columns of the
// same rows, one kv head shared by all query heads of its group (128 for DeepSeek-V3).
//
// This is a GEMM-shaped problem (arithmetic intensity ~ 2*heads flop per KV byte): the query HEADS
// play the role of query rows of a flash-attention forward.
//   * S^T[kv,head] = K Q^T and O^T[dv,head] += V^T P^T with v_mfma_f32_16x16x32; a lane owns one
//     head's online row state; Q stays in registers for the whole kernel (AE_D/32 fragments);
//   * a wave owns 16 heads and HALF of the value dimension, so its state -- 64 accumulator
//     registers + 72 of Q -- fits two waves per SIMD with plain VGPR accumulators.  (A 32-head
//     wave needs the 512-register budget of one wave per SIMD; the compiler then keeps Q in AGPRs
//     and copies four registers back before every MFMA, which measured 5x slower.)
//     A workgroup is 8 waves = 4 head blocks x 2 value halves = 64 heads of one (batch, kv head,
//     split); the two waves of a head block compute the same scores;
//   * each KV tile goes from HBM straight into LDS (global_load_lds_dwordx4: no staging registers,
//     no ds_write) once per workgroup and serves both products: K rows are read with ds_read_b128,
//     the V operand is read from the SAME LDS rows through ds_read_b64_tr_b16.  Direct loads cannot
//     pad rows, so bank conflicts are avoided by permuting the 16-byte chunks inside every aligned
//     group of eight: LDS chunk c' of row r holds global chunk c' ^ f(r),
//     f(r) = 2*((r>>1)&3) + ((r>>3)&1).  AE_NSTAGE tiles are in flight;
//   * the workgroups that share a KV range (the head tiles of one batch entry) get ids 8 apart, so
//     the round-robin dispatch puts them on the same XCD and the second reads the tile from its L2;
//   * partial (o, rowscales) per split in fp32, merged by ae_decode_combine_kernel.

#define AE_LAYOUT 1
#include "ae_hip.h"
#include "ae_config.h"
#include "ae_device.h"
#include "ae_functors.h"

#define AE_D (AE_D1 + AE_D2)
#define AE_NWAVES 8
#define AE_NT (AE_NWAVES * 64)
#define AE_HEADS_PER_WG ((AE_NWAVES / 2) * 16)
#define AE_BN 32                          // kv rows per tile
#define AE_NS 8                           // score elements per lane per tile (2 blocks of 4)
#define AE_NDB (AE_DV / 32)               // 16-wide dv blocks of this wave's half of DV
#define AE_NO (AE_NDB * 4)
#define AE_NKS (AE_D / 32)                // 32-deep k-steps of QK^T
#define AE_KSTR (AE_D * 2)                // LDS row pitch, bytes (unpadded: swizzled)
#define AE_STAGE_BYTES (AE_BN * AE_KSTR)
#define AE_CPR (AE_D / 8)                 // 16-byte chunks per K row
#define AE_CPR1 (AE_D1 / 8)               // chunks that come from the latent tensor
#define AE_BLOCKS ((AE_BN * AE_CPR) / 64) // 1 KiB blocks per tile
#define AE_LOADS ((AE_BLOCKS + AE_NWAVES - 1) / AE_NWAVES)   // direct loads per lane per tile
#ifndef AE_NSTAGE
#define AE_NSTAGE 3
#endif
// chunk permutation of row r (see the header comment)
#define AE_SWZ(r) ((((r) >> 1) & 3) * 2 + (((r) >> 3) & 1))

static_assert(AE_D1 % 32 == 0 && AE_D2 % 32 == 0, "latent / rope dims must be multiples of 32");
static_assert(AE_DV % 32 == 0 && AE_DV <= AE_D1, "V must be a prefix of the latent part");
static_assert(AE_CPR % 8 == 0 && AE_CPR1 % 8 == 0, "chunk groups of eight must not straddle the two K tensors");
static_assert((AE_BN * AE_CPR) % 64 == 0, "tile must be a whole number of 1 KiB blocks");
static_assert(2 * AE_LOADS <= 63, "vmcnt bookkeeping");

#ifndef AE_PAGED
#define AE_PAGED 0
#endif
#if AE_PAGED
#include "ae_mla_paged.h"
#endif

typedef __attribute__((address_space(3))) unsigned char ae_lds_byte;

extern "C" __global__ __launch_bounds__(AE_NT)
__attribute__((amdgpu_waves_per_eu(2, 2)))
void ae_mla_decode_split_kernel(const ae_attn_params p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ae_smem[];
  ae_lds_byte* lds = (ae_lds_byte*)ae_smem;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15;
  const int g4 = lane >> 4;

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
  const int hblk = wave >> 1;     // which 16 heads of the workgroup
  const int dvh = wave & 1;       // which half of the value dimension
  const int head_in_group = ht * AE_HEADS_PER_WG + hblk * 16 + l16;
  const bool head_ok = head_in_group < group;
  const int hq = hk * group + (head_ok ? head_in_group : 0);

  // ---- Q fragments: B operand of S^T = K Q^T (n = head = l16, k = d = 32*ks + 8*g4 + j) ------------
  const ae_elem* q1 = (const ae_elem*)p.q + (int64_t)b * p.q_stride_b + (int64_t)hq * p.q_stride_h;
  const ae_elem* q2 = (const ae_elem*)p.q2 + (int64_t)b * p.q2_stride_b + (int64_t)hq * p.q2_stride_h;
  ae_elem8 qf[AE_NKS];
#pragma unroll
  for (int ks = 0; ks < AE_D1 / 32; ks++) qf[ks] = *(const ae_elem8*)(q1 + ks * 32 + g4 * 8);
#pragma unroll
  for (int ks = 0; ks < AE_D2 / 32; ks++) qf[AE_D1 / 32 + ks] = *(const ae_elem8*)(q2 + ks * 32 + g4 * 8);

#if AE_PAGED
  // paged cache (cute_template_kvshared/kernels/params.h:33-36): rows are found through the block table,
  // every batch entry has its own length; a kv tile never straddles two pages
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

  const int kv_begin = split * p.kv_per_split;
  int kv_end = kv_begin + p.kv_per_split;
  kv_end = kv_end < seqlen_b ? kv_end : seqlen_b;
  const int n_tiles = kv_end > kv_begin ? (kv_end - kv_begin + AE_BN - 1) / AE_BN : 0;
#if AE_PAGED
  // a split beyond this entry's length writes nothing (the merge passes it over); split 0 of an entry of
  // length 0 writes that entry's "no keys" result
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

  // Direct HBM -> LDS tile load.  Instruction i of wave w fills the 1 KiB block
  // (w*AE_LOADS + i) mod AE_BLOCKS (a few blocks are fetched twice so every wave issues the same
  // number of loads); LDS slot s = 64*block + lane is chunk c' = s % CPR of row s / CPR and
  // receives global chunk c' ^ f(row).
  auto load_tile = [&](int t, int stage) AE_LAMBDA {
    const int kv0 = kv_begin + t * AE_BN;
    ae_lds_byte* dst = lds + stage * AE_STAGE_BYTES;
#if AE_PAGED
    // t < n_tiles, so kv0 < seqlen_b and its table entry is set; an entry outside the cache is clamped
    const int slot = kv0 / p.page_block_size;
    int page = pages[slot];
    page = page < 0 ? 0 : (page < p.num_pages ? page : p.num_pages - 1);
    page = __builtin_amdgcn_readfirstlane(page);
    const int page_row0 = slot * p.page_block_size;
    const ae_elem* k1t = k1 + (int64_t)page * p.k_stride_b - (int64_t)page_row0 * p.k_stride_s;
    const ae_elem* k2t = k2 + (int64_t)page * p.k2_stride_b - (int64_t)page_row0 * p.k2_stride_s;
#else
    const ae_elem* k1t = k1;
    const ae_elem* k2t = k2;
#endif
#pragma unroll
    for (int i = 0; i < AE_LOADS; i++) {
      const int blk = (wave * AE_LOADS + i) % AE_BLOCKS;
      const int sidx = blk * 64 + lane;
      const int row = sidx / AE_CPR, cp = sidx % AE_CPR;
      const int c = cp ^ AE_SWZ(row);
      int kv = kv0 + row;
      kv = kv < seqlen_b ? kv : seqlen_b - 1;
      const ae_elem* src = c < AE_CPR1 ? k1t + (int64_t)kv * p.k_stride_s + c * 8
                                       : k2t + (int64_t)kv * p.k2_stride_s + (c - AE_CPR1) * 8;
      ae_load_lds16(src, dst + blk * 1024);
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

  // lane-constant pieces of the swizzled read addresses
  // K fragment: row 16*rb + l16, global chunk 4*ks + g4
  const int k_row_off = l16 * AE_KSTR;
  const int k_sw = AE_SWZ(l16);                 // rows 16*rb + l16: same low bits
  // transpose read: lane i of a 16-lane group reads row 4*g4 + i/4 (+16 for kv slots 4..7),
  // 8 bytes at global chunk 2*dvblock + (i%4)/2, half (i%4)%2
  const int v_row = 4 * g4 + (l16 >> 2);
  const int v_row_off = v_row * AE_KSTR + (lane & 1) * 8;
  const int v_sw = AE_SWZ(v_row);               // +16 rows: same low bits
  const int v_c0 = (lane & 3) >> 1;

  // ---- pipeline: AE_NSTAGE - 1 tiles in flight ahead of the one being multiplied -----------------
  // The tile loads are invisible to the compiler's wait-count bookkeeping (see ae_load_lds16), so
  // everything it does know about (the Q fragments) is drained first: otherwise it would wait for
  // "its" loads with a vmcnt(0) inside the loop, which also waits for every tile in flight.
  __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
  for (int t = 0; t < AE_NSTAGE - 1; t++)
    if (t < n_tiles) load_tile(t, t);

  int stage = 0;
  for (int t = 0; t < n_tiles; t++) {
    // tile t has landed when at most the loads of the tiles issued after it are outstanding
    {
      const int newer = (n_tiles - 1 - t) < (AE_NSTAGE - 2) ? (n_tiles - 1 - t) : (AE_NSTAGE - 2);
      if (newer >= 2) __builtin_amdgcn_s_waitcnt(0x0F70 | ((2 * AE_LOADS) & 15) | (((2 * AE_LOADS) >> 4) << 14));
      else if (newer == 1) __builtin_amdgcn_s_waitcnt(0x0F70 | (AE_LOADS & 15) | ((AE_LOADS >> 4) << 14));
      else __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    __syncthreads();   // tile t visible to all waves; everyone is done with tile t-1's stage
    if (t + AE_NSTAGE - 1 < n_tiles) {
      int st_next = stage + AE_NSTAGE - 1;
      st_next = st_next >= AE_NSTAGE ? st_next - AE_NSTAGE : st_next;
      load_tile(t + AE_NSTAGE - 1, st_next);   // overwrites the stage of tile t-1
    }
    ae_lds_byte* ks_ = lds + stage * AE_STAGE_BYTES;
    const int kv0 = kv_begin + t * AE_BN;

    // ---- S^T = K Q^T: two 16-row kv blocks -----------------------------------------------------------
    ae_f32x4 sacc[2];
#pragma unroll
    for (int rb = 0; rb < 2; rb++) sacc[rb] = (ae_f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < AE_NKS; ks++) {
#pragma unroll
      for (int rb = 0; rb < 2; rb++) {
        ae_elem8 kf = *(__attribute__((address_space(3))) ae_elem8*)(
            ks_ + k_row_off + rb * 16 * AE_KSTR + (((4 * ks + g4) ^ k_sw) << 4));
        sacc[rb] = ae_mfma16(kf, qf[ks], sacc[rb]);
      }
    }
    float s[AE_NS];
#pragma unroll
    for (int rb = 0; rb < 2; rb++)
#pragma unroll
      for (int r = 0; r < 4; r++) s[rb * 4 + r] = sacc[rb][r];

    ctx.kv_base = kv0 + 4 * g4;
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
    // P as B operand of O^T += V^T P^T: slot j<4 is kv 4*g4+j, slot j>=4 is kv 16+4*g4+(j-4)
    ae_elem8 pf;
#pragma unroll
    for (int j = 0; j < 8; j++) pf[j] = (ae_elem)s[j];

#if !AE_O_SCALE_ONE
    if (__builtin_amdgcn_ballot_w64(o_scale != 1.0f) != 0) {
#pragma unroll
      for (int db = 0; db < AE_NDB; db++)
#pragma unroll
        for (int r = 0; r < 4; r++) oacc[db][r] *= o_scale;
    }
#else
    (void)o_scale;
#endif

    // ---- O^T += V^T P^T with V = the first AE_DV columns of the K rows already in LDS ---------------
#pragma unroll
    for (int db = 0; db < AE_NDB; db++) {
      const int cg = 2 * (dvh * AE_NDB + db) + v_c0;          // global 16-byte chunk of this lane
      ae_lds_byte* a0 = ks_ + v_row_off + ((cg ^ v_sw) << 4);
      ae_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) ae_s16x4*)a0);
      ae_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) ae_s16x4*)(a0 + 16 * AE_KSTR));
      ae_elem8 vf = __builtin_bit_cast(
          ae_elem8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      oacc[db] = ae_mfma16(vf, pf, oacc[db]);
    }
    stage = stage + 1 == AE_NSTAGE ? 0 : stage + 1;
  }

  // ---- per-split epilogue ------------------------------------------------------------------------------
  float o[AE_NO];
#pragma unroll
  for (int db = 0; db < AE_NDB; db++)
#pragma unroll
    for (int r = 0; r < 4; r++) o[db * 4 + r] = oacc[db][r];
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
  // no merge needed: write the output row and its rowscales directly
  if (head_ok && direct) {
    ae_elem* optr = (ae_elem*)p.out + (int64_t)b * p.o_stride_b + (int64_t)hq * p.o_stride_h +
                    dvh * (AE_DV / 2);
#pragma unroll
    for (int db = 0; db < AE_NDB; db++) {
      ae_elem4 w;
#pragma unroll
      for (int r = 0; r < 4; r++) w[r] = (ae_elem)o[db * 4 + r];
      *(ae_elem4*)(optr + db * 16 + g4 * 4) = w;
    }
    if (g4 == 0 && dvh == 0) {
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++)
        if (p.rowscale_out[i]) p.rowscale_out[i][(int64_t)b * p.heads_q + hq] = frs[i];
    }
  }
  if (head_ok && !direct) {
    const int64_t row = ((int64_t)b * p.heads_q + hq) * p.num_splits + split;
    float* po = p.partial_o + row * AE_DV + dvh * (AE_DV / 2);
#pragma unroll
    for (int db = 0; db < AE_NDB; db++) {
      ae_f32x4 w = {o[db * 4 + 0], o[db * 4 + 1], o[db * 4 + 2], o[db * 4 + 3]};
      *(ae_f32x4*)(po + db * 16 + g4 * 4) = w;
    }
    if (g4 == 0 && dvh == 0) {
#pragma unroll
      for (int i = 0; i < AE_N_ROWSCALES; i++)
        p.partial_rs[(int64_t)i * p.batch * p.heads_q * p.num_splits + row] = frs[i];
    }
  }
}

#include "ae_combine.h"
