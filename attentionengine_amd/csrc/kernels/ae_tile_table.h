// Tile classes from the block table (AE_MASK_MODE 2), shared by the prefill kernels.
//
// The table (ae_attn_params.block_mask, int8 [B|1, H|1, mask_nq, mask_nkv], blocks of mask_block_m x
// mask_block_n positions) says per block: 0 = no visible position (skip), 2 = every position visible,
// 1 = ask mask_mod per element (tables planned on the host from mask_mod), or simply "visible" for a block
// mask the user supplies (blockattn_tl.py:90-101 of the reference: a tile whose mask entry is 0 is skipped).
//
// A workgroup's q tile spans up to AE_TT_ROWS table rows and walks the kv tiles in order.  Reading the table
// tile by tile inside the loop is what must not happen: each skipped tile would cost a dependent memory access,
// and behind the tile loads' asm statements the compiler reads the entry with a vector load whose wait
// (vmcnt(0)) also waits for every tile in flight.  Instead every wave reads the classes of 64 consecutive kv
// tiles at once, one tile per lane and table row, and keeps them as ballots: one 64-bit mask per table row for
// "visible" and one for "fully visible".  The next tile with work is then a find-first-set on scalar registers
// and the class of a lane's own rows a few selects; the table is touched again only every 64 kv tiles.
#pragma once

#ifndef AE_TT_ROWS
#define AE_TT_ROWS 8      // table rows one q tile may span (checked on the host)
#endif

struct ae_tile_table {
  const int8_t* base;     // table of this (batch, head)
  int r0, nr;             // table rows of the workgroup's q tile: r0 ... r0 + nr - 1
  int c0;                 // the masks cover kv tiles c0 ... c0 + 63 (c0 a multiple of 64; -64: nothing loaded)
  unsigned long vis;      // some row of the q tile sees the tile
  unsigned long rvis[AE_TT_ROWS], rfull[AE_TT_ROWS];
};

AE_DEV void ae_tt_init(ae_tile_table& t, const ae_attn_params& p, int b, int h, int q0, int rows) {
  t.base = p.block_mask +
      ((int64_t)(p.mask_b == 1 ? 0 : b) * p.mask_h + (p.mask_h == 1 ? 0 : h)) * p.mask_nq * (int64_t)p.mask_nkv;
  t.r0 = q0 / p.mask_block_m;
  int r1 = (q0 + rows - 1) / p.mask_block_m;
  r1 = r1 < p.mask_nq ? r1 : p.mask_nq - 1;
  t.nr = r1 - t.r0 + 1;
  t.nr = t.nr < AE_TT_ROWS ? t.nr : AE_TT_ROWS;
  t.c0 = -64;
  t.vis = 0;
}

// classes of kv tiles c0 ... c0 + 63 (tiles of `bn` positions, n_kvt of them in all); every lane of the wave
AE_DEV void ae_tt_load(ae_tile_table& t, const ae_attn_params& p, int c0, int bn, int n_kvt) {
  const int lane = threadIdx.x & 63;
  const int j = c0 + lane;
  int col = ((j < n_kvt ? j : n_kvt - 1) * bn) / p.mask_block_n;
  col = col < p.mask_nkv ? col : p.mask_nkv - 1;
  t.c0 = c0;
  t.vis = 0;
#pragma unroll
  for (int r = 0; r < AE_TT_ROWS; r++) {
    int c = 0;
    if (r < t.nr && j < n_kvt) c = t.base[(int64_t)(t.r0 + r) * p.mask_nkv + col];
    t.rvis[r] = __builtin_amdgcn_ballot_w64(c != 0);
    t.rfull[r] = __builtin_amdgcn_ballot_w64(c == 2);
    t.vis |= t.rvis[r];
  }
}

// first kv tile >= j (and < j_end) that some row of the q tile sees, or j_end; leaves the masks on its chunk
AE_DEV int ae_tt_next(ae_tile_table& t, const ae_attn_params& p, int j, int j_end, int bn, int n_kvt) {
  while (j < j_end) {
    if (j < t.c0 || j >= t.c0 + 64) ae_tt_load(t, p, j & ~63, bn, n_kvt);
    const unsigned long m = t.vis >> (j - t.c0);
    if (m != 0) {
      j += __builtin_ctzl(m);
      break;
    }
    j = t.c0 + 64;
  }
  return j < j_end ? j : j_end;
}

// class of kv tile j (inside the chunk the masks are on) for query row q_row: 0, 1 or 2
AE_DEV int ae_tt_class(const ae_tile_table& t, const ae_attn_params& p, int j, int q_row) {
  const int bit = j - t.c0;
  int ri = q_row / p.mask_block_m - t.r0;
  ri = ri < t.nr - 1 ? ri : t.nr - 1;
  int cls = 0;
#pragma unroll
  for (int r = 0; r < AE_TT_ROWS; r++) {
    const int c = ((t.rvis[r] >> bit) & 1ul) ? (((t.rfull[r] >> bit) & 1ul) ? 2 : 1) : 0;    // wave-uniform
    cls = ri == r ? c : cls;
  }
  return cls;
}
