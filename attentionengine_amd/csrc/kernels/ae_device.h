// Device-side helpers shared by the gfx950 attention kernel templates.
//
// Element types, MFMA wrappers, the register layouts of the 32x32x16 MFMA accumulator and
// the row reductions / transcendentals the generated functors call. The transcendental
// definitions follow the reference's code generator (core/codegen/tl_gen.py:89-117):
// exp(x) = exp2(x * log2 e), log(x) = log2(x) * ln 2, tanh via a fast approximation.
#ifndef AE_DEVICE_H
#define AE_DEVICE_H

// hipRTC predefines the HIP device environment; an offline hipcc build has to include it.
#ifndef __HIPCC_RTC__
#include <hip/hip_runtime.h>
#endif
#include "ae_hip.h"

#if AE_DTYPE_BF16
typedef __bf16 ae_elem;
#else
typedef _Float16 ae_elem;
#endif
typedef ae_elem ae_elem8 __attribute__((ext_vector_type(8)));
typedef ae_elem ae_elem4 __attribute__((ext_vector_type(4)));
typedef ae_elem ae_elem2 __attribute__((ext_vector_type(2)));
typedef float ae_f32x16 __attribute__((ext_vector_type(16)));
typedef float ae_f32x4 __attribute__((ext_vector_type(4)));
typedef short ae_s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned int ae_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int ae_u32x2 __attribute__((ext_vector_type(2)));

#define AE_DEV __device__ inline __attribute__((always_inline))
// for the call operator of a lambda: a lambda that the inliner leaves as a function keeps the arrays it captures
// by reference in scratch memory (seen with the larger bf16 builds of the pipelined prefill kernel: 752 bytes of
// scratch per lane, 30 times the run time)
#define AE_LAMBDA __attribute__((always_inline))
#define AE_NEG_INF (-__builtin_inff())
#define AE_LOG2E 1.4426950408889634f
#define AE_LN2 0.6931471805599453f

// D[m][n] += sum_k A[m][k] B[k][n], 32x32 output, 16-deep. Lane l supplies A[l%32][8*(l/32)+j]
// and B[8*(l/32)+j][l%32], j=0..7, and owns D[8*(r/4) + 4*(l/32) + r%4][l%32], r=0..15.
AE_DEV ae_f32x16 ae_mfma32(ae_elem8 a, ae_elem8 b, ae_f32x16 c) {
#if AE_DTYPE_BF16
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
#else
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
#endif
}

// D[m][n], 16x16 output, 32-deep. Lane l supplies A[l%16][8*(l/16)+j], B[8*(l/16)+j][l%16]
// and owns D[4*(l/16) + r][l%16], r=0..3.
AE_DEV ae_f32x4 ae_mfma16(ae_elem8 a, ae_elem8 b, ae_f32x4 c) {
#if AE_DTYPE_BF16
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
#else
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
#endif
}

// ---- direct HBM -> LDS load --------------------------------------------------------------------
// 16 bytes per lane from `gptr` (any per-lane address) to LDS at lds_base + lane*16, lds_base wave
// uniform.  Issued as inline assembly rather than through __builtin_amdgcn_global_load_lds: when the
// compiler knows about a pending LDS-DMA write it makes every LDS read it cannot prove disjoint
// (all ds_read_tr*, which carry no precise memory operand) wait for vmcnt(0), i.e. for the tile that
// was just requested for LATER, which serialises the prefetch.  Callers order these loads against
// their consumers themselves: s_waitcnt vmcnt(..) followed by a workgroup barrier.
typedef __attribute__((address_space(3))) unsigned char ae_lds_u8;
AE_DEV void ae_load_lds16(const void* gptr, ae_lds_u8* lds_base) {
  const unsigned m0v = __builtin_amdgcn_readfirstlane((unsigned)(unsigned long)lds_base);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(gptr), "s"(m0v) : "memory");
}

// The 4-byte form: lane i's dword lands at lds_base + 4*i.
AE_DEV void ae_load_lds4(const void* gptr, ae_lds_u8* lds_base) {
  const unsigned m0v = __builtin_amdgcn_readfirstlane((unsigned)(unsigned long)lds_base);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" : : "v"(gptr), "s"(m0v) : "memory");
}

// N (1..8) such loads behind ONE write of M0.  Every write of M0 makes the wave wait for its LDS reads
// in flight, which costs a kernel that keeps its LDS pipe busy about 40 ns per load; a burst pays that
// once.  Load i lands at lds_mid + (i - N/2) KiB + lane*16.  The instruction's immediate offset moves
// the LDS address AND the global address, so the caller passes g[i] = source pointer - (i - N/2) KiB
// (the sum is what is dereferenced).  g must have 8 entries; those from N on are ignored.
template <int N>
AE_DEV void ae_load_lds16_burst(const void* const* g, ae_lds_u8* lds_mid) {
  static_assert(N >= 1 && N <= 8, "the 13-bit signed immediate offset reaches -4 KiB .. +3 KiB");
  const unsigned m0v = __builtin_amdgcn_readfirstlane((unsigned)(unsigned long)lds_mid);
  asm volatile(
      "s_mov_b32 m0, %8\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %0, off offset:(0-%9/2)*1024\n\t"
      ".if %9 > 1\n\tglobal_load_lds_dwordx4 %1, off offset:(1-%9/2)*1024\n\t.endif\n\t"
      ".if %9 > 2\n\tglobal_load_lds_dwordx4 %2, off offset:(2-%9/2)*1024\n\t.endif\n\t"
      ".if %9 > 3\n\tglobal_load_lds_dwordx4 %3, off offset:(3-%9/2)*1024\n\t.endif\n\t"
      ".if %9 > 4\n\tglobal_load_lds_dwordx4 %4, off offset:(4-%9/2)*1024\n\t.endif\n\t"
      ".if %9 > 5\n\tglobal_load_lds_dwordx4 %5, off offset:(5-%9/2)*1024\n\t.endif\n\t"
      ".if %9 > 6\n\tglobal_load_lds_dwordx4 %6, off offset:(6-%9/2)*1024\n\t.endif\n\t"
      ".if %9 > 7\n\tglobal_load_lds_dwordx4 %7, off offset:(7-%9/2)*1024\n\t.endif"
      :
      : "v"(g[0]), "v"(g[1]), "v"(g[2]), "v"(g[3]), "v"(g[4]), "v"(g[5]), "v"(g[6]), "v"(g[7]), "s"(m0v), "n"(N)
      : "memory");
}

// The same burst for loads whose lanes all read from one wave-uniform base: address = base (SGPR pair)
// + off[i] (unsigned 32-bit, per lane) + immediate.  No 64-bit address arithmetic and one VGPR per load.
// The caller passes off[i] = byte offset from base - (i - N/2) KiB, which must not be negative.
template <int N>
AE_DEV void ae_load_lds16_burst_base(const void* base, const unsigned* off, ae_lds_u8* lds_mid) {
  static_assert(N >= 1 && N <= 8, "the 13-bit signed immediate offset reaches -4 KiB .. +3 KiB");
  const unsigned m0v = __builtin_amdgcn_readfirstlane((unsigned)(unsigned long)lds_mid);
  // the base must sit in scalar registers even where the compiler cannot prove it wave uniform
  const unsigned long bv = (unsigned long)base;
  // (readfirstlane returns a signed int: go through unsigned, or the low half sign-extends into the high)
  const unsigned b_hi = (unsigned)__builtin_amdgcn_readfirstlane((unsigned)(bv >> 32));
  const unsigned b_lo = (unsigned)__builtin_amdgcn_readfirstlane((unsigned)bv);
  const unsigned long ub = ((unsigned long)b_hi << 32) | (unsigned long)b_lo;
  asm volatile(
      "s_mov_b32 m0, %8\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %0, %10 offset:(0-%9/2)*1024\n\t"
      ".if %9 > 1\n\tglobal_load_lds_dwordx4 %1, %10 offset:(1-%9/2)*1024\n\t.endif\n\t"
      ".if %9 > 2\n\tglobal_load_lds_dwordx4 %2, %10 offset:(2-%9/2)*1024\n\t.endif\n\t"
      ".if %9 > 3\n\tglobal_load_lds_dwordx4 %3, %10 offset:(3-%9/2)*1024\n\t.endif\n\t"
      ".if %9 > 4\n\tglobal_load_lds_dwordx4 %4, %10 offset:(4-%9/2)*1024\n\t.endif\n\t"
      ".if %9 > 5\n\tglobal_load_lds_dwordx4 %5, %10 offset:(5-%9/2)*1024\n\t.endif\n\t"
      ".if %9 > 6\n\tglobal_load_lds_dwordx4 %6, %10 offset:(6-%9/2)*1024\n\t.endif\n\t"
      ".if %9 > 7\n\tglobal_load_lds_dwordx4 %7, %10 offset:(7-%9/2)*1024\n\t.endif"
      :
      : "v"(off[0]), "v"(off[1]), "v"(off[2]), "v"(off[3]), "v"(off[4]), "v"(off[5]), "v"(off[6]), "v"(off[7]),
        "s"(m0v), "n"(N), "s"(ub)
      : "memory");
}

// ---- transcendentals ------------------------------------------------------------------
AE_DEV float ae_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
AE_DEV float ae_exp(float x) { return __builtin_amdgcn_exp2f(x * AE_LOG2E); }
AE_DEV float ae_log2(float x) { return __builtin_amdgcn_logf(x); }
AE_DEV float ae_log(float x) { return __builtin_amdgcn_logf(x) * AE_LN2; }
AE_DEV float ae_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
// tanh(x) = 1 - 2 / (exp(2x) + 1); saturates cleanly at +-1 for large |x|.
AE_DEV float ae_tanh(float x) {
  float e = __builtin_amdgcn_exp2f(x * (2.0f * AE_LOG2E));
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}
AE_DEV float ae_abs(float x) { return __builtin_fabsf(x); }
AE_DEV float ae_max(float a, float b) { return __builtin_fmaxf(a, b); }

// ---- exchange between the lanes that share one query row -----------------------------------
// AE_LAYOUT 0 (prefill, 32x32x16 MFMA, S^T accumulators): a row lives in lanes l and l^32.
//   permlane32_swap with both operands equal returns (value of the low half, value of the
//   high half) in every lane of the pair.
// AE_LAYOUT 1 (decode, 16x16x32 MFMA): a row (one query head) lives in lanes l, l^16, l^32, l^48.
#ifndef AE_LAYOUT
#define AE_LAYOUT 0
#endif
AE_DEV float ae_swap32_lo_hi(float v, float& hi) {
  unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  hi = __builtin_bit_cast(float, (unsigned)r[1]);
  return __builtin_bit_cast(float, (unsigned)r[0]);
}
// the values of the even and of the odd 16-lane row of a lane's row pair (v_permlane16_swap with both operands
// equal): an exchange inside the VALU, where ds_bpermute goes through the LDS pipeline and back
AE_DEV float ae_swap16_even_odd(float v, float& odd) {
  unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  odd = __builtin_bit_cast(float, (unsigned)r[1]);
  return __builtin_bit_cast(float, (unsigned)r[0]);
}
AE_DEV float ae_group_max(float v) {
#if AE_LAYOUT == 1
  {
    float od;
    const float ev = ae_swap16_even_odd(v, od);
    v = __builtin_fmaxf(ev, od);
  }
#endif
  float hi;
  float lo = ae_swap32_lo_hi(v, hi);
  return __builtin_fmaxf(lo, hi);
}
AE_DEV float ae_group_sum(float v) {
#if AE_LAYOUT == 1
  {
    float od;
    const float ev = ae_swap16_even_odd(v, od);
    v = ev + od;
  }
#endif
  float hi;
  float lo = ae_swap32_lo_hi(v, hi);
  return lo + hi;
}

// ---- row reductions over the lane's slice of a score row + the lanes sharing the row --------
// (ReduceMax / ReduceSum / ReduceAbsSum over dim=1 of the [block_M, block_N] tile,
//  core/codegen/tl_gen.py:9-21.)
template <int N>
AE_DEV float ae_row_max(const float (&s)[N]) {
  float m = s[0];
#pragma unroll
  for (int e = 1; e < N; e++) m = __builtin_fmaxf(m, s[e]);
  return ae_group_max(m);
}
template <int N>
AE_DEV float ae_row_sum(const float (&s)[N]) {
  // four independent chains keep the adds off one dependency path
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
  for (int e = 0; e + 3 < N; e += 4) {
    a0 += s[e];
    a1 += s[e + 1];
    a2 += s[e + 2];
    a3 += s[e + 3];
  }
#pragma unroll
  for (int e = N & ~3; e < N; e++) a0 += s[e];
  return ae_group_sum((a0 + a1) + (a2 + a3));
}
template <int N>
AE_DEV float ae_row_abssum(const float (&s)[N]) {
  float a0 = 0.f, a1 = 0.f;
#pragma unroll
  for (int e = 0; e + 1 < N; e += 2) {
    a0 += __builtin_fabsf(s[e]);
    a1 += __builtin_fabsf(s[e + 1]);
  }
#pragma unroll
  for (int e = N & ~1; e < N; e++) a0 += __builtin_fabsf(s[e]);
  return ae_group_sum(a0 + a1);
}

// ---- reductions over the split axis (ColReduce*, used by OnlineFunc.combine) -----------------
template <int N>
AE_DEV float ae_arr_max(const float (&s)[N]) {
  float m = s[0];
#pragma unroll
  for (int e = 1; e < N; e++) m = __builtin_fmaxf(m, s[e]);
  return m;
}
template <int N>
AE_DEV float ae_arr_sum(const float (&s)[N]) {
  float a = 0.f;
#pragma unroll
  for (int e = 0; e < N; e++) a += s[e];
  return a;
}
template <int N>
AE_DEV float ae_arr_abssum(const float (&s)[N]) {
  float a = 0.f;
#pragma unroll
  for (int e = 0; e < N; e++) a += __builtin_fabsf(s[e]);
  return a;
}

// Per-row context handed to the functors.
struct ae_ctx {
  int b;        // batch index
  int h;        // query head index
  int q_idx;    // absolute query position of this lane's row
  int kv_base;  // absolute kv position of element 0 of the lane's slice in the current tile
};

// kv offset (relative to ae_ctx::kv_base) of element e of a lane's slice of a score row.
// AE_LAYOUT 0: the slice is NB accumulator blocks of 16; block nb covers kv 32*nb .. 32*nb+31 and
//   register r of half-wave hf holds kv 8*(r/4) + 4*hf + r%4 (4*hf is folded into kv_base).
// AE_LAYOUT 1: blocks of 4; block rb covers kv 16*rb .. 16*rb+15 and register r of lane group g
//   holds kv 4*g + r (4*g is folded into kv_base).
#if AE_LAYOUT == 1
AE_DEV constexpr int ae_kv_off(int e) { return (e >> 2) * 16 + (e & 3); }
#else
AE_DEV constexpr int ae_kv_off(int e) { return (e >> 4) * 32 + ((e & 15) >> 2) * 8 + (e & 3); }
#endif

#endif  // AE_DEVICE_H
