// Matrix-pipe ceiling probe: nothing but MFMAs in a loop (optionally with the least other work a flash
// attention loop needs per MFMA), with clock stamps.
//
// It exists to put a measured number next to the published dense fp16 peak of the chip: the rate a wave
// per SIMD reaches when it issues MFMAs back to back with no memory traffic, no LDS traffic and no other
// arithmetic, and the shader clock the chip granted while it did.  The operands come from memory once, so
// the SAME code object runs on all-zero operands and on random ones; any difference between the two runs
// is the chip's power management reacting to the data the matrix pipe sees, not the program.
//
// Every workgroup reports two counter differences taken around its loop: shader-clock cycles (s_memtime)
// and constant-rate ticks (s_memrealtime, 100 MHz).  Their ratio is the shader clock during the loop.
//
// Configuration ("ae_config.h", may be empty):
//   AE_PROBE_WAVES_PER_SIMD  1 or 2 waves per SIMD (one: the accumulators sit in the accumulator file; two: each wave has
//                            256 registers and the compiler picks the form of the MFMA whose accumulators are ordinary
//                            registers -- the rates of the two forms do not differ)
//   AE_PROBE_BF16            1: bf16 operands (the pool is read as bf16), else fp16
//   AE_PROBE_M16             1: the 16x16x32 shape, two MFMAs where the other builds have one 32x32x16 (same flops,
//                            half the accumulator registers read and written per flop, twice the operand registers)
//   AE_PROBE_EXTRA_VALU      independent v_fma_f32 per MFMA, issued between the MFMAs (0: the pure ceiling)
//   AE_PROBE_EXP             v_exp_f32 per MFMA, likewise
//   AE_PROBE_LDS             1: every second MFMA takes a fresh A fragment (1 KiB per wave) from LDS, read two
//                            fragments ahead - the LDS traffic of a kernel whose every fragment feeds two MFMAs;
//                            2: every 32768 flop take one (a wave of 32 rows: a fragment feeds one 32x32x16 or two 16x16x32)
//   AE_PROBE_SKELETON        1 (with AE_PROBE_EXP 1, AE_PROBE_LDS 1): what a kernel's loop cannot avoid on top of the mix --
//                            the exponentials take MFMA RESULTS (read out of the accumulators) and their packed
//                            results become B operands of later MFMAs, each accumulator starts from zero every trip
//                            (chains of four MFMAs, values stay bounded), and every trip (32 MFMAs) each wave requests
//                            4 KiB of the pool straight into LDS, waits for it and meets the workgroup's barrier: the
//                            tile traffic of a 256-row q tile with 64-key tiles at head dim 128
// A flash attention forward at head dim 128 spends one 32x32x16 MFMA per 64 scores, i.e. per score and lane:
// one exponential, a maximum, a sum and half a packed conversion at the very least, and half a fragment read.
// AE_PROBE_EXTRA_VALU 2 + AE_PROBE_EXP 1 (an exponential and the v_fma that consumes it) + AE_PROBE_LDS 1 is that
// mix - three plain VALU instructions, one transcendental and half a fragment read per MFMA - with nothing else
// around it: no accumulator read-outs, no tile loads, no barriers, no masks.
#ifndef __HIPCC_RTC__
#include <hip/hip_runtime.h>
#endif
#include "ae_config.h"

#ifndef AE_PROBE_WAVES_PER_SIMD
#define AE_PROBE_WAVES_PER_SIMD 1
#endif
#ifndef AE_PROBE_EXTRA_VALU
#define AE_PROBE_EXTRA_VALU 0
#endif
#ifndef AE_PROBE_EXP
#define AE_PROBE_EXP 0
#endif
#ifndef AE_PROBE_LDS
#define AE_PROBE_LDS 0
#endif
#ifndef AE_PROBE_BF16
#define AE_PROBE_BF16 0
#endif
#ifndef AE_PROBE_M16
#define AE_PROBE_M16 0
#endif
#ifndef AE_PROBE_SKELETON
#define AE_PROBE_SKELETON 0
#endif
#define AE_PROBE_NACC 8   // accumulator tuples the MFMAs rotate over

#if AE_PROBE_BF16
typedef __bf16 ae_probe_elem;
#else
typedef _Float16 ae_probe_elem;
#endif
typedef ae_probe_elem ae_probe_half8 __attribute__((ext_vector_type(8)));
typedef float ae_probe_f32x16 __attribute__((ext_vector_type(16)));

struct ae_mfma_probe_params {
  const void* src;                // operand pool, n_src 16-bit elements (a power of two, at least 32768)
  float* sink;                    // never written in practice (keeps the results alive)
  unsigned long long* stamps;     // [gridDim.x][2]: shader-clock cycles, 100 MHz ticks of the loop
  unsigned n_src;
  int iters;                      // loop trips; one trip = 32 MFMAs per wave
};

__device__ __attribute__((always_inline)) inline ae_probe_f32x16 ae_probe_mfma(const int QP, ae_probe_half8 a, ae_probe_half8 b, ae_probe_half8 b2,
                                                                              ae_probe_f32x16 c) {
#if AE_PROBE_M16
  // two 16x16x32 MFMAs on registers 8 QP .. 8 QP + 7 of the accumulator tuple
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  f32x4 lo = {c[8 * QP], c[8 * QP + 1], c[8 * QP + 2], c[8 * QP + 3]}, hi = {c[8 * QP + 4], c[8 * QP + 5], c[8 * QP + 6], c[8 * QP + 7]};
#if AE_PROBE_BF16
  lo = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, lo, 0, 0, 0);
  hi = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b2, hi, 0, 0, 0);
#else
  lo = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, lo, 0, 0, 0);
  hi = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b2, hi, 0, 0, 0);
#endif
#pragma unroll
  for (int i = 0; i < 4; i++) c[8 * QP + i] = lo[i], c[8 * QP + 4 + i] = hi[i];
  return c;
#elif AE_PROBE_BF16
  (void)QP, (void)b2;
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
#else
  (void)QP, (void)b2;
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
#endif
}

extern "C" __global__ __launch_bounds__(256 * AE_PROBE_WAVES_PER_SIMD)
__attribute__((amdgpu_waves_per_eu(AE_PROBE_WAVES_PER_SIMD, AE_PROBE_WAVES_PER_SIMD)))
void ae_mfma_probe_kernel(const ae_mfma_probe_params p) {
  const unsigned tid = threadIdx.x;
  const ae_probe_elem* src = (const ae_probe_elem*)p.src;
  // four A and four B fragments per lane, each lane and workgroup at its own place of the pool
  ae_probe_half8 a[4], b[4];
  const unsigned base = (blockIdx.x * 8191u + tid * 64u) & (p.n_src - 1);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    a[i] = *(const ae_probe_half8*)(src + ((base + i * 8) & (p.n_src - 8)));
    b[i] = *(const ae_probe_half8*)(src + ((base + 32 + i * 8) & (p.n_src - 8)));
  }
#if AE_PROBE_LDS
  // 16 fragments of pool data per wave in LDS (16 KiB a wave), lane-contiguous 16-byte pieces: conflict-free reads
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[4 * AE_PROBE_WAVES_PER_SIMD * (16 + 4 * AE_PROBE_SKELETON) * 1024];
  typedef __attribute__((address_space(3))) ae_probe_half8 lds_frag;
  lds_frag* mine = (lds_frag*)((__attribute__((address_space(3))) unsigned char*)lds_raw) + (tid >> 6) * 16 * 64 + (tid & 63);
#pragma unroll
  for (int f = 0; f < 16; f++)
    mine[f * 64] = *(const ae_probe_half8*)(src + ((base + 4096 + f * 520) & (p.n_src - 8)));
#endif
  ae_probe_f32x16 c[AE_PROBE_NACC];
#pragma unroll
  for (int i = 0; i < AE_PROBE_NACC; i++) {
#pragma unroll
    for (int r = 0; r < 16; r++) c[i][r] = 0.f;
  }
#if AE_PROBE_EXTRA_VALU || AE_PROBE_EXP
  float x[8];
#pragma unroll
  for (int i = 0; i < 8; i++) x[i] = (float)a[i & 3][i] * 0.25f;
#endif
  // the operands have arrived before the first stamp is taken
#pragma unroll
  for (int i = 0; i < 4; i++) asm volatile("" : "+v"(a[i]), "+v"(b[i]));
  __syncthreads();
  const unsigned long long t0 = __builtin_amdgcn_s_memtime();
  const unsigned long long w0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < p.iters; it++) {
#if AE_PROBE_SKELETON
    {
      // this trip's "tile": four direct loads of 1 KiB per wave behind one write of M0, into the wave's staging area
      // behind the fragments (the data are never read: the fragments above stand for them)
      const unsigned m0v = __builtin_amdgcn_readfirstlane(
          (unsigned)(unsigned long)((__attribute__((address_space(3))) unsigned char*)lds_raw) +
          4u * AE_PROBE_WAVES_PER_SIMD * 16u * 1024u + (tid >> 6) * 4096u);
      const char* gsrc = (const char*)src + (((blockIdx.x * 4099u + (unsigned)it * 64u + tid) * 16u) & (p.n_src * 2u - 4096u - 16u));
      asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\t"
                   "global_load_lds_dwordx4 %0, off\n\tglobal_load_lds_dwordx4 %0, off offset:1024\n\t"
                   "global_load_lds_dwordx4 %0, off offset:2048\n\tglobal_load_lds_dwordx4 %0, off offset:3072"
                   : : "v"(gsrc), "s"(m0v) : "memory");
    }
#endif
#pragma unroll
    for (int j = 0; j < 32; j++) {
#if AE_PROBE_SKELETON
      if (j < AE_PROBE_NACC) {
#pragma unroll
        for (int r = 0; r < 16; r++) c[j][r] = 0.f;      // (folds into the MFMA's C operand)
      }
#endif
#if AE_PROBE_LDS
#if AE_PROBE_LDS == 2
      // a fresh fragment for every slot, read two slots ahead (a[] is a ring of four)
      a[(j + 2) & 3] = mine[(j & 15) * 64];
      c[j % AE_PROBE_NACC] = ae_probe_mfma((j / AE_PROBE_NACC) & 1, a[j & 3], b[j & 3], b[(j + 1) & 3], c[j % AE_PROBE_NACC]);
#else
      // fragment for the MFMAs j + 4, j + 5 (a[] is a ring of four: one in use, two on their way)
      if ((j & 1) == 0) a[((j >> 1) + 2) & 3] = mine[((j >> 1) & 15) * 64];
      c[j % AE_PROBE_NACC] = ae_probe_mfma((j / AE_PROBE_NACC) & 1, a[(j >> 1) & 3], b[j & 3], b[(j + 1) & 3], c[j % AE_PROBE_NACC]);
#endif
#else
      c[j % AE_PROBE_NACC] = ae_probe_mfma((j / AE_PROBE_NACC) & 1, a[j & 3], b[(j >> 2) & 3], b[((j >> 2) + 1) & 3], c[j % AE_PROBE_NACC]);
#endif
#if AE_PROBE_EXTRA_VALU
#pragma unroll
      for (int e = 0; e < AE_PROBE_EXTRA_VALU; e++)
        x[(j + e) & 7] = __builtin_fmaf(x[(j + e) & 7], 0.999f, 0.001f);
#endif
#if AE_PROBE_EXP && AE_PROBE_SKELETON
      {
        // a result of the MFMA issued four slots ago -> exponent -> packed into a B operand used four slots on
        const float sres = c[(j + 4) % AE_PROBE_NACC][j & 15];
        const float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(sres, 0.125f, -4.0f));
        b[(j + 2) & 3][j & 7] = (ae_probe_elem)pe;
      }
#elif AE_PROBE_EXP
#pragma unroll
      for (int e = 0; e < AE_PROBE_EXP; e++)
        x[(j + 4 + e) & 7] = __builtin_amdgcn_exp2f(x[(j + 4 + e) & 7]) * 0.5f - 0.75f;   // stays in (-0.75, 0.1)
#endif
#if AE_PROBE_EXTRA_VALU || AE_PROBE_EXP || AE_PROBE_LDS
      __builtin_amdgcn_sched_barrier(0);      // keep the other work between the MFMAs, where a kernel has it
#endif
    }
#if AE_PROBE_SKELETON
    __builtin_amdgcn_s_waitcnt(0x0070 | 0x0f00);      // vmcnt(0): the tile has landed
    __syncthreads();
#endif
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memtime();
  const unsigned long long w1 = __builtin_amdgcn_s_memrealtime();
  if (tid == 0) {
    p.stamps[2 * blockIdx.x] = t1 - t0;
    p.stamps[2 * blockIdx.x + 1] = w1 - w0;
  }
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < AE_PROBE_NACC; i++) acc += c[i][tid & 15];
#if AE_PROBE_EXTRA_VALU || AE_PROBE_EXP
#pragma unroll
  for (int i = 0; i < 8; i++) acc += x[i];
#endif
  if (acc == 1.2345678f) p.sink[tid] = acc;     // practically never: the results only have to be "used"
}
