// Matrix-pipe ceiling probe: nothing but mfma_f32_32x32x16_f16 in a loop, with clock stamps.
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
// Configuration ("ae_config.h", may be empty): AE_PROBE_WAVES_PER_SIMD (1 or 2) waves per SIMD; AE_PROBE_EXTRA_VALU independent v_fma_f32 per MFMA
// interleaved into the loop (0 by default: the pure matrix ceiling).
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

typedef _Float16 ae_probe_half8 __attribute__((ext_vector_type(8)));
typedef float ae_probe_f32x16 __attribute__((ext_vector_type(16)));

struct ae_mfma_probe_params {
  const _Float16* src;            // operand pool, n_src elements (a power of two, at least 32768)
  float* sink;                    // never written in practice (keeps the accumulators alive)
  unsigned long long* stamps;     // [gridDim.x][2]: shader-clock cycles, 100 MHz ticks of the loop
  unsigned n_src;
  int iters;                      // loop trips; one trip = 32 MFMAs per wave
};

extern "C" __global__ __launch_bounds__(256 * AE_PROBE_WAVES_PER_SIMD)
__attribute__((amdgpu_waves_per_eu(AE_PROBE_WAVES_PER_SIMD, AE_PROBE_WAVES_PER_SIMD)))
void ae_mfma_probe_kernel(const ae_mfma_probe_params p) {
  const unsigned tid = threadIdx.x;
  // four A and four B fragments per lane, each lane and workgroup at its own place of the pool
  ae_probe_half8 a[4], b[4];
  const unsigned base = (blockIdx.x * 8191u + tid * 64u) & (p.n_src - 1);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    a[i] = *(const ae_probe_half8*)(p.src + ((base + i * 8) & (p.n_src - 8)));
    b[i] = *(const ae_probe_half8*)(p.src + ((base + 32 + i * 8) & (p.n_src - 8)));
  }
  ae_probe_f32x16 c[8];
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) c[i][r] = 0.f;
#if AE_PROBE_EXTRA_VALU
  float x[8];
#pragma unroll
  for (int i = 0; i < 8; i++) x[i] = (float)a[i & 3][i];
#endif
  // the operands have arrived before the first stamp is taken
#pragma unroll
  for (int i = 0; i < 4; i++) asm volatile("" : "+v"(a[i]), "+v"(b[i]));
  __syncthreads();
  const unsigned long long t0 = __builtin_amdgcn_s_memtime();
  const unsigned long long w0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < p.iters; it++) {
#pragma unroll
    for (int j = 0; j < 32; j++) {
      c[j & 7] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j & 3], b[(j >> 2) & 3], c[j & 7], 0, 0, 0);
#if AE_PROBE_EXTRA_VALU
#pragma unroll
      for (int e = 0; e < AE_PROBE_EXTRA_VALU; e++)
        x[(j + e) & 7] = __builtin_fmaf(x[(j + e) & 7], 0.999f, 0.001f);
      __builtin_amdgcn_sched_barrier(0);      // keep the arithmetic between the MFMAs, where a kernel has it
#endif
    }
  }
  const unsigned long long t1 = __builtin_amdgcn_s_memtime();
  const unsigned long long w1 = __builtin_amdgcn_s_memrealtime();
  if (tid == 0) {
    p.stamps[2 * blockIdx.x] = t1 - t0;
    p.stamps[2 * blockIdx.x + 1] = w1 - w0;
  }
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) acc += c[i][tid & 15];
#if AE_PROBE_EXTRA_VALU
#pragma unroll
  for (int i = 0; i < 8; i++) acc += x[i];
#endif
  if (acc == 1.2345678f) p.sink[tid] = acc;     // practically never: the results only have to be "used"
}
