// Plain device-to-device copy of a known size.  It exists to calibrate hardware counters: the
// ratio between what a memory counter reports for this kernel and the bytes it is known to move
// turns the same counter's reading for an attention kernel into bytes.
#ifndef __HIPCC_RTC__
#include <hip/hip_runtime.h>
#endif

struct ae_copy_params {
  const uint4* src;
  uint4* dst;
  unsigned long long n_vec;   // number of 16-byte elements
};

extern "C" __global__ void __launch_bounds__(256) ae_copy_probe_kernel(const ae_copy_params p) {
  const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
  for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < p.n_vec; i += stride)
    p.dst[i] = p.src[i];
}
