// ae_decode_fwd_noalloc: the GQA split-KV decode launch for callers that cannot allocate.
//
// ae_decode_fwd (ae_hip.cpp) takes its split-KV work buffers -- fp32 partial outputs and partial row
// scales -- from the caller.  Code under HIP graph capture, tight serving loops and harnesses that
// forbid hipMalloc cannot provide them per call, so this entry point runs the same two kernels on a
// work buffer that lives in the library's own device image: a file-scope __device__ array of fixed size,
// one copy per GPU, resident from the moment the library's code object is loaded on that GPU until the
// process ends.  The array's name is only a host-side handle; its device address is looked up once per
// device with hipGetSymbolAddress and everything after that uses the address.
//
// Built with hipcc (this is the one translation unit of the library that carries device data).

#include <hip/hip_runtime.h>

#include <mutex>

#include "ae_hip.h"

// 16 MiB (AE_NOALLOC_SCRATCH_BYTES): the decode of B64 Hq32 Hkv8 Skv8192 D128 plans 4 partials per head
// and needs 4.2 MB; the array holds up to 32.5k (batch, head, split) rows of 128 columns.
// (No `used` attribute: the compiler gives a static device variable that host code names a global
// device-side symbol, which is what hipGetSymbolAddress looks up; marked `used` it stays a local symbol
// and the runtime's lookup by name aborts the process.)
static __device__ __align__(256) unsigned char scratch[AE_NOALLOC_SCRATCH_BYTES];

// defined in ae_hip.cpp: sets the calling thread's ae_last_error text and returns `code`
extern "C" __attribute__((visibility("hidden"))) int ae_internal_fail(int code, const char* fmt, ...);
// defined in ae_hip.cpp: every argument check of ae_decode_fwd, no launch
extern "C" __attribute__((visibility("hidden"))) int ae_internal_decode_check(
    ae_kernel* split, ae_kernel* combine, const ae_attn_params* p, const ae_tile_cfg* cfg,
    const ae_tile_cfg* combine_cfg);

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_lock;
unsigned char* g_scratch_ptr[kMaxDevices] = {};   // device address of `scratch` on each GPU, 0 = not looked up

// Device address of this GPU's copy of `scratch` (looked up on the first call per device, with that
// device current -- the caller's current device is the one its kernels were loaded on).
int scratch_address(unsigned char** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return ae_internal_fail(AE_ERR_HIP, "ae_decode_fwd_noalloc: hipGetDevice failed: %s (%d)", hipGetErrorString(e), (int)e);
  if (dev < 0 || dev >= kMaxDevices)
    return ae_internal_fail(AE_ERR_INVALID_ARG, "ae_decode_fwd_noalloc: device %d out of range", dev);
  std::lock_guard<std::mutex> g(g_lock);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return ae_internal_fail(AE_ERR_HIP, "ae_decode_fwd_noalloc: hipGetSymbolAddress(scratch) on device %d failed: %s (%d)",
                              dev, hipGetErrorString(e), (int)e);
    g_scratch_ptr[dev] = (unsigned char*)ptr;
  }
  *out = g_scratch_ptr[dev];
  return AE_OK;
}

}  // namespace

extern "C" int ae_decode_fwd_noalloc(ae_kernel* split, ae_kernel* combine, const ae_attn_params* p,
                                     const ae_tile_cfg* cfg, const ae_tile_cfg* combine_cfg, void* stream) {
  if (!p || !cfg)
    return ae_internal_fail(AE_ERR_INVALID_ARG, "ae_decode_fwd_noalloc: params/cfg is NULL");
  if (p->batch <= 0 || p->heads_q <= 0 || p->num_splits <= 0 || cfg->head_dim_v <= 0 || cfg->n_rowscales < 0)
    return ae_internal_fail(AE_ERR_INVALID_ARG, "ae_decode_fwd_noalloc: bad extents (B=%d Hq=%d splits=%d DV=%d)",
                            p->batch, p->heads_q, p->num_splits, cfg->head_dim_v);
  // a kernel whose last workgroup merges counts arrivals in counters that must read zero when it starts; the
  // built-in buffer keeps whatever the last call left and is not cleared here
  if (cfg->merge_in_wg == 2)
    return ae_internal_fail(AE_ERR_INVALID_ARG, "ae_decode_fwd_noalloc: a split kernel whose last workgroup merges "
                            "(merge_in_wg=2) needs zeroed arrival counters: launch it through ae_decode_fwd");
  // layout inside the array: partial_o fp32 [B,Hq,splits,DV], then (256-byte aligned) partial_rs fp32
  // [max(1, n_rowscales),B,Hq,splits] -- the shapes ae_decode_fwd documents for the caller's buffers
  const uint64_t rows = (uint64_t)p->batch * (uint64_t)p->heads_q * (uint64_t)p->num_splits;
  const uint64_t o_bytes = (rows * (uint64_t)cfg->head_dim_v * 4 + 255) & ~(uint64_t)255;
  const uint64_t rs_bytes = rows * (uint64_t)(cfg->n_rowscales > 0 ? cfg->n_rowscales : 1) * 4;
  if (o_bytes + rs_bytes > (uint64_t)AE_NOALLOC_SCRATCH_BYTES)
    return ae_internal_fail(AE_ERR_INVALID_ARG,
                            "ae_decode_fwd_noalloc: B=%d Hq=%d splits=%d DV=%d needs %llu bytes of split-KV work space, "
                            "the built-in buffer holds %llu (use ae_decode_fwd with caller-allocated buffers)",
                            p->batch, p->heads_q, p->num_splits, cfg->head_dim_v,
                            (unsigned long long)(o_bytes + rs_bytes), (unsigned long long)AE_NOALLOC_SCRATCH_BYTES);
  // every check of ae_decode_fwd runs before the device is touched (the work buffers stand in as non-NULL
  // placeholders: a split kernel that merges in its workgroup ignores them, any other needs them)
  ae_attn_params q = *p;
  q.partial_o = (float*)(uintptr_t)256;
  q.partial_rs = (float*)(uintptr_t)256;
  int rc = ae_internal_decode_check(split, combine, &q, cfg, combine_cfg);
  if (rc) return rc;
  unsigned char* base = nullptr;
  rc = scratch_address(&base);
  if (rc) return rc;
  q.partial_o = (float*)base;
  q.partial_rs = (float*)(base + o_bytes);
  // Nothing has to start at zero: every wave of the split kernel writes its partial and its row scales in
  // full, and the merge kernel reads exactly those.  What the previous call left behind is overwritten.
  return ae_decode_fwd(split, combine, &q, cfg, combine_cfg, stream);
}
