// libae_hip.so: hipRTC compile + code-object cache + checked launches behind a C ABI.
// Declarations and the reference interfaces they stand in for: include/ae_hip.h.
//
// Host-only translation unit (built with g++ or hipcc); links libamdhip64 + libhiprtc.  The library's
// second translation unit, ae_noalloc.hip, carries its one piece of device data.

#include <cstdint>
#include "ae_hip.h"

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <unistd.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace {

thread_local std::string g_last_error;
std::mutex g_mutex;  // guards compilation and module load/unload

int fail(int code, const char* fmt, ...) {
  char buf[4096];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

int fail_str(int code, const std::string& s) {
  g_last_error = s;
  return code;
}

#define AE_HIP_TRY(expr)                                                           \
  do {                                                                             \
    hipError_t e_ = (expr);                                                        \
    if (e_ != hipSuccess)                                                          \
      return fail(AE_ERR_HIP, "%s failed: %s (%d)", #expr, hipGetErrorString(e_),  \
                  (int)e_);                                                        \
  } while (0)

}  // namespace

// the same for the library's other translation unit (ae_noalloc.hip); not part of the ABI
extern "C" __attribute__((visibility("hidden"))) int ae_internal_fail(int code, const char* fmt, ...) {
  char buf[4096];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

struct ae_kernel {
  hipFunction_t fn = nullptr;
  int device = -1;
  std::string name;
};

struct ae_module {
  std::vector<char> code;
  std::string log;
  std::string name;
  // one loaded hipModule_t per device, created on demand
  std::map<int, hipModule_t> loaded;
  std::map<std::pair<int, std::string>, ae_kernel*> kernels;
};

struct ae_event {
  hipEvent_t ev = nullptr;
};

extern "C" {

int ae_abi_version(void) { return AE_ABI_VERSION; }

const char* ae_last_error(void) { return g_last_error.c_str(); }

int ae_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

int ae_device_info(int device, ae_devinfo* out) {
  if (!out) return fail(AE_ERR_INVALID_ARG, "ae_device_info: out is NULL");
  hipDeviceProp_t pr;
  AE_HIP_TRY(hipGetDeviceProperties(&pr, device));
  memset(out, 0, sizeof *out);
  snprintf(out->name, sizeof out->name, "%.127s", pr.name);
  snprintf(out->arch, sizeof out->arch, "%.63s", pr.gcnArchName);
  out->compute_units = pr.multiProcessorCount;
  out->clock_khz = pr.clockRate;
  out->mem_clock_khz = pr.memoryClockRate;
  out->mem_bus_bits = pr.memoryBusWidth;
  out->lds_per_block = (int32_t)pr.sharedMemPerBlock;
  out->l2_bytes = pr.l2CacheSize;
  out->wavefront_size = pr.warpSize;
  out->global_mem_bytes = pr.totalGlobalMem;
  return AE_OK;
}

int ae_compile(const char* src, const char* name, const char* arch,
               const char* const* opts, int nopts,
               const char* const* header_names, const char* const* headers, int nheaders,
               ae_module** out) {
  if (out) *out = nullptr;
  if (!src || !out) return fail(AE_ERR_INVALID_ARG, "ae_compile: src/out is NULL");
  if (nopts < 0 || nheaders < 0 || (nopts && !opts) ||
      (nheaders && (!headers || !header_names)))
    return fail(AE_ERR_INVALID_ARG, "ae_compile: bad option/header arrays");
  std::lock_guard<std::mutex> lock(g_mutex);

  hiprtcProgram prog = nullptr;
  hiprtcResult r = hiprtcCreateProgram(&prog, src, name ? name : "ae_kernel.hip", nheaders,
                                       const_cast<const char**>(headers),
                                       const_cast<const char**>(header_names));
  if (r != HIPRTC_SUCCESS)
    return fail(AE_ERR_COMPILE, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));

  std::vector<std::string> held;
  held.push_back(std::string("--offload-arch=") + (arch && *arch ? arch : "gfx950"));
  for (int i = 0; i < nopts; i++)
    if (opts[i]) held.push_back(opts[i]);
  std::vector<const char*> argv;
  for (auto& s : held) argv.push_back(s.c_str());

  r = hiprtcCompileProgram(prog, (int)argv.size(), argv.data());
  std::string log;
  size_t log_size = 0;
  if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
    log.resize(log_size);
    if (hiprtcGetProgramLog(prog, &log[0]) != HIPRTC_SUCCESS) log.clear();
    while (!log.empty() && log.back() == '\0') log.pop_back();
  }
  if (r != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    return fail_str(AE_ERR_COMPILE, std::string("hipRTC compile failed (") +
                                        hiprtcGetErrorString(r) + "):\n" + log);
  }
  size_t code_size = 0;
  r = hiprtcGetCodeSize(prog, &code_size);
  if (r != HIPRTC_SUCCESS || code_size == 0) {
    hiprtcDestroyProgram(&prog);
    return fail(AE_ERR_COMPILE, "hiprtcGetCodeSize: %s", hiprtcGetErrorString(r));
  }
  ae_module* m = new ae_module();
  m->code.resize(code_size);
  r = hiprtcGetCode(prog, m->code.data());
  hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS) {
    delete m;
    return fail(AE_ERR_COMPILE, "hiprtcGetCode: %s", hiprtcGetErrorString(r));
  }
  m->log = log;
  m->name = name ? name : "";
  *out = m;
  return AE_OK;
}

int ae_compiler_version(int* major, int* minor) {
  if (!major || !minor) return fail(AE_ERR_INVALID_ARG, "ae_compiler_version: NULL argument");
  hiprtcResult r = hiprtcVersion(major, minor);
  if (r != HIPRTC_SUCCESS)
    return fail(AE_ERR_COMPILE, "hiprtcVersion failed: %s", hiprtcGetErrorString(r));
  return AE_OK;
}

const char* ae_module_log(const ae_module* m) { return m ? m->log.c_str() : ""; }

int ae_module_code(const ae_module* m, const void** data, size_t* size) {
  if (!m || !data || !size) return fail(AE_ERR_INVALID_ARG, "ae_module_code: NULL argument");
  *data = m->code.data();
  *size = m->code.size();
  return AE_OK;
}

int ae_module_save(const ae_module* m, const char* path) {
  if (!m || !path) return fail(AE_ERR_INVALID_ARG, "ae_module_save: NULL argument");
  // write to a temporary name first so a concurrent reader never sees a torn file; the name is unique
  // per process and call, so two processes compiling the same key never write one temporary file
  static std::atomic<unsigned> counter{0};
  std::string tmp = std::string(path) + ".tmp." + std::to_string((long)getpid()) + "." +
                    std::to_string(counter.fetch_add(1));
  FILE* f = fopen(tmp.c_str(), "wb");
  if (!f) return fail(AE_ERR_IO, "ae_module_save: cannot open %s", tmp.c_str());
  size_t n = fwrite(m->code.data(), 1, m->code.size(), f);
  int rc = fclose(f);
  if (n != m->code.size() || rc != 0) {
    remove(tmp.c_str());
    return fail(AE_ERR_IO, "ae_module_save: short write to %s", tmp.c_str());
  }
  if (rename(tmp.c_str(), path) != 0) {
    remove(tmp.c_str());
    return fail(AE_ERR_IO, "ae_module_save: cannot rename to %s", path);
  }
  return AE_OK;
}

int ae_module_load(const char* path, ae_module** out) {
  if (out) *out = nullptr;
  if (!path || !out) return fail(AE_ERR_INVALID_ARG, "ae_module_load: NULL argument");
  FILE* f = fopen(path, "rb");
  if (!f) return fail(AE_ERR_IO, "ae_module_load: cannot open %s", path);
  fseek(f, 0, SEEK_END);
  long sz = ftell(f);
  fseek(f, 0, SEEK_SET);
  if (sz <= 0) {
    fclose(f);
    return fail(AE_ERR_IO, "ae_module_load: %s is empty", path);
  }
  ae_module* m = new ae_module();
  m->code.resize((size_t)sz);
  size_t n = fread(m->code.data(), 1, (size_t)sz, f);
  fclose(f);
  if (n != (size_t)sz) {
    delete m;
    return fail(AE_ERR_IO, "ae_module_load: short read from %s", path);
  }
  m->name = path;
  *out = m;
  return AE_OK;
}

void ae_module_free(ae_module* m) {
  if (!m) return;
  std::lock_guard<std::mutex> lock(g_mutex);
  for (auto& kv : m->kernels) delete kv.second;
  for (auto& kv : m->loaded) {
    if (kv.second) (void)hipModuleUnload(kv.second);
  }
  delete m;
}

int ae_module_get_kernel(ae_module* m, const char* kernel_name, ae_kernel** out) {
  if (out) *out = nullptr;
  if (!m || !kernel_name || !out)
    return fail(AE_ERR_INVALID_ARG, "ae_module_get_kernel: NULL argument");
  std::lock_guard<std::mutex> lock(g_mutex);
  int dev = -1;
  AE_HIP_TRY(hipGetDevice(&dev));
  auto key = std::make_pair(dev, std::string(kernel_name));
  auto it = m->kernels.find(key);
  if (it != m->kernels.end()) {
    *out = it->second;
    return AE_OK;
  }
  hipModule_t mod = nullptr;
  auto lit = m->loaded.find(dev);
  if (lit == m->loaded.end()) {
    AE_HIP_TRY(hipModuleLoadData(&mod, m->code.data()));
    m->loaded[dev] = mod;
  } else {
    mod = lit->second;
  }
  hipFunction_t fn = nullptr;
  hipError_t e = hipModuleGetFunction(&fn, mod, kernel_name);
  if (e != hipSuccess || !fn)
    return fail(AE_ERR_NOT_FOUND, "kernel '%s' not found in module '%s': %s", kernel_name,
                m->name.c_str(), hipGetErrorString(e));
  ae_kernel* k = new ae_kernel();
  k->fn = fn;
  k->device = dev;
  k->name = kernel_name;
  m->kernels[key] = k;
  *out = k;
  return AE_OK;
}

int ae_launch(ae_kernel* k, const void* params, size_t params_bytes, const uint32_t grid[3],
              const uint32_t block[3], uint32_t lds_bytes, void* stream) {
  if (!k || !k->fn || !grid || !block)
    return fail(AE_ERR_INVALID_ARG, "ae_launch: NULL kernel/grid/block");
  if (params_bytes && !params) return fail(AE_ERR_INVALID_ARG, "ae_launch: params is NULL");
  for (int i = 0; i < 3; i++)
    if (grid[i] == 0 || block[i] == 0)
      return fail(AE_ERR_INVALID_ARG, "ae_launch: zero grid/block extent");
  uint64_t threads = (uint64_t)block[0] * block[1] * block[2];
  if (threads > 1024) return fail(AE_ERR_INVALID_ARG, "ae_launch: %llu threads per block",
                                  (unsigned long long)threads);
  if (lds_bytes > 160u * 1024u)
    return fail(AE_ERR_INVALID_ARG, "ae_launch: %u bytes of LDS exceed 160 KiB", lds_bytes);
  size_t size = params_bytes;
  void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void*>(params),
                    HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
  AE_HIP_TRY(hipModuleLaunchKernel(k->fn, grid[0], grid[1], grid[2], block[0], block[1],
                                   block[2], lds_bytes, (hipStream_t)stream, nullptr,
                                   params_bytes ? config : nullptr));
  return AE_OK;
}

static int check_common(const char* who, const ae_attn_params* p, const ae_tile_cfg* cfg, bool paged_ok = false) {
  if (!p || !cfg) return fail(AE_ERR_INVALID_ARG, "%s: params/cfg is NULL", who);
  if (!p->q || !p->k || !p->v || !p->out)
    return fail(AE_ERR_INVALID_ARG, "%s: q/k/v/out pointer is NULL", who);
  if (p->batch <= 0 || p->heads_q <= 0 || p->heads_kv <= 0 || p->seqlen_q <= 0 ||
      p->seqlen_kv <= 0)
    return fail(AE_ERR_INVALID_ARG, "%s: non-positive extent (B=%d Hq=%d Hkv=%d Sq=%d Skv=%d)",
                who, p->batch, p->heads_q, p->heads_kv, p->seqlen_q, p->seqlen_kv);
  if (p->heads_q % p->heads_kv != 0)
    return fail(AE_ERR_INVALID_ARG, "%s: Hq=%d is not a multiple of Hkv=%d", who, p->heads_q,
                p->heads_kv);
  if (cfg->block_m <= 0 || cfg->block_n <= 0 || cfg->threads <= 0 || cfg->threads % 64 != 0 ||
      cfg->threads > 1024 || cfg->lds_bytes < 0 || cfg->lds_bytes > 160 * 1024)
    return fail(AE_ERR_INVALID_ARG, "%s: bad tile configuration (bm=%d bn=%d threads=%d lds=%d)",
                who, cfg->block_m, cfg->block_n, cfg->threads, cfg->lds_bytes);
  if (cfg->n_rowscales < 0 || cfg->n_rowscales > AE_MAX_ROWSCALES)
    return fail(AE_ERR_INVALID_ARG, "%s: n_rowscales=%d out of range", who, cfg->n_rowscales);
  // only ae_mla_decode_fwd knows the paged cache (and checks the table's geometry itself)
  if (!paged_ok && (cfg->paged || p->block_table || p->seqlens_k))
    return fail(AE_ERR_INVALID_ARG, "%s: a block table / per-entry lengths were passed to a launch that reads a dense cache", who);
  if (cfg->mask_mode == 2) {
    if (!p->block_mask) return fail(AE_ERR_INVALID_ARG, "%s: block-mask kernel without a mask", who);
    if (p->mask_block_m <= 0 || p->mask_block_n <= 0 || p->mask_nq <= 0 || p->mask_nkv <= 0)
      return fail(AE_ERR_INVALID_ARG, "%s: bad block-mask geometry", who);
    if ((p->mask_b != 1 && p->mask_b != p->batch) || (p->mask_h != 1 && p->mask_h != p->heads_q))
      return fail(AE_ERR_INVALID_ARG, "%s: block-mask batch/head extent (%d,%d) must be 1 or (B,Hq)",
                  who, p->mask_b, p->mask_h);
    if ((int64_t)p->mask_nq * p->mask_block_m < p->seqlen_q ||
        (int64_t)p->mask_nkv * p->mask_block_n < p->seqlen_kv)
      return fail(AE_ERR_INVALID_ARG, "%s: block mask [%d x %d] of %dx%d blocks does not cover %d x %d",
                  who, p->mask_nq, p->mask_nkv, p->mask_block_m, p->mask_block_n, p->seqlen_q,
                  p->seqlen_kv);
  }
  // the kernels move 16-byte pieces of rows: every tensor starts on a 16-byte boundary and its batch / position /
  // head strides are multiples of 8 elements (the last dimension is dense)
  const void* ptrs[] = {p->q, p->k, p->v, p->out, p->q2, p->k2};
  for (const void* ptr : ptrs)
    if (ptr && ((uintptr_t)ptr & 15) != 0)
      return fail(AE_ERR_INVALID_ARG, "%s: q / k / v / out must start on a 16-byte boundary", who);
  const int64_t strides[] = {p->q_stride_b, p->q_stride_s, p->q_stride_h, p->k_stride_b, p->k_stride_s, p->k_stride_h,
                             p->v_stride_b, p->v_stride_s, p->v_stride_h, p->o_stride_b, p->o_stride_s, p->o_stride_h,
                             p->q2 ? p->q2_stride_b : 0, p->q2 ? p->q2_stride_s : 0, p->q2 ? p->q2_stride_h : 0,
                             p->k2 ? p->k2_stride_b : 0, p->k2 ? p->k2_stride_s : 0, p->k2 ? p->k2_stride_h : 0};
  for (int64_t st : strides)
    if (st % 8 != 0)
      return fail(AE_ERR_INVALID_ARG, "%s: a stride of %lld elements is not a multiple of 8 (rows are moved 16 bytes at a time)",
                  who, (long long)st);
  return AE_OK;
}

// mask_mode 2: the block table's geometry against the kernel's tiles (shared by ae_prefill_fwd and
// ae_prefill_split_fwd)
static int check_block_table_geometry(const char* who, const ae_attn_params* p, const ae_tile_cfg* cfg) {
  if (cfg->mask_mode != 2) return AE_OK;
  if (cfg->block_m % p->mask_block_m != 0 && p->mask_block_m % cfg->block_m != 0)
    return fail(AE_ERR_INVALID_ARG, "%s: mask block rows %d incompatible with tile %d", who,
                p->mask_block_m, cfg->block_m);
  // a kv tile must lie inside ONE column of the table: the kernels classify a tile by the column of its
  // first key
  if (p->mask_block_n % cfg->block_n != 0)
    return fail(AE_ERR_INVALID_ARG, "%s: block-mask columns of %d keys are not a multiple of the %d-key kv tile",
                who, p->mask_block_n, cfg->block_n);
  // a q tile spans ceil(block_m / mask_block_m) table rows; the kernel keeps masks for the AE_TT_ROWS it was
  // compiled with and would apply the last of them to every further row
  if (cfg->table_rows < 0)
    return fail(AE_ERR_INVALID_ARG, "%s: table_rows=%d", who, cfg->table_rows);
  const int compiled_rows = cfg->table_rows ? cfg->table_rows : 8;
  const int spanned = (cfg->block_m + p->mask_block_m - 1) / p->mask_block_m;
  if (spanned > compiled_rows)
    return fail(AE_ERR_INVALID_ARG, "%s: a %d-row q tile spans %d rows of a table with %d-row blocks, the kernel was "
                "compiled for %d", who, cfg->block_m, spanned, p->mask_block_m, compiled_rows);
  return AE_OK;
}

int ae_prefill_fwd(ae_kernel* k, const ae_attn_params* p, const ae_tile_cfg* cfg, void* stream) {
  if (!k) return fail(AE_ERR_INVALID_ARG, "ae_prefill_fwd: kernel is NULL");
  int rc = check_common("ae_prefill_fwd", p, cfg);
  if (rc) return rc;
  for (int i = 0; i < cfg->n_rowscales; i++)
    if (!p->rowscale_out[i])
      return fail(AE_ERR_INVALID_ARG, "ae_prefill_fwd: rowscale_out[%d] is NULL", i);
  rc = check_block_table_geometry("ae_prefill_fwd", p, cfg);
  if (rc) return rc;
  // ids are 8*slot + xcd with slot = (batch*head / 8)*q_tiles + q_tile, see ae_prefill.hip
  uint64_t q_tiles = ((uint64_t)p->seqlen_q + cfg->block_m - 1) / cfg->block_m;
  uint64_t bh = (uint64_t)p->heads_q * (uint64_t)p->batch;
  uint64_t total = q_tiles * ((bh + 7) / 8) * 8;
  if (total == 0 || total > 0x7fffffffull)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_fwd: grid of %llu workgroups",
                (unsigned long long)total);
  uint32_t grid[3] = {(uint32_t)total, 1, 1};
  uint32_t block[3] = {(uint32_t)cfg->threads, 1, 1};
  return ae_launch(k, p, sizeof *p, grid, block, (uint32_t)cfg->lds_bytes, stream);
}

// launch == false: only the argument checks (ae_decode_fwd_noalloc runs them before it touches the device)
static int decode_fwd_impl(ae_kernel* split, ae_kernel* combine, const ae_attn_params* p,
                           const ae_tile_cfg* cfg, const ae_tile_cfg* combine_cfg, void* stream, bool launch) {
  if (!split) return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: split kernel is NULL");
  int rc = check_common("ae_decode_fwd", p, cfg);
  if (rc) return rc;
  if (p->seqlen_q != 1)
    return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: seqlen_q=%d (decode handles one query token)",
                p->seqlen_q);
  if (p->num_splits <= 0 || p->kv_per_split <= 0 ||
      (int64_t)p->num_splits * p->kv_per_split < p->seqlen_kv)
    return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: %d splits of %d do not cover Skv=%d",
                p->num_splits, p->kv_per_split, p->seqlen_kv);
  if (p->kv_per_split % cfg->block_n != 0)
    return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: kv_per_split=%d is not a multiple of block_n=%d",
                p->kv_per_split, cfg->block_n);
  // one partial per wave: a workgroup of W waves produces W consecutive partials
  int waves = cfg->threads / 64;
  // cfg->merge_in_wg: the split kernel was built with AE_MERGE_IN_WG 1 - its one workgroup per (batch, kv head,
  // head tile) merges its waves' partial results itself and writes out; no combine kernel, no work buffers.
  // The host cannot see how a kernel was compiled, so the flag travels with the tile configuration: a kernel
  // built WITHOUT the merge stores its partials through p->partial_o and must never run with NULL buffers.
  if (cfg->merge_in_wg < 0 || cfg->merge_in_wg > 2)
    return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: merge_in_wg=%d", cfg->merge_in_wg);
  // (2: built with AE_MERGE_LAST 1 - the workgroup that finishes last merges; it needs the work buffers, whose
  // row-scale buffer ends with the arrival counters, but no combine kernel)
  const bool merge_last = cfg->merge_in_wg == 2;
  if (merge_last) {
    if (combine)
      return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: a split kernel whose last workgroup merges takes no combine kernel");
    if (!p->partial_o || !p->partial_rs)
      return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: split-KV work buffers are NULL");
    // (the kernel merges exactly the AE_NSPLIT partial results it was compiled for; the host cannot see that
    // number, so it travels as it does for the merge kernel)
    if (!combine_cfg)
      return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: a split kernel whose last workgroup merges needs combine_cfg "
                  "(its block_n is the number of splits the kernel was compiled for)");
  }
  const bool merged = cfg->merge_in_wg == 1 || merge_last;
  if (merged && combine)
    return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: a split kernel that merges in the workgroup takes no combine kernel");
  if (merged && !merge_last && p->num_splits != waves)
    return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: a split kernel that merges in the workgroup needs the %d splits to be "
                "the %d waves of one workgroup", p->num_splits, waves);
  if (!merged && !combine)
    return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: combine kernel is NULL and the split kernel does not merge in the "
                "workgroup (cfg->merge_in_wg is 0)");
  if (!merged && (!p->partial_o || !p->partial_rs))
    return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: split-KV work buffers are NULL");
  if (!merged && !combine_cfg)
    return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: combine configuration is NULL");
  if (merged)     // the split kernel itself writes the merged row scales
    for (int i = 0; i < cfg->n_rowscales; i++)
      if (!p->rowscale_out[i])
        return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: rowscale_out[%d] is NULL", i);
  if (p->num_splits % waves != 0)
    return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: num_splits=%d is not a multiple of %d waves",
                p->num_splits, waves);
  if (combine_cfg && combine_cfg->block_n != p->num_splits)
    return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: combine kernel built for %d splits, got %d",
                combine_cfg->block_n, p->num_splits);
  int group = p->heads_q / p->heads_kv;
  int head_tiles = (group + cfg->block_m - 1) / cfg->block_m;
  uint32_t grid[3] = {(uint32_t)(p->num_splits / waves), (uint32_t)(head_tiles * p->heads_kv),
                      (uint32_t)p->batch};
  uint32_t block[3] = {(uint32_t)cfg->threads, 1, 1};
  if (!merged) {
    if (combine_cfg->threads <= 0 || combine_cfg->threads % 64 != 0 || combine_cfg->threads > 1024)
      return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: bad combine workgroup size %d",
                  combine_cfg->threads);
    for (int i = 0; i < combine_cfg->n_rowscales; i++)
      if (!p->rowscale_out[i])
        return fail(AE_ERR_INVALID_ARG, "ae_decode_fwd: rowscale_out[%d] is NULL", i);
  }
  if (!launch) return AE_OK;
  rc = ae_launch(split, p, sizeof *p, grid, block, (uint32_t)cfg->lds_bytes, stream);
  if (rc || merged) return rc;
  uint32_t cgrid[3] = {(uint32_t)p->heads_q, (uint32_t)p->batch, 1};
  uint32_t cblock[3] = {(uint32_t)combine_cfg->threads, 1, 1};
  return ae_launch(combine, p, sizeof *p, cgrid, cblock, (uint32_t)combine_cfg->lds_bytes, stream);
}

int ae_decode_fwd(ae_kernel* split, ae_kernel* combine, const ae_attn_params* p,
                  const ae_tile_cfg* cfg, const ae_tile_cfg* combine_cfg, void* stream) {
  return decode_fwd_impl(split, combine, p, cfg, combine_cfg, stream, true);
}

// for ae_noalloc.hip: the checks of ae_decode_fwd without the launches
extern "C" __attribute__((visibility("hidden"))) int ae_internal_decode_check(
    ae_kernel* split, ae_kernel* combine, const ae_attn_params* p, const ae_tile_cfg* cfg,
    const ae_tile_cfg* combine_cfg) {
  return decode_fwd_impl(split, combine, p, cfg, combine_cfg, nullptr, false);
}

int ae_prefill_split_fwd(ae_kernel* split, ae_kernel* combine, const ae_attn_params* p,
                         const ae_tile_cfg* cfg, const ae_tile_cfg* combine_cfg, void* stream) {
  if (!split || !combine || !combine_cfg)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_split_fwd: kernel/cfg is NULL");
  int rc = check_common("ae_prefill_split_fwd", p, cfg);
  if (rc) return rc;
  rc = check_block_table_geometry("ae_prefill_split_fwd", p, cfg);
  if (rc) return rc;
  if (p->num_splits <= 1 || p->kv_per_split <= 0 ||
      (int64_t)p->num_splits * p->kv_per_split < p->seqlen_kv)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_split_fwd: %d splits of %d do not cover Skv=%d",
                p->num_splits, p->kv_per_split, p->seqlen_kv);
  if (p->kv_per_split % cfg->block_n != 0)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_split_fwd: kv_per_split=%d is not a multiple of block_n=%d",
                p->kv_per_split, cfg->block_n);
  if (combine_cfg->block_n != p->num_splits)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_split_fwd: combine kernel built for %d splits, got %d",
                combine_cfg->block_n, p->num_splits);
  if (!p->partial_o || !p->partial_rs)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_split_fwd: split-KV work buffers are NULL");
  if (combine_cfg->threads <= 0 || combine_cfg->threads % 64 != 0 || combine_cfg->threads > 1024)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_split_fwd: bad combine workgroup size %d",
                combine_cfg->threads);
  for (int i = 0; i < combine_cfg->n_rowscales; i++)
    if (!p->rowscale_out[i])
      return fail(AE_ERR_INVALID_ARG, "ae_prefill_split_fwd: rowscale_out[%d] is NULL", i);
  if (p->o_stride_h != cfg->head_dim_v || p->o_stride_s != (int64_t)p->heads_q * cfg->head_dim_v ||
      p->o_stride_b != (int64_t)p->seqlen_q * p->heads_q * cfg->head_dim_v)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_split_fwd: out must be contiguous [B,Sq,Hq,DV]");
  uint64_t q_tiles = ((uint64_t)p->seqlen_q + cfg->block_m - 1) / cfg->block_m;
  uint64_t bh = (uint64_t)p->heads_q * (uint64_t)p->batch;
  uint64_t total = q_tiles * ((bh + 7) / 8) * 8 * (uint64_t)p->num_splits;
  uint64_t rows = (uint64_t)p->seqlen_q * (uint64_t)p->heads_q;
  if (total == 0 || total > 0x7fffffffull || rows > 0x7fffffffull)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_split_fwd: grid of %llu workgroups",
                (unsigned long long)total);
  uint32_t grid[3] = {(uint32_t)total, 1, 1};
  uint32_t block[3] = {(uint32_t)cfg->threads, 1, 1};
  rc = ae_launch(split, p, sizeof *p, grid, block, (uint32_t)cfg->lds_bytes, stream);
  if (rc) return rc;
  // the merge kernel sees the (q position, head) pairs as the heads of a one-token decode; seqlen_q stays, and
  // tells it to write the merged row scales in [B, Hq, Sq] order
  ae_attn_params cp = *p;
  cp.heads_q = (int32_t)rows;
  uint32_t cgrid[3] = {(uint32_t)rows, (uint32_t)p->batch, 1};
  uint32_t cblock[3] = {(uint32_t)combine_cfg->threads, 1, 1};
  return ae_launch(combine, &cp, sizeof cp, cgrid, cblock, (uint32_t)combine_cfg->lds_bytes, stream);
}

int ae_mla_decode_fwd(ae_kernel* split, ae_kernel* combine, const ae_attn_params* p,
                      const ae_tile_cfg* cfg, const ae_tile_cfg* combine_cfg, void* stream) {
  if (!split || !combine_cfg)
    return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: kernel/cfg is NULL");
  int rc = check_common("ae_mla_decode_fwd", p, cfg, true);
  if (rc) return rc;
  if (cfg->paged) {
    if (!p->block_table || !p->seqlens_k)
      return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: paged kernel without block_table / seqlens_k");
    if (p->page_block_size <= 0 || p->page_block_size % cfg->block_n != 0)
      return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: pages of %d tokens are not a multiple of the %d-token kv tile",
                  p->page_block_size, cfg->block_n);
    if (p->num_pages <= 0)
      return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: num_pages=%d", p->num_pages);
    if ((int64_t)p->block_table_stride * p->page_block_size < p->seqlen_kv)
      return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: %d table entries of %d tokens do not cover Skv=%d",
                  p->block_table_stride, p->page_block_size, p->seqlen_kv);
    if (p->kv_per_split % cfg->block_n != 0)
      return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: kv_per_split=%d is not a multiple of the %d-token kv tile",
                  p->kv_per_split, cfg->block_n);
    // (the wave-specialised kernel keeps a split's part of the block table in LDS: AE_PTAB = 1024 entries)
    if (p->kv_per_split / p->page_block_size + 2 > 1024)
      return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: a split of %d tokens spans more than 1022 pages of %d tokens "
                                      "(use more splits)", p->kv_per_split, p->page_block_size);
    // the paged kernels address the rope columns as an offset from the latent ones inside one cache tensor
    if (p->k2 && (p->k2_stride_b != p->k_stride_b || p->k2_stride_s != p->k_stride_s || p->k2_stride_h != p->k_stride_h ||
                  (const char*)p->k2 < (const char*)p->k || (const char*)p->k2 - (const char*)p->k > (1 << 20)))
      return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: in a paged cache k2 must be a column range of the tensor k "
                                      "(equal strides, at most 1 MiB behind it)");
  } else if (p->block_table || p->seqlens_k) {
    return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: block_table / seqlens_k passed to a kernel built for a dense cache");
  }
  // with one split the kernel writes `out` itself and no merge pass runs
  const bool direct = p->num_splits == 1;
  if (!direct && !combine)
    return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: combine kernel is NULL with %d splits",
                p->num_splits);
  if (!p->q2 || !p->k2)
    return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: rope pointers q2/k2 are NULL");
  if (p->seqlen_q != 1)
    return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: seqlen_q=%d (decode handles one query token)",
                p->seqlen_q);
  if (p->num_splits <= 0 || p->kv_per_split <= 0 ||
      (int64_t)p->num_splits * p->kv_per_split < p->seqlen_kv)
    return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: %d splits of %d do not cover Skv=%d",
                p->num_splits, p->kv_per_split, p->seqlen_kv);
  if (combine_cfg->block_n != p->num_splits)
    return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: combine kernel built for %d splits, got %d",
                combine_cfg->block_n, p->num_splits);
  if (!direct && (!p->partial_o || !p->partial_rs))
    return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: split-KV work buffers are NULL");
  if (combine_cfg->threads <= 0 || combine_cfg->threads % 64 != 0 || combine_cfg->threads > 1024)
    return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: bad combine workgroup size %d",
                combine_cfg->threads);
  for (int i = 0; i < combine_cfg->n_rowscales; i++)
    if (!p->rowscale_out[i])
      return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: rowscale_out[%d] is NULL", i);
  // 1-D grid: head tiles of one (batch, kv head, split) sit 8 ids apart (same XCD); the
  // (batch, kv head, split) count is padded to a multiple of 8, surplus workgroups exit at once.
  int group = p->heads_q / p->heads_kv;
  int64_t n_ht = (group + cfg->block_m - 1) / cfg->block_m;
  int64_t units = (int64_t)p->batch * p->heads_kv * p->num_splits;
  int64_t total = ((units + 7) / 8) * 8 * n_ht;
  if (total > 0x7fffffffll) return fail(AE_ERR_INVALID_ARG, "ae_mla_decode_fwd: grid too large");
  uint32_t grid[3] = {(uint32_t)total, 1, 1};
  uint32_t block[3] = {(uint32_t)cfg->threads, 1, 1};
  rc = ae_launch(split, p, sizeof *p, grid, block, (uint32_t)cfg->lds_bytes, stream);
  if (rc || direct) return rc;
  uint32_t cgrid[3] = {(uint32_t)p->heads_q, (uint32_t)p->batch, 1};
  uint32_t cblock[3] = {(uint32_t)combine_cfg->threads, 1, 1};
  return ae_launch(combine, p, sizeof *p, cgrid, cblock, (uint32_t)combine_cfg->lds_bytes, stream);
}

int ae_prefill_bwd(ae_kernel* delta, ae_kernel* dkv, ae_kernel* dq, const ae_attn_bwd_params* p,
                   const ae_tile_cfg* cfg, void* stream) {
  // delta == NULL: kernels built with AE_BWD_FUSE_DELTA 1 - the dq launch fills the work buffer and goes first
  if (!dkv || !dq) return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: kernel is NULL");
  if (!p || !cfg) return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: params/cfg is NULL");
  if (!p->q || !p->k || !p->v || !p->out || !p->dout || !p->delta || !p->dq || !p->dk || !p->dv)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: a tensor pointer is NULL");
  if (p->batch <= 0 || p->heads_q <= 0 || p->heads_kv <= 0 || p->seqlen_q <= 0 || p->seqlen_kv <= 0)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: non-positive extent (B=%d Hq=%d Hkv=%d Sq=%d Skv=%d)",
                p->batch, p->heads_q, p->heads_kv, p->seqlen_q, p->seqlen_kv);
  if (p->heads_q % p->heads_kv != 0)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: Hq=%d is not a multiple of Hkv=%d", p->heads_q,
                p->heads_kv);
  {
    const void* ptrs[] = {p->q, p->k, p->v, p->out, p->dout, p->dq, p->dk, p->dv};
    for (const void* ptr : ptrs)
      if (((uintptr_t)ptr & 15) != 0)
        return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: the tensors must start on a 16-byte boundary");
    const int64_t strides[] = {p->q_stride_b, p->q_stride_s, p->q_stride_h, p->k_stride_b, p->k_stride_s, p->k_stride_h,
                               p->v_stride_b, p->v_stride_s, p->v_stride_h, p->o_stride_b, p->o_stride_s, p->o_stride_h,
                               p->do_stride_b, p->do_stride_s, p->do_stride_h, p->dq_stride_b, p->dq_stride_s, p->dq_stride_h,
                               p->dk_stride_b, p->dk_stride_s, p->dk_stride_h, p->dv_stride_b, p->dv_stride_s, p->dv_stride_h};
    for (int64_t st : strides)
      if (st % 8 != 0)
        return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: a stride of %lld elements is not a multiple of 8 (rows are moved 16 bytes at a time)",
                    (long long)st);
  }
  // block_m / threads describe the dq launch (4 or 8 waves of 32 resident rows); dk/dv always runs 4 waves
  if ((cfg->block_m != 128 && cfg->block_m != 256) || cfg->block_n != 64 || cfg->threads != 2 * cfg->block_m || cfg->lds_bytes <= 0 ||
      cfg->lds_bytes > 160 * 1024 || cfg->head_dim_v <= 0 || cfg->head_dim_v % 8 != 0)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: bad tile configuration (bm=%d bn=%d threads=%d lds=%d dv=%d)",
                cfg->block_m, cfg->block_n, cfg->threads, cfg->lds_bytes, cfg->head_dim_v);
  if (cfg->mask_mode == 2) {
    if (!p->mask_dq || !p->mask_dkv)
      return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: tile-class kernels without their tables");
    if ((p->mask_b != 1 && p->mask_b != p->batch) || (p->mask_h != 1 && p->mask_h != p->heads_q))
      return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: table batch/head extent (%d,%d) must be 1 or (B,Hq)",
                  p->mask_b, p->mask_h);
    // a block mask of the user's (kernels built with AE_EXT_BLOCK_MASK 1 read it per element on partly visible tiles)
    if (p->block_mask && (p->mask_nq <= 0 || p->mask_nkv <= 0 || p->mask_block_m <= 0 || p->mask_block_n <= 0 ||
                          (int64_t)p->mask_nq * p->mask_block_m < p->seqlen_q ||
                          (int64_t)p->mask_nkv * p->mask_block_n < p->seqlen_kv))
      return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: block mask [%d x %d] of %dx%d blocks does not cover %d x %d",
                  p->mask_nq, p->mask_nkv, p->mask_block_m, p->mask_block_n, p->seqlen_q, p->seqlen_kv);
  } else if (p->block_mask) {
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: a block mask was passed to kernels built without tile-class tables");
  }
  const uint64_t rows = (uint64_t)p->batch * p->seqlen_q * p->heads_q;
  const uint64_t rows_per_wg = 256u / (uint32_t)(cfg->head_dim_v / 8);
  const uint64_t g_delta = (rows + rows_per_wg - 1) / rows_per_wg;
  // ids are 8*slot + xcd, slot = tile*ceil(batch*heads/8) + head group (see ae_prefill_bwd.hip)
  const uint64_t g_dkv = (((uint64_t)p->seqlen_kv + 127) / 128) * ((((uint64_t)p->batch * p->heads_kv) + 7) / 8) * 8;
  const uint64_t g_dq = (((uint64_t)p->seqlen_q + cfg->block_m - 1) / cfg->block_m) * ((((uint64_t)p->batch * p->heads_q) + 7) / 8) * 8;
  if (g_delta > 0x7fffffffull || g_dkv > 0x7fffffffull || g_dq > 0x7fffffffull)
    return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: grid too large");
  uint32_t block[3] = {256, 1, 1};
  uint32_t grid[3] = {(uint32_t)g_delta, 1, 1};
  int rc;
  if (!delta) {
    if (!p->lse) return fail(AE_ERR_INVALID_ARG, "ae_prefill_bwd: the dq launch forms the row scales from lse, which is NULL");
    grid[0] = (uint32_t)g_dq;
    block[0] = (uint32_t)cfg->threads;
    rc = ae_launch(dq, p, sizeof *p, grid, block, (uint32_t)cfg->lds_bytes, stream);
    if (rc) return rc;
    grid[0] = (uint32_t)g_dkv;
    block[0] = 256;
    return ae_launch(dkv, p, sizeof *p, grid, block, (uint32_t)cfg->lds_bytes, stream);
  }
  rc = ae_launch(delta, p, sizeof *p, grid, block, 0, stream);
  if (rc) return rc;
  grid[0] = (uint32_t)g_dkv;
  rc = ae_launch(dkv, p, sizeof *p, grid, block, (uint32_t)cfg->lds_bytes, stream);
  if (rc) return rc;
  grid[0] = (uint32_t)g_dq;
  block[0] = (uint32_t)cfg->threads;
  return ae_launch(dq, p, sizeof *p, grid, block, (uint32_t)cfg->lds_bytes, stream);
}

int ae_event_create(ae_event** out) {
  if (!out) return fail(AE_ERR_INVALID_ARG, "ae_event_create: out is NULL");
  *out = nullptr;
  hipEvent_t ev = nullptr;
  AE_HIP_TRY(hipEventCreate(&ev));
  ae_event* e = new ae_event();
  e->ev = ev;
  *out = e;
  return AE_OK;
}

int ae_event_record(ae_event* e, void* stream) {
  if (!e) return fail(AE_ERR_INVALID_ARG, "ae_event_record: event is NULL");
  AE_HIP_TRY(hipEventRecord(e->ev, (hipStream_t)stream));
  return AE_OK;
}

int ae_event_elapsed_ms(ae_event* start, ae_event* stop, float* ms) {
  if (!start || !stop || !ms) return fail(AE_ERR_INVALID_ARG, "ae_event_elapsed_ms: NULL argument");
  AE_HIP_TRY(hipEventSynchronize(stop->ev));
  AE_HIP_TRY(hipEventElapsedTime(ms, start->ev, stop->ev));
  return AE_OK;
}

void ae_event_destroy(ae_event* e) {
  if (!e) return;
  if (e->ev) (void)hipEventDestroy(e->ev);
  delete e;
}

}  // extern "C"
