/*
 * ae_hip.h -- C ABI of libae_hip.so, the native boundary of the MI355X (gfx950)
 * attention path (forward launches and the backward of the prefill shapes).
 *
 * What it replaces in the reference (microsoft/AttentionEngine):
 *   - the TileLang JIT boundary `tl.compile(prim_func, out_idx=[...])` that turns a
 *     rendered kernel template into a callable
 *     (attention_engine/core/template/tl_template/attn/attn_tl.py:523-528, 567-580;
 *      attn_gqa_decode_tl.py:338-349; mla_decode_tl.py:326-335), and
 *   - the pybind11 torch extensions of the CuTe backend, `fwd(...)`
 *     (core/template/cute_template/flash_api.cpp:283-467, 694-697) and
 *     `fwd_kvcache_mla(...)`
 *     (core/template/cute_template_kvshared/flash_api.cpp:61-210, 212-216).
 *
 * Conventions
 *   - plain C: pointers, sizes and PODs only; no torch, no C++ types, no exceptions.
 *   - every function returns 0 on success and a non-zero ae_status otherwise; the text
 *     of the last error of the calling thread is available from ae_last_error().
 *     Nothing in the library calls exit()/abort().
 *   - the caller owns every tensor and allocates all outputs and split-KV work
 *     buffers before a launch; device pointers are passed inside ae_attn_params
 *     together with their strides in ELEMENTS (the layout of Flash_fwd_params,
 *     core/template/cute_template/flash.h:14-60, reduced to what the forward needs).
 *     The kernels move rows 16 bytes at a time: the last dimension is dense, every
 *     tensor starts on a 16-byte boundary and every stride is a multiple of 8
 *     elements; the launch functions refuse anything else (AE_ERR_INVALID_ARG).
 *   - launches are asynchronous on the caller's HIP stream (`void* stream` is a
 *     hipStream_t; NULL is the default stream). The library never synchronises the
 *     device except inside ae_event_elapsed_ms().
 *   - compilation (ae_compile) needs no GPU: hipRTC cross-compiles for `arch`.
 *     Loading a code object onto a device happens lazily in ae_module_get_kernel().
 *   - ae_compile / ae_module_* are serialised by an internal mutex; launches take no
 *     lock and may be issued from any thread whose current device matches the one the
 *     kernel was loaded on.
 */
#ifndef AE_HIP_H
#define AE_HIP_H

/* hipRTC supplies the fixed-width integer types itself and has no libc headers. */
#ifndef __HIPCC_RTC__
#include <stddef.h>
#include <stdint.h>
#else
using __hip_internal::int8_t;
using __hip_internal::int32_t;
using __hip_internal::int64_t;
using __hip_internal::uint32_t;
using __hip_internal::uint64_t;
#endif

#ifdef __cplusplus
extern "C" {
#endif

#define AE_ABI_VERSION 6

typedef enum ae_status {
  AE_OK = 0,
  AE_ERR_INVALID_ARG = 1,   /* NULL pointer, bad size, shape/tile mismatch        */
  AE_ERR_COMPILE = 2,       /* hipRTC rejected the source; see ae_module-less log  */
  AE_ERR_HIP = 3,           /* a HIP runtime call failed (no device, load, launch) */
  AE_ERR_IO = 4,            /* code-object cache file could not be read/written    */
  AE_ERR_NOT_FOUND = 5      /* kernel symbol missing from the module               */
} ae_status;

typedef struct ae_module ae_module; /* a compiled code object (host memory)        */
typedef struct ae_kernel ae_kernel; /* a function of a module loaded on one device  */

/* Maximum counts baked into ae_attn_params. */
#define AE_MAX_ROWSCALES 4
#define AE_MAX_CUSTOM 4

/*
 * Kernel argument block shared by the prefill, split-KV decode and combine kernels.
 * Passed BY VALUE as the single kernel parameter. Runtime tensors use the reference's
 * layouts: q [B,Sq,Hq,D], k [B,Skv,Hkv,D], v [B,Skv,Hkv,DV], out [B,Sq,Hq,DV]
 * (attention_engine/attn_engine/attn_engine.py:388-395; attn_tl.py:82-84), final
 * rowscales fp32 [B,Hq,Sq] (core/lower/lower.py:385-392).
 */
typedef struct ae_attn_params {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* rowscale_out[AE_MAX_ROWSCALES]; /* final rowscales, fp32 [B,Hq,Sq]; may be NULL */
  const void* custom[AE_MAX_CUSTOM];     /* CustomIO tensors in dict order                */
  const int8_t* block_mask;              /* [mask_b,mask_h,mask_nq,mask_nkv] int8 or NULL */
  float* partial_o;                      /* decode: fp32 [B,Hq,splits,DV]                 */
  float* partial_rs;                     /* decode: fp32 [nrowscales,B,Hq,splits]         */
  const void* q2;                        /* MLA: rope part of q  [B,Sq,Hq,D2] or NULL     */
  const void* k2;                        /* MLA: rope part of k  [B,Skv,Hkv,D2] or NULL   */
  int64_t q_stride_b, q_stride_s, q_stride_h;
  int64_t k_stride_b, k_stride_s, k_stride_h;
  int64_t v_stride_b, v_stride_s, v_stride_h;
  int64_t o_stride_b, o_stride_s, o_stride_h;
  int64_t q2_stride_b, q2_stride_s, q2_stride_h;
  int64_t k2_stride_b, k2_stride_s, k2_stride_h;
  int32_t batch, heads_q, heads_kv, seqlen_q, seqlen_kv;
  int32_t mask_b, mask_h, mask_nq, mask_nkv; /* block-mask extents (mask_b/h may be 1)   */
  int32_t mask_block_m, mask_block_n;        /* rows/cols one block-mask entry covers     */
  int32_t num_splits;                        /* decode: KV splits per (batch, q-head)     */
  int32_t kv_per_split;                      /* decode: KV positions per split            */
  int32_t reserved[3];
  /* MLA decode on a paged cache (kernels whose ae_tile_cfg.paged is 1; NULL / 0 otherwise): the cache is
   * [num_pages, page_block_size, Hkv, D] (k_stride_b = elements between pages, k_stride_s between the
   * rows of a page), token t of batch entry b is row t % page_block_size of page
   * block_table[b * block_table_stride + t / page_block_size], and entry b holds
   * min(seqlens_k[b], seqlen_kv) tokens.  Stands where the reference passes block_table,
   * block_table_batch_stride, page_block_size and seqlens_k_ptr
   * (core/template/cute_template_kvshared/kernels/params.h:33-36, flash_api.cpp:61-72).
   * The latent part (k) and the rope part (k2) are column ranges of that ONE cache tensor: equal strides,
   * k2 at most 1 MiB behind k.  A split spans at most 1022 pages (kv_per_split / page_block_size + 2 <= 1024).
   * In a split launch an entry whose keys all lie in the first split writes `out` itself; splits without
   * keys write nothing and the merge reads only the splits that hold keys. */
  const int32_t* block_table;                /* int32 [B, block_table_stride]             */
  const int32_t* seqlens_k;                  /* int32 [B]                                 */
  int32_t block_table_stride;                /* entries per batch row of block_table      */
  int32_t page_block_size;                   /* tokens per page, a multiple of block_n    */
  int32_t num_pages;                         /* pages in the cache: table entries are clamped to it */
  int32_t reserved2;
} ae_attn_params;

/* Static facts of one compiled kernel instance, filled by the code generator. */
typedef struct ae_tile_cfg {
  int32_t block_m;     /* q rows per workgroup (prefill) / q-heads per workgroup (decode) */
  int32_t block_n;     /* kv positions per inner tile                                     */
  int32_t threads;     /* workgroup size, a multiple of 64                                */
  int32_t lds_bytes;   /* dynamic LDS per workgroup                                       */
  int32_t head_dim;    /* D (for MLA: latent + rope)                                      */
  int32_t head_dim_v;  /* DV                                                              */
  int32_t elem_bytes;  /* 2 for fp16/bf16                                                 */
  int32_t n_rowscales; /* number of final rowscales the kernel writes                     */
  int32_t mask_mode;   /* 0 none, 1 analytic causal, 2 block table                        */
  int32_t paged;       /* MLA decode: 1 when the kernel reads KV through block_table / seqlens_k */
  int32_t merge_in_wg; /* GQA decode: 1 when the split kernel was compiled with AE_MERGE_IN_WG 1 (its one
                          workgroup per (batch, kv head, head tile) merges its waves' partial results and
                          writes out itself: no combine kernel, no work buffers); 2 when it was compiled with
                          AE_MERGE_LAST 1 (the workgroup that finishes last merges: no combine kernel, work
                          buffers with arrival counters, see ae_decode_fwd); else 0                        */
  int32_t table_rows;  /* mask_mode 2: block-mask rows one q tile may span, the AE_TT_ROWS the kernel was
                          compiled with (1, 2, 4 or 8); 0 stands for the kernels' default of 8             */
} ae_tile_cfg;

/*
 * Kernel argument block of the backward kernels (softmax attention, prefill shapes). Same layouts as
 * ae_attn_params; dout [B,Sq,Hq,DV] is the gradient of `out`, dq/dk/dv have the shapes of q/k/v, lse
 * is the forward's natural-log row scale fp32 [B,Hq,Sq] (NULL for graphs without row scales), delta a caller-allocated fp32 [2,B,Hq,Sq]
 * work buffer (the first launch fills it: rowsum(dout * out), and lse in log2 units; [1 + AE_BWD_NRS,B,Hq,Sq] for kernels that read
 * several final row scales). Stands where the reference passes Q, K, V, dO, lse
 * and Delta to flashattn_bwd (core/template/tl_template/attn/attn_tl.py:271-295).
 */
typedef struct ae_attn_bwd_params {
  const void* q;
  const void* k;
  const void* v;
  const void* out;
  const void* dout;
  const float* lse;
  float* delta;
  void* dq;
  void* dk;
  void* dv;
  const int8_t* mask_dq;   /* mask mode 2: tile classes [mask_b,mask_h,ceil(Sq/128),ceil(Skv/64)], else NULL */
  const int8_t* mask_dkv;  /* mask mode 2: tile classes [mask_b,mask_h,ceil(Sq/64),ceil(Skv/128)], else NULL */
  const void* custom[AE_MAX_CUSTOM]; /* scalar CustomIO tensors (fp32 [1]) of score_mod, in dict order   */
  /* kernels compiled with AE_EXT_BLOCK_MASK 1 (the forward ran on a block mask the user supplied, the
   * reference's blockattn_tl.py:195-470): that mask, int8 [mask_b,mask_h,mask_nq,mask_nkv] with blocks of
   * mask_block_m x mask_block_n positions (0 = invisible); tiles of class 1 in the two tables above test
   * their elements against it.  NULL otherwise. */
  const int8_t* block_mask;
  /* kernels compiled with AE_BWD_KIND 2 and AE_BWD_NRS > 1 (an online function that hands more than one final
   * row scale to its traced forward() / backward(), the reference's core/lower/lower.py:413-453): row scales
   * 1 .. AE_BWD_NRS - 1, fp32 [B,Hq,Sq] each; `lse` carries row scale 0 and `delta` has 1 + AE_BWD_NRS planes.
   * NULL otherwise. */
  const float* more_rowscales[AE_MAX_ROWSCALES - 1];
  int64_t q_stride_b, q_stride_s, q_stride_h;
  int64_t k_stride_b, k_stride_s, k_stride_h;
  int64_t v_stride_b, v_stride_s, v_stride_h;
  int64_t o_stride_b, o_stride_s, o_stride_h;
  int64_t do_stride_b, do_stride_s, do_stride_h;
  int64_t dq_stride_b, dq_stride_s, dq_stride_h;
  int64_t dk_stride_b, dk_stride_s, dk_stride_h;
  int64_t dv_stride_b, dv_stride_s, dv_stride_h;
  int32_t batch, heads_q, heads_kv, seqlen_q, seqlen_kv;
  int32_t mask_b, mask_h;  /* batch / head extents of the two tables (and of block_mask): 1 or (B, Hq) */
  int32_t mask_nq, mask_nkv, mask_block_m, mask_block_n;  /* geometry of block_mask (0 without one)   */
  int32_t reserved[1];
} ae_attn_bwd_params;

typedef struct ae_devinfo {
  char name[128];
  char arch[64];            /* e.g. "gfx950:sramecc+:xnack-" */
  int32_t compute_units;
  int32_t clock_khz;
  int32_t mem_clock_khz;
  int32_t mem_bus_bits;
  int32_t lds_per_block;
  int32_t l2_bytes;
  int32_t wavefront_size;
  int32_t reserved;
  uint64_t global_mem_bytes;
} ae_devinfo;

typedef struct ae_event ae_event; /* a hipEvent_t with timing enabled */

/* ---- library ------------------------------------------------------------------ */
int ae_abi_version(void);
/* Text of the calling thread's most recent failure ("" if none). Never NULL. */
const char* ae_last_error(void);
/* Number of HIP devices visible (0 when there is none); never fails. */
int ae_device_count(void);
int ae_device_info(int device, ae_devinfo* out);

/* ---- compile: replaces tl.compile / torch.utils.cpp_extension.load -------------- */
/*
 * Compile HIP source `src` for `arch` ("gfx950") with hipRTC. `headers`/`header_names`
 * are in-memory include files (`#include "name"`), `opts` extra compiler options.
 * On failure *out is NULL and ae_last_error() holds the compiler log.
 */
int ae_compile(const char* src, const char* name, const char* arch,
               const char* const* opts, int nopts,
               const char* const* header_names, const char* const* headers, int nheaders,
               ae_module** out);
/* Version of the hipRTC that ae_compile drives (callers fold it into their code-object cache keys; the
 * reference's cache key is an md5 of the rendered source only, attn_engine.py:369-375). */
int ae_compiler_version(int* major, int* minor);
/* hipRTC log of the compilation that produced the module (warnings; "" if none). */
const char* ae_module_log(const ae_module* m);
/* Borrowed view of the code object bytes. */
int ae_module_code(const ae_module* m, const void** data, size_t* size);
/* Code-object cache: write to / read from a file (the reference caches generated
 * source under attn_engine/cache/<md5>.py, attn_engine.py:369-375). */
int ae_module_save(const ae_module* m, const char* path);
int ae_module_load(const char* path, ae_module** out);
void ae_module_free(ae_module* m);

/* ---- load + launch -------------------------------------------------------------- */
/* Load the module on the current device (first call) and look up `kernel_name`.
 * The returned handle is owned by the module and dies with it. */
int ae_module_get_kernel(ae_module* m, const char* kernel_name, ae_kernel** out);
/* Raw launch: `params` (params_bytes) is copied into the kernel argument buffer. */
int ae_launch(ae_kernel* k, const void* params, size_t params_bytes,
              const uint32_t grid[3], const uint32_t block[3],
              uint32_t lds_bytes, void* stream);

/*
 * Typed launches. They validate the argument block against the tile configuration
 * (NULL pointers, non-positive extents, head-group divisibility, block-mask extents,
 * split-KV work buffers) and derive the grid; nothing is launched when a check fails.
 *
 * ae_prefill_fwd: one workgroup per (q-tile, q-head, batch) -- the grid of
 *   attn_tl.py:86 -- flattened to 1-D (padded to a multiple of 8 (batch, head) pairs) so the
 *   kernel can keep the q-tiles of one (batch, head) on one XCD and issue heavy causal tiles first.
 * ae_decode_fwd:  split-KV pass followed by the combine kernel, grid (Hq, B)
 *   (attn_gqa_decode_tl.py:150-151, 224-266). Every WAVE of the split kernel produces one partial,
 *   so its grid is (num_splits / (threads/64), ceil(Hq/Hkv / block_m)*Hkv, B); kv_per_split is the
 *   share of one partial and must be a multiple of block_n; combine_cfg->block_n is the number of
 *   splits the combine kernel was compiled for and must equal num_splits.  A split kernel compiled with
 *   AE_MERGE_IN_WG 1 is announced by cfg->merge_in_wg = 1: num_splits must then equal the waves of one
 *   workgroup, `combine` must be NULL (that workgroup merges its waves' partial results itself and writes
 *   out: one launch, no work buffers).  A split kernel compiled with AE_MERGE_LAST 1 is announced by
 *   cfg->merge_in_wg = 2: `combine` must be NULL, both work buffers and combine_cfg are required (block_n = the
 *   number of splits the kernel was compiled for, which must equal num_splits); the workgroup of a (batch,
 *   kv head, head tile) that finishes last merges all partial results and writes out (one launch).  Its arrival
 *   counters are 32-bit integers BEHIND the row scales in partial_rs -- after max(1, n_rowscales) * batch * heads_q *
 *   num_splits floats, batch * ceil(Hq/Hkv / block_m) * Hkv of them -- which must be zero before the first launch
 *   and which every launch leaves at zero; launches that share these buffers must not overlap.  With
 *   cfg->merge_in_wg = 0 the combine kernel, its configuration and both work buffers are required; a launch that
 *   lacks any of them is refused, nothing runs.
 */
int ae_prefill_fwd(ae_kernel* k, const ae_attn_params* p, const ae_tile_cfg* cfg, void* stream);
int ae_decode_fwd(ae_kernel* split, ae_kernel* combine, const ae_attn_params* p,
                  const ae_tile_cfg* cfg, const ae_tile_cfg* combine_cfg, void* stream);

/*
 * ae_prefill_split_fwd: split-KV attention for a FEW query tokens against a long KV ("MHA decode",
 *   the reference's generic decode template core/template/tl_template/attn/attn_decode_tl.py:47-205,
 *   selected in attn_engine/attn_engine.py:273-290).  The prefill kernel compiled with AE_NSPLIT =
 *   num_splits runs once per (q tile, head, batch, split) on kv_per_split positions (a multiple of
 *   block_n) and writes fp32 partials ordered (batch, q position, head, split); the combine kernel then
 *   merges them with the user's combine() into `out`, which must be contiguous [B,Sq,Hq,DV], and writes
 *   the merged rowscales to rowscale_out as fp32 [B,Hq,Sq], the layout of ae_prefill_fwd.
 */
int ae_prefill_split_fwd(ae_kernel* split, ae_kernel* combine, const ae_attn_params* p,
                         const ae_tile_cfg* cfg, const ae_tile_cfg* combine_cfg, void* stream);

/*
 * ae_mla_decode_fwd: shared-latent-KV (MLA) decode. K = [k | k2] (latent | rope), q = [q | q2],
 *   V = the first head_dim_v columns of k. Stands where the reference calls its TileLang MLA
 *   kernel (mla_decode_tl.py:326-335) or `fwd_kvcache_mla`
 *   (cute_template_kvshared/flash_api.cpp:61-210). Every workgroup covers cfg->block_m query heads
 *   of one (batch, kv head, split); 1-D grid ordered so workgroups sharing a KV range run on one XCD.
 *   With num_splits == 1 the split kernel writes `out` / `rowscale_out` itself: no merge pass runs,
 *   `combine` may be NULL and the partial buffers are not touched.
 */
int ae_mla_decode_fwd(ae_kernel* split, ae_kernel* combine, const ae_attn_params* p,
                      const ae_tile_cfg* cfg, const ae_tile_cfg* combine_cfg, void* stream);

/*
 * ae_prefill_bwd: backward of softmax attention. Three launches on `stream`: `delta`
 *   (rowsum(dout*out), the reference's flashattn_bwd_preprocess, attn_tl.py:196-221), `dkv` (one
 *   workgroup per 128 kv rows of a (batch, kv head): dk and dv, summed over the q heads of the group)
 *   and `dq` (one workgroup per cfg->block_m q rows of a (batch, q head)). The reference's single backward
 *   kernel with fp32 atomics on dq and its postprocess (attn_tl.py:238-455) are replaced by these two
 *   atomic-free launches. cfg describes the dq launch: block_m = 128 with threads = 256, or block_m = 256
 *   with threads = 512 for a dq kernel compiled with AE_BWD_NWAVES 8 (dkv always runs 256 threads);
 *   block_n = 64 and the dynamic LDS of the compiled kernels, mask_mode as compiled (2 needs the two tile-class tables: 0 skip, 1 test per
 *   element, 2 fully visible); head dims as compiled. All gradients are written in full (no accumulation).
 *   The same three launches serve the graphs whose online function does nothing (sigmoid, relu attention:
 *   kernels compiled with AE_BWD_KIND 1 and the generated derivative of score_mod; lse is NULL then).
 *   `delta` may be NULL for softmax kernels compiled with AE_BWD_FUSE_DELTA 1: the dq launch then forms
 *   rowsum(dout*out) for its own rows, fills the work buffer and runs first, dkv second (two launches).
 */
int ae_prefill_bwd(ae_kernel* delta, ae_kernel* dkv, ae_kernel* dq, const ae_attn_bwd_params* p,
                   const ae_tile_cfg* cfg, void* stream);

/*
 * ae_decode_fwd_noalloc: ae_decode_fwd for callers that cannot allocate.  It has no counterpart in the
 *   reference (whose generated _attention.forward allocates its split-KV buffers with torch.empty on every
 *   call, attn_gqa_decode_tl.py:345-348); it is for code under HIP graph capture, tight serving loops and
 *   harnesses that forbid hipMalloc.  Same arguments and checks as ae_decode_fwd, but p->partial_o and
 *   p->partial_rs are ignored: the split-KV partials go to a work buffer of AE_NOALLOC_SCRATCH_BYTES that
 *   is part of the library's device image (one copy per GPU, held until the process ends).  The entry
 *   point calls no hipMalloc / hipFree or any allocating routine; its first call on a device looks up the
 *   buffer's address once (make that call outside a graph capture).  A launch whose partials
 *   (B*Hq*num_splits*(DV + max(1,n_rowscales)) fp32 values, the first part rounded up to 256 bytes) do not
 *   fit returns AE_ERR_INVALID_ARG and launches nothing.  All calls on one GPU share that GPU's buffer:
 *   calls that may overlap in time on one GPU (different streams, different threads) race -- serialise
 *   them, or use ae_decode_fwd with separate buffers.  Nothing in the buffer has to be cleared between
 *   calls (every partial that is read has been written by the same call); for that reason a split kernel
 *   whose last workgroup merges (cfg->merge_in_wg == 2, which needs arrival counters that read zero) is
 *   refused here.
 */
#define AE_NOALLOC_SCRATCH_BYTES (16u << 20)
int ae_decode_fwd_noalloc(ae_kernel* split, ae_kernel* combine, const ae_attn_params* p,
                          const ae_tile_cfg* cfg, const ae_tile_cfg* combine_cfg, void* stream);

/* ---- timing on the launch stream ------------------------------------------------- */
int ae_event_create(ae_event** out);
int ae_event_record(ae_event* e, void* stream);
/* Blocks until `stop` has completed, then returns the elapsed milliseconds. */
int ae_event_elapsed_ms(ae_event* start, ae_event* stop, float* ms);
void ae_event_destroy(ae_event* e);

#ifdef __cplusplus
}
#endif
#endif /* AE_HIP_H */
