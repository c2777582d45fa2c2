"""ctypes binding of libae_hip.so (C ABI declared in include/ae_hip.h).

This is the only place Python touches the native boundary.  It stands where the reference
calls ``tl.compile(...)`` on a rendered template
(attention_engine/core/template/tl_template/attn/attn_tl.py:523-528) or JIT-builds its CuTe
extension (core/template/cute_template/flash_attn_interface.py:136-147).

There is no CPU fallback: if the shared library is missing, or a launch is requested without
a GPU, the calls raise.
"""
from __future__ import annotations

import ctypes as C
import hashlib
import os
import os.path as osp
import threading

_PKG_ROOT = osp.dirname(osp.dirname(osp.dirname(osp.abspath(__file__))))
CSRC_DIR = osp.join(_PKG_ROOT, "csrc")
KERNEL_DIR = osp.join(CSRC_DIR, "kernels")
INCLUDE_DIR = osp.join(osp.dirname(_PKG_ROOT), "include")
LIB_PATH = osp.join(CSRC_DIR, "libae_hip.so")

AE_MAX_ROWSCALES = 4
AE_MAX_CUSTOM = 4

# Options every kernel is compiled with.  Infinities stay meaningful (masks are additive
# -inf), so no -ffast-math / -ffinite-math-only.  Packed-fp32 instruction selection is
# switched off on purpose (scalar fp32 code only).
COMPILE_OPTS = [
    "-O3",
    "-std=c++17",
    "-fno-math-errno", "-fno-trapping-math", "-fno-signed-zeros", "-freciprocal-math",
    "-ffp-contract=fast",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


class AEError(RuntimeError):
    """A call into libae_hip.so returned a non-zero status."""


class AttnParams(C.Structure):
    """Mirror of ``ae_attn_params``."""
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("out", C.c_void_p),
        ("rowscale_out", C.c_void_p * AE_MAX_ROWSCALES),
        ("custom", C.c_void_p * AE_MAX_CUSTOM),
        ("block_mask", C.c_void_p),
        ("partial_o", C.c_void_p), ("partial_rs", C.c_void_p),
        ("q2", C.c_void_p), ("k2", C.c_void_p),
        ("q_stride_b", C.c_int64), ("q_stride_s", C.c_int64), ("q_stride_h", C.c_int64),
        ("k_stride_b", C.c_int64), ("k_stride_s", C.c_int64), ("k_stride_h", C.c_int64),
        ("v_stride_b", C.c_int64), ("v_stride_s", C.c_int64), ("v_stride_h", C.c_int64),
        ("o_stride_b", C.c_int64), ("o_stride_s", C.c_int64), ("o_stride_h", C.c_int64),
        ("q2_stride_b", C.c_int64), ("q2_stride_s", C.c_int64), ("q2_stride_h", C.c_int64),
        ("k2_stride_b", C.c_int64), ("k2_stride_s", C.c_int64), ("k2_stride_h", C.c_int64),
        ("batch", C.c_int32), ("heads_q", C.c_int32), ("heads_kv", C.c_int32),
        ("seqlen_q", C.c_int32), ("seqlen_kv", C.c_int32),
        ("mask_b", C.c_int32), ("mask_h", C.c_int32), ("mask_nq", C.c_int32), ("mask_nkv", C.c_int32),
        ("mask_block_m", C.c_int32), ("mask_block_n", C.c_int32),
        ("num_splits", C.c_int32), ("kv_per_split", C.c_int32),
        ("reserved", C.c_int32 * 3),
        ("block_table", C.c_void_p), ("seqlens_k", C.c_void_p),
        ("block_table_stride", C.c_int32), ("page_block_size", C.c_int32), ("num_pages", C.c_int32),
        ("reserved2", C.c_int32),
    ]


class AttnBwdParams(C.Structure):
    """Mirror of ``ae_attn_bwd_params``."""
    _fields_ = (
        [(n, C.c_void_p) for n in ("q", "k", "v", "out", "dout", "lse", "delta", "dq", "dk", "dv",
                                   "mask_dq", "mask_dkv")]
        + [("custom", C.c_void_p * AE_MAX_CUSTOM), ("block_mask", C.c_void_p),
           ("more_rowscales", C.c_void_p * (AE_MAX_ROWSCALES - 1))]
        + [(f"{t}_stride_{a}", C.c_int64) for t in ("q", "k", "v", "o", "do", "dq", "dk", "dv") for a in "bsh"]
        + [("batch", C.c_int32), ("heads_q", C.c_int32), ("heads_kv", C.c_int32),
           ("seqlen_q", C.c_int32), ("seqlen_kv", C.c_int32), ("mask_b", C.c_int32), ("mask_h", C.c_int32),
           ("mask_nq", C.c_int32), ("mask_nkv", C.c_int32), ("mask_block_m", C.c_int32), ("mask_block_n", C.c_int32),
           ("reserved", C.c_int32 * 1)]
    )


class TileCfg(C.Structure):
    """Mirror of ``ae_tile_cfg``."""
    _fields_ = [
        ("block_m", C.c_int32), ("block_n", C.c_int32), ("threads", C.c_int32),
        ("lds_bytes", C.c_int32), ("head_dim", C.c_int32), ("head_dim_v", C.c_int32),
        ("elem_bytes", C.c_int32), ("n_rowscales", C.c_int32), ("mask_mode", C.c_int32),
        ("paged", C.c_int32), ("merge_in_wg", C.c_int32), ("table_rows", C.c_int32),
    ]


class DevInfo(C.Structure):
    """Mirror of ``ae_devinfo``."""
    _fields_ = [
        ("name", C.c_char * 128), ("arch", C.c_char * 64),
        ("compute_units", C.c_int32), ("clock_khz", C.c_int32), ("mem_clock_khz", C.c_int32),
        ("mem_bus_bits", C.c_int32), ("lds_per_block", C.c_int32), ("l2_bytes", C.c_int32),
        ("wavefront_size", C.c_int32), ("reserved", C.c_int32),
        ("global_mem_bytes", C.c_uint64),
    ]


# every symbol include/ae_hip.h declares: name -> (restype, argtypes)
_VP = C.c_void_p
_SIGNATURES = {
    "ae_abi_version": (C.c_int, []),
    "ae_last_error": (C.c_char_p, []),
    "ae_device_count": (C.c_int, []),
    "ae_device_info": (C.c_int, [C.c_int, C.POINTER(DevInfo)]),
    "ae_compile": (C.c_int, [C.c_char_p, C.c_char_p, C.c_char_p, C.POINTER(C.c_char_p), C.c_int,
                             C.POINTER(C.c_char_p), C.POINTER(C.c_char_p), C.c_int, C.POINTER(_VP)]),
    "ae_compiler_version": (C.c_int, [C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "ae_module_log": (C.c_char_p, [_VP]),
    "ae_module_code": (C.c_int, [_VP, C.POINTER(_VP), C.POINTER(C.c_size_t)]),
    "ae_module_save": (C.c_int, [_VP, C.c_char_p]),
    "ae_module_load": (C.c_int, [C.c_char_p, C.POINTER(_VP)]),
    "ae_module_free": (None, [_VP]),
    "ae_module_get_kernel": (C.c_int, [_VP, C.c_char_p, C.POINTER(_VP)]),
    "ae_launch": (C.c_int, [_VP, _VP, C.c_size_t, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32),
                            C.c_uint32, _VP]),
    "ae_prefill_fwd": (C.c_int, [_VP, C.POINTER(AttnParams), C.POINTER(TileCfg), _VP]),
    "ae_decode_fwd": (C.c_int, [_VP, _VP, C.POINTER(AttnParams), C.POINTER(TileCfg),
                                C.POINTER(TileCfg), _VP]),
    "ae_decode_fwd_noalloc": (C.c_int, [_VP, _VP, C.POINTER(AttnParams), C.POINTER(TileCfg),
                                        C.POINTER(TileCfg), _VP]),
    "ae_mla_decode_fwd": (C.c_int, [_VP, _VP, C.POINTER(AttnParams), C.POINTER(TileCfg),
                                    C.POINTER(TileCfg), _VP]),
    "ae_prefill_split_fwd": (C.c_int, [_VP, _VP, C.POINTER(AttnParams), C.POINTER(TileCfg),
                                       C.POINTER(TileCfg), _VP]),
    "ae_prefill_bwd": (C.c_int, [_VP, _VP, _VP, C.POINTER(AttnBwdParams), C.POINTER(TileCfg), _VP]),
    "ae_event_create": (C.c_int, [C.POINTER(_VP)]),
    "ae_event_record": (C.c_int, [_VP, _VP]),
    "ae_event_elapsed_ms": (C.c_int, [_VP, _VP, C.POINTER(C.c_float)]),
    "ae_event_destroy": (None, [_VP]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None
_lib_lock = threading.Lock()


AE_ABI_VERSION = 6      # AE_ABI_VERSION of include/ae_hip.h


def lib():
    """Load libae_hip.so once; raise if it has not been built (no fallback)."""
    global _lib
    if _lib is None:
        with _lib_lock:
            if _lib is None:
                if not osp.exists(LIB_PATH):
                    raise AEError(
                        f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; "
                        "g.build()'` (or attentionengine_amd/csrc/build.py)")
                handle = C.CDLL(LIB_PATH)
                for name, (res, args) in _SIGNATURES.items():
                    fn = getattr(handle, name)
                    fn.restype = res
                    fn.argtypes = args
                if handle.ae_abi_version() != AE_ABI_VERSION:
                    # (a library built from another header: its structures may be laid out differently)
                    raise AEError(f"{LIB_PATH} has C ABI version {handle.ae_abi_version()}, this binding is written for "
                                  f"{AE_ABI_VERSION}: rebuild it (python -c 'import __graft_entry__ as g; g.build()')")
                _lib = handle
    return _lib


def _check(rc):
    if rc != 0:
        raise AEError(f"[ae status {rc}] " + lib().ae_last_error().decode("utf-8", "replace"))


def device_count() -> int:
    return lib().ae_device_count()


def device_info(device: int = 0) -> dict:
    info = DevInfo()
    _check(lib().ae_device_info(device, C.byref(info)))
    out = {f: getattr(info, f) for f, _ in DevInfo._fields_ if f != "reserved"}
    out["name"] = info.name.decode()
    out["arch"] = info.arch.decode()
    return out


_compiler_version = None


def compiler_version() -> str:
    """"major.minor" of the hipRTC that ae_compile uses (part of the code-object cache key: objects
    cached by one toolchain are not reused by another)."""
    global _compiler_version
    if _compiler_version is None:
        major, minor = C.c_int(), C.c_int()
        _check(lib().ae_compiler_version(C.byref(major), C.byref(minor)))
        _compiler_version = f"hiprtc {major.value}.{minor.value}"
    return _compiler_version


def cache_dir() -> str:
    """Directory of cached code objects (the reference caches rendered source under
    attn_engine/cache/<md5>.py, attn_engine.py:369-375)."""
    d = os.environ.get("AE_CACHE_DIR") or osp.join(_PKG_ROOT, "_cache")
    try:
        os.makedirs(d, exist_ok=True)
        if not os.access(d, os.W_OK):
            raise OSError
    except OSError:
        d = osp.join(osp.expanduser("~"), ".cache", "attentionengine_amd")
        os.makedirs(d, exist_ok=True)
    return d


def _read(path):
    with open(path, "r") as f:
        return f.read()


class Kernel:
    """A kernel of a loaded module, bound to the device it was loaded on."""

    def __init__(self, module: "Module", name: str):
        self.module = module
        self.name = name
        h = _VP()
        _check(lib().ae_module_get_kernel(module.handle, name.encode(), C.byref(h)))
        self.handle = h

    def launch(self, params: C.Structure, grid, block, lds_bytes: int, stream: int = 0):
        g = (C.c_uint32 * 3)(*grid)
        b = (C.c_uint32 * 3)(*block)
        _check(lib().ae_launch(self.handle, C.byref(params), C.sizeof(params), g, b, lds_bytes,
                               _VP(stream)))


class Module:
    """A compiled code object.  Compilation needs no GPU; ``kernel()`` does."""

    def __init__(self, handle, source_key: str, from_cache: bool):
        self.handle = handle
        self.key = source_key
        self.from_cache = from_cache
        self._kernels = {}

    @property
    def log(self) -> str:
        return lib().ae_module_log(self.handle).decode("utf-8", "replace")

    def code(self) -> bytes:
        data, size = _VP(), C.c_size_t()
        _check(lib().ae_module_code(self.handle, C.byref(data), C.byref(size)))
        return C.string_at(data, size.value)

    def kernel_info(self) -> dict:
        """{kernel name: its metadata from the code object's AMDGPU note (register counts, ``.vgpr_spill_count``,
        scratch and LDS bytes, ...)}.  What the compiler that built THIS code object did - hipRTC's, which need not
        agree with an offline hipcc of another ROCm release about how many registers it spills."""
        import struct
        import msgpack
        f = self.code()
        if f[:4] != b"\x7fELF" or f[4] != 2:
            raise AEError("not a 64-bit ELF code object")
        shoff = struct.unpack_from("<Q", f, 0x28)[0]
        shentsize, shnum, _ = struct.unpack_from("<HHH", f, 0x3A)
        for i in range(shnum):
            _, typ, _, _, offset, size = struct.unpack_from("<IIQQQQ", f, shoff + i * shentsize)
            if typ != 7:                                   # SHT_NOTE
                continue
            pos = offset
            while pos < offset + size:
                namesz, descsz, ntype = struct.unpack_from("<III", f, pos)
                pos += 12 + ((namesz + 3) & ~3)
                desc = f[pos:pos + descsz]
                pos += (descsz + 3) & ~3
                if ntype == 32:                            # NT_AMDGPU_METADATA (msgpack)
                    md = msgpack.unpackb(desc, raw=False, strict_map_key=False)
                    return {k[".name"]: k for k in md.get("amdhsa.kernels", [])}
        raise AEError("code object without an AMDGPU metadata note")

    def scratch_accesses(self) -> dict:
        """{"single": n, "wide": m}: scratch-memory instructions in the code object's .text that move one
        dword, and those that move two to four (``scratch_load/store_dwordx2/x3/x4``) -- the form in which the
        compiler spills and reloads register TUPLES (matrix accumulators, MFMA operands).  Found by matching
        the instruction words (FLAT encoding, scratch segment); no disassembler is involved."""
        import struct
        f = self.code()
        shoff = struct.unpack_from("<Q", f, 0x28)[0]
        shentsize, shnum, shstrndx = struct.unpack_from("<HHH", f, 0x3A)
        secs = [struct.unpack_from("<IIQQQQ", f, shoff + i * shentsize) for i in range(shnum)]
        strtab = secs[shstrndx][4]
        out = {"single": 0, "wide": 0}
        for name_off, typ, _, _, offset, size in secs:
            name = f[strtab + name_off:f.index(b"\0", strtab + name_off)]
            if name != b".text":
                continue
            for (w,) in struct.iter_unpack("<I", f[offset:offset + (size & ~3)]):
                if (w & 0xFC00C000) != 0xDC004000:        # FLAT encoding, segment = scratch
                    continue
                op = (w >> 18) & 0x7F
                if op in (20, 28):                          # scratch_load_dword, scratch_store_dword
                    out["single"] += 1
                elif op in (21, 22, 23, 29, 30, 31):        # ..._dwordx2, x3, x4
                    out["wide"] += 1
        return out

    def kernel(self, name: str) -> Kernel:
        k = self._kernels.get(name)
        if k is None:
            k = self._kernels[name] = Kernel(self, name)
        return k

    def __del__(self):
        try:
            if self.handle:
                lib().ae_module_free(self.handle)
                self.handle = None
        except Exception:
            pass


_modules = {}
_modules_lock = threading.Lock()


class SpillError(AEError):
    """A compiled kernel keeps part of its vector registers in scratch memory (see ``check_spills``)."""


# scratch bytes per lane beyond which a build counts as spilling heavily (slow, and refused)
MAX_SCRATCH_BYTES = 128


def check_spills(module: "Module", what: str, allow_spills=None, strict=False):
    """Warns about -- or, where asked to be strict, refuses -- a code object that moves register TUPLES through
    scratch memory or spills heavily.

    Every attention template holds its matrix accumulators as 16-register tuples, several of them pinned to the
    accumulator file by ``asm`` statements.  One build of the compiler in use (wide value heads, tile table, ragged
    tiles: 16 spilled values) spilled such a tuple -- twelve registers with three ``scratch_store_dwordx4``, a
    thirteenth alone, three kept in other registers -- and, where it put the tuple together again, never emitted
    the copy of one of the three: the reloaded tuple carried a stale register and the kernel returned one wrong
    pair of output columns, silently (found by reading that build's code; the kernel has since been changed so
    that the build no longer spills).  Builds that spill a few single values (a row's running maximum, a lane
    index: plain ``scratch_store_dword`` / ``scratch_load_dword``) take none of that path.

    A build is SUSPECT when its code contains scratch accesses wider than one dword, or when it keeps more than
    MAX_SCRATCH_BYTES per lane in scratch memory.  Many of the less common configurations (odd head-dim pairs,
    decode shapes with few heads, backward launches under elementwise masks) are suspect builds that pass their
    parity tests, so by default a suspect build only raises a RuntimeWarning naming the kernel.  It is refused
    (SpillError) when ``strict`` is set -- the operators set it for the family of builds in which the wrong
    columns were seen, the wide value heads of ae_prefill.hip, which do not spill as the kernel stands -- when
    ``allow_spills`` is False (``AttentionEngine(..., allow_spills=False)``), or with AE_ALLOW_SPILLS=0 in the
    environment, which refuses every build that spills at all.  ``allow_spills=True`` / AE_ALLOW_SPILLS=1
    switch the check off."""
    env = os.environ.get("AE_ALLOW_SPILLS", "")
    if allow_spills is True or (allow_spills is None and env == "1"):
        return
    info = module.kernel_info()
    spilling = {name: (k.get(".vgpr_spill_count", 0), k.get(".private_segment_fixed_size", 0))
                for name, k in info.items() if k.get(".vgpr_spill_count", 0)}
    if not spilling:
        return
    acc = module.scratch_accesses()
    heavy = any(b > MAX_SCRATCH_BYTES for _, b in spilling.values())
    if not (acc["wide"] or heavy or env == "0"):
        return
    text = ", ".join(f"{n}: {c} spilled registers, {b} bytes of scratch per lane" for n, (c, b) in sorted(spilling.items()))
    why = (f"{acc['wide']} scratch accesses wider than one dword: a register tuple goes through scratch memory"
           if acc["wide"] else "it spills heavily" if heavy else "AE_ALLOW_SPILLS=0")
    msg = (f"{what}: the compiled kernel spills vector registers ({text}; {why}).  One such build has returned wrong "
           "results (a register tuple put together again from scratch memory lost a register)")
    if strict or allow_spills is False or env == "0":
        raise SpillError(msg + "; this build is refused -- choose other head dims / tiles, or pass allow_spills=True "
                               "(AE_ALLOW_SPILLS=1) to run it anyway")
    import warnings
    warnings.warn(msg + "; check its results, or pass allow_spills=False to refuse such builds", RuntimeWarning,
                  stacklevel=3)


def compile_module(template: str, headers: dict, arch: str = None, use_cache: bool = True,
                   allow_spills=None, strict_spills=False) -> Module:
    """Compile kernel template ``template`` (a file name under csrc/kernels) with the generated
    in-memory ``headers`` ({"ae_config.h": text, "ae_functors.h": text}).

    The code object is cached on disk under a key that covers the template text, every header,
    the architecture and the compiler options, and in memory for the life of the process.  A code object
    that moves register tuples through scratch memory is reported or refused (``check_spills``).
    """
    m = _compile_module(template, headers, arch, use_cache)
    check_spills(m, template, allow_spills, strict_spills)
    return m


def _compile_module(template: str, headers: dict, arch: str = None, use_cache: bool = True) -> Module:
    arch = arch or os.environ.get("AE_HIP_ARCH", "gfx950")
    src = _read(osp.join(KERNEL_DIR, template))
    all_headers = {
        "ae_hip.h": _read(osp.join(INCLUDE_DIR, "ae_hip.h")),
        "ae_device.h": _read(osp.join(KERNEL_DIR, "ae_device.h")),
        "ae_combine.h": _read(osp.join(KERNEL_DIR, "ae_combine.h")),
        "ae_mla_paged.h": _read(osp.join(KERNEL_DIR, "ae_mla_paged.h")),
        "ae_tile_table.h": _read(osp.join(KERNEL_DIR, "ae_tile_table.h")),
    }
    all_headers.update(headers)
    hsh = hashlib.sha256()
    for part in [template, src, arch, " ".join(COMPILE_OPTS), compiler_version()]:
        hsh.update(part.encode())
        hsh.update(b"\0")
    for name in sorted(all_headers):
        hsh.update(name.encode() + b"\0" + all_headers[name].encode() + b"\0")
    key = hsh.hexdigest()[:32]
    with _modules_lock:
        m = _modules.get(key)
        if m is not None:
            return m
        path = osp.join(cache_dir(), f"{osp.splitext(template)[0]}_{key}.hsaco")
        handle = _VP()
        if use_cache and osp.exists(path):
            _check(lib().ae_module_load(path.encode(), C.byref(handle)))
            m = Module(handle, key, True)
        else:
            names = list(all_headers)
            n = len(names)
            c_names = (C.c_char_p * n)(*[s.encode() for s in names])
            c_srcs = (C.c_char_p * n)(*[all_headers[s].encode() for s in names])
            c_opts = (C.c_char_p * len(COMPILE_OPTS))(*[o.encode() for o in COMPILE_OPTS])
            _check(lib().ae_compile(src.encode(), template.encode(), arch.encode(), c_opts,
                                    len(COMPILE_OPTS), c_names, c_srcs, n, C.byref(handle)))
            m = Module(handle, key, False)
            if use_cache:
                try:
                    _check(lib().ae_module_save(handle, path.encode()))
                except AEError:
                    pass  # an unwritable cache only costs a recompile next time
        _modules[key] = m
        return m


class Event:
    """HIP event recorded on the stream the kernels are launched on."""

    def __init__(self):
        h = _VP()
        _check(lib().ae_event_create(C.byref(h)))
        self.handle = h

    def record(self, stream: int = 0):
        _check(lib().ae_event_record(self.handle, _VP(stream)))

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        _check(lib().ae_event_elapsed_ms(self.handle, stop.handle, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self.handle:
                lib().ae_event_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


def rows_for_kernels(t):
    """``t`` as the kernels can read it: dense in the last dimension, starting on a 16-byte boundary, every
    other stride a multiple of 8 elements (rows are moved 16 bytes at a time; the C entry points refuse anything
    else).  Tensors laid out otherwise - a column slice that starts at an odd offset, say - are copied."""
    st = t.stride()
    if st[-1] == 1 and t.data_ptr() % 16 == 0:
        for x in st[:-1]:
            if x % 8:
                break
        else:
            return t
    return t.contiguous()


_raw_stream = None


def current_stream(device) -> int:
    """The raw handle of torch's current stream on ``device`` (what ``torch.cuda.current_stream(device).cuda_stream``
    returns, without building the Stream object: a third of the time of a small call)."""
    global _raw_stream
    if _raw_stream is None:
        import torch
        raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        _raw_stream = raw if raw is not None else (lambda index: torch.cuda.current_stream(index).cuda_stream)
    index = device.index
    if index is None:
        import torch
        index = torch.cuda.current_device()
    return _raw_stream(index)


def prefill_fwd(kernel: Kernel, params: AttnParams, cfg: TileCfg, stream: int = 0):
    _check(lib().ae_prefill_fwd(kernel.handle, C.byref(params), C.byref(cfg), _VP(stream)))


def decode_fwd(split: Kernel, combine: Kernel, params: AttnParams, cfg: TileCfg,
               combine_cfg: TileCfg, stream: int = 0):
    _check(lib().ae_decode_fwd(split.handle, combine.handle if combine else None, C.byref(params),
                               C.byref(cfg), C.byref(combine_cfg) if combine_cfg else None,
                               _VP(stream)))


def decode_fwd_noalloc(split: Kernel, combine: Kernel, params: AttnParams, cfg: TileCfg,
                       combine_cfg: TileCfg, stream: int = 0):
    """ae_decode_fwd on the library's built-in split-KV work buffer (params.partial_* are ignored)."""
    _check(lib().ae_decode_fwd_noalloc(split.handle, combine.handle if combine else None, C.byref(params),
                                       C.byref(cfg), C.byref(combine_cfg) if combine_cfg else None,
                                       _VP(stream)))


NOALLOC_SCRATCH_BYTES = 16 << 20      # AE_NOALLOC_SCRATCH_BYTES of include/ae_hip.h


def prefill_split_fwd(split: Kernel, combine: Kernel, params: AttnParams, cfg: TileCfg,
                      combine_cfg: TileCfg, stream: int = 0):
    _check(lib().ae_prefill_split_fwd(split.handle, combine.handle, C.byref(params), C.byref(cfg),
                                      C.byref(combine_cfg), _VP(stream)))


def mla_decode_fwd(split: Kernel, combine: Kernel, params: AttnParams, cfg: TileCfg,
                   combine_cfg: TileCfg, stream: int = 0):
    _check(lib().ae_mla_decode_fwd(split.handle, combine.handle, C.byref(params), C.byref(cfg),
                                   C.byref(combine_cfg), _VP(stream)))


def prefill_bwd(delta: Kernel, dkv: Kernel, dq: Kernel, params: AttnBwdParams, cfg: TileCfg, stream: int = 0):
    _check(lib().ae_prefill_bwd(delta.handle if delta is not None else None, dkv.handle, dq.handle, C.byref(params),
                                C.byref(cfg), _VP(stream)))
