"""The C-ABI library loads, exports every symbol include/ae_hip.h declares, compiles for gfx950
without a GPU, caches code objects, and fails loudly (status + message, no exit) on bad input."""
import ctypes
import os
import re

import pytest
import torch

from core.runtime import hip_rt as rt

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ae_hip.h")

KERNEL = r'''
#include "ae_hip.h"
extern "C" __global__ void ae_probe(const ae_attn_params p) {
  if (threadIdx.x == 0) ((float*)p.out)[0] = (float)sizeof(ae_attn_params);
}
'''


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ae_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    names = _declared_functions()
    assert "ae_compile" in names and "ae_prefill_fwd" in names and "ae_mla_decode_fwd" in names
    lib = ctypes.CDLL(rt.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in ae_hip.h but not exported"
    assert sorted(rt.EXPORTED_SYMBOLS) == names
    assert rt.lib().ae_abi_version() == 6


def test_struct_layout_matches_the_header():
    """Size and every field offset of the three parameter structs, as the DEVICE compiler lays them out
    from include/ae_hip.h, equal the ctypes mirrors: a probe whose static_asserts carry the ctypes figures
    is compiled for gfx950 through ae_compile (needs no GPU).  A reordered or retyped field of equal size
    in either place fails the compilation."""
    # 4 + 4 + 4 + 1 + 2 + 2 pointers, 18 strides, 13 + 3 ints, then the paged-cache part: 2 pointers, 3 + 1 ints
    assert ctypes.sizeof(rt.AttnParams) == 8 * 17 + 8 * 18 + 4 * 16 + 8 * 2 + 4 * 4
    assert ctypes.sizeof(rt.TileCfg) == 4 * 12
    # backward: 12 + 4 + 1 + 3 pointers, 8 tensors x 3 strides, 7 + 4 + 1 ints
    assert ctypes.sizeof(rt.AttnBwdParams) == 8 * 20 + 8 * 24 + 4 * 12
    lines = ['#include "ae_hip.h"']
    n_fields = 0
    for cname, mirror in (("ae_attn_params", rt.AttnParams), ("ae_tile_cfg", rt.TileCfg),
                          ("ae_attn_bwd_params", rt.AttnBwdParams), ("ae_devinfo", rt.DevInfo)):
        lines.append(f'static_assert(sizeof({cname}) == {ctypes.sizeof(mirror)}, "sizeof {cname}");')
        for fname, ftype in mirror._fields_:
            off, size = getattr(mirror, fname).offset, ctypes.sizeof(ftype)
            lines.append(f'static_assert(__builtin_offsetof({cname}, {fname}) == {off}, "{cname}.{fname} offset");')
            lines.append(f'static_assert(sizeof((({cname}*)0)->{fname}) == {size}, "{cname}.{fname} size");')
            n_fields += 1
    lines.append('extern "C" __global__ void probe(int* p) { p[0] = 0; }')
    assert n_fields > 80
    rc, handle = _compile("\n".join(lines))
    assert rc == 0, rt.lib().ae_last_error().decode()
    rt.lib().ae_module_free(handle)
    # ... and the probe does notice a wrong figure
    bad = "\n".join(lines).replace("__builtin_offsetof(ae_attn_params, k2) == ", "__builtin_offsetof(ae_attn_params, k2) == 1 + ")
    rc, _ = _compile(bad)
    assert rc != 0 and "ae_attn_params.k2 offset" in rt.lib().ae_last_error().decode()


def test_the_binding_sketch_in_the_integration_notes_matches_the_header():
    """The integration notes at the repository root show the ctypes structures a maintainer of the reference would
    copy.  They are executed here as written (the two class statements only) and must have the size of
    ae_attn_params / ae_tile_cfg,
    with every field the ctypes mirror of the library also has at the same offset; a sketch that is one ABI
    behind hands the launch functions a short struct."""
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    start = text.index("class AttnParams(C.Structure):")
    end = text.index("assert _lib.ae_abi_version()", start)
    ns = {"C": ctypes}
    exec(text[start:end], ns)
    version = int(re.search(r"assert _lib\.ae_abi_version\(\) == (\d+)", text).group(1))
    assert version == rt.lib().ae_abi_version()
    for doc, mirror in ((ns["AttnParams"], rt.AttnParams), (ns["TileCfg"], rt.TileCfg)):
        assert ctypes.sizeof(doc) == ctypes.sizeof(mirror)
        mine = {n: getattr(mirror, n).offset for n, _ in mirror._fields_}
        for name, _ in doc._fields_:
            if name == "strides":          # the sketch folds the 18 strides into one array
                assert doc.strides.offset == mirror.q_stride_b.offset and doc.strides.size == 18 * 8
            else:
                assert getattr(doc, name).offset == mine[name], name
        assert doc._fields_[-1][0] == mirror._fields_[-1][0]


def _compile(src, opts=()):
    lib = rt.lib()
    handle = ctypes.c_void_p()
    hdr = open(HEADER).read().encode()
    names = (ctypes.c_char_p * 1)(b"ae_hip.h")
    srcs = (ctypes.c_char_p * 1)(hdr)
    copts = (ctypes.c_char_p * max(1, len(opts)))(*[o.encode() for o in opts]) if opts else None
    rc = lib.ae_compile(src.encode(), b"probe.hip", b"gfx950", copts, len(opts), names, srcs, 1,
                        ctypes.byref(handle))
    return rc, handle


def test_compile_save_load_roundtrip(tmp_path):
    lib = rt.lib()
    rc, h = _compile(KERNEL, ["-O3"])
    assert rc == 0, lib.ae_last_error()
    data, size = ctypes.c_void_p(), ctypes.c_size_t()
    assert lib.ae_module_code(h, ctypes.byref(data), ctypes.byref(size)) == 0
    code = ctypes.string_at(data, size.value)
    assert code[:4] == b"\x7fELF" and size.value > 1000
    path = str(tmp_path / "probe.hsaco").encode()
    assert lib.ae_module_save(h, path) == 0
    h2 = ctypes.c_void_p()
    assert lib.ae_module_load(path, ctypes.byref(h2)) == 0
    assert lib.ae_module_code(h2, ctypes.byref(data), ctypes.byref(size)) == 0
    assert ctypes.string_at(data, size.value) == code
    lib.ae_module_free(h)
    lib.ae_module_free(h2)


def test_compile_error_returns_status_and_log():
    lib = rt.lib()
    rc, h = _compile("extern \"C\" __global__ void k() { this is not C++; }")
    assert rc == 2 and not h.value
    msg = lib.ae_last_error().decode()
    assert "hipRTC compile failed" in msg and "error" in msg


def test_bad_arguments_fail_without_exiting(tmp_path):
    lib = rt.lib()
    assert lib.ae_compile(None, None, None, None, 0, None, None, 0, None) == 1
    h = ctypes.c_void_p()
    assert lib.ae_module_load(str(tmp_path / "missing.hsaco").encode(), ctypes.byref(h)) == 4
    assert b"cannot open" in lib.ae_last_error()
    p, cfg = rt.AttnParams(), rt.TileCfg()
    assert lib.ae_prefill_fwd(None, ctypes.byref(p), ctypes.byref(cfg), None) == 1
    assert lib.ae_device_info(0, None) == 1


def test_paged_cache_arguments_are_checked_before_any_launch():
    """ae_mla_decode_fwd refuses an inconsistent block table; the other launches refuse any.  Every case
    fails in the argument checks, so the kernel handle (never dereferenced before them) is a dummy."""
    lib = rt.lib()
    fake = ctypes.c_void_p(8)
    buf = ctypes.create_string_buffer(64)
    addr = ctypes.addressof(buf)

    def params(**kw):
        p = rt.AttnParams()
        p.q = p.k = p.v = p.out = p.q2 = p.k2 = addr
        p.batch, p.heads_q, p.heads_kv, p.seqlen_q, p.seqlen_kv = 2, 128, 1, 1, 256
        p.num_splits, p.kv_per_split = 1, 256
        for k, v in kw.items():
            setattr(p, k, v)
        return p

    def cfg(**kw):
        c = rt.TileCfg(block_m=64, block_n=32, threads=512, lds_bytes=1024, head_dim=576, head_dim_v=512,
                       elem_bytes=2, n_rowscales=0, mask_mode=0)
        for k, v in kw.items():
            setattr(c, k, v)
        return c

    def mla(p, c):
        cc = rt.TileCfg(block_m=1, block_n=p.num_splits, threads=128)
        rc = lib.ae_mla_decode_fwd(fake, fake, ctypes.byref(p), ctypes.byref(c), ctypes.byref(cc), None)
        return rc, lib.ae_last_error().decode()

    rc, msg = mla(params(), cfg(paged=1))
    assert rc == 1 and "without block_table" in msg
    table = dict(block_table=addr, seqlens_k=addr, block_table_stride=4, page_block_size=64, num_pages=8)
    rc, msg = mla(params(**table), cfg())
    assert rc == 1 and "built for a dense cache" in msg
    rc, msg = mla(params(**{**table, "page_block_size": 48}), cfg(paged=1))
    assert rc == 1 and "not a multiple of the 32-token kv tile" in msg
    rc, msg = mla(params(**{**table, "block_table_stride": 3}), cfg(paged=1))
    assert rc == 1 and "do not cover Skv=256" in msg
    rc, msg = mla(params(**{**table, "num_pages": 0}), cfg(paged=1))
    assert rc == 1 and "num_pages" in msg
    p = params(**table)
    assert lib.ae_prefill_fwd(fake, ctypes.byref(p), ctypes.byref(cfg()), None) == 1
    assert "reads a dense cache" in lib.ae_last_error().decode()
    cc = rt.TileCfg(block_m=1, block_n=1, threads=128)
    assert lib.ae_decode_fwd(fake, fake, ctypes.byref(p), ctypes.byref(cfg()), ctypes.byref(cc), None) == 1
    assert "reads a dense cache" in lib.ae_last_error().decode()


def test_decode_merge_form_is_checked_before_any_launch():
    """Whether a GQA split kernel merges its waves' partial results itself (AE_MERGE_IN_WG) travels in
    ae_tile_cfg.merge_in_wg, and ae_decode_fwd holds every launch to it: a kernel that does not merge never
    runs without a combine kernel and both work buffers (it would store through NULL), a kernel that merges
    takes no combine kernel and needs its splits to be the waves of one workgroup.  All refusals happen in the
    argument checks, so the kernel handles are dummies."""
    lib = rt.lib()
    fake = ctypes.c_void_p(8)
    buf = ctypes.create_string_buffer(64)
    addr = ctypes.addressof(buf)

    def params(**kw):
        p = rt.AttnParams()
        p.q = p.k = p.v = p.out = addr
        p.batch, p.heads_q, p.heads_kv, p.seqlen_q, p.seqlen_kv = 2, 32, 8, 1, 256
        p.num_splits, p.kv_per_split = 4, 64
        for k, v in kw.items():
            setattr(p, k, v)
        return p

    def cfg(**kw):
        c = rt.TileCfg(block_m=16, block_n=32, threads=256, lds_bytes=1024, head_dim=128, head_dim_v=128,
                       elem_bytes=2, n_rowscales=0, mask_mode=0)
        for k, v in kw.items():
            setattr(c, k, v)
        return c

    def run(entry, p, c, combine, ccfg=True):
        cc = rt.TileCfg(block_m=1, block_n=p.num_splits, threads=64)
        rc = entry(fake, combine, ctypes.byref(p), ctypes.byref(c), ctypes.byref(cc) if ccfg else None, None)
        return rc, lib.ae_last_error().decode()

    for entry in (lib.ae_decode_fwd, lib.ae_decode_fwd_noalloc):
        # a kernel that does not merge, launched without a combine kernel (what a stale kernel cache once did)
        rc, msg = run(entry, params(), cfg(merge_in_wg=0), None)
        assert rc == 1 and "does not merge in the workgroup" in msg, msg
        # a merging kernel takes no combine kernel, and only the waves of one workgroup as its splits
        rc, msg = run(entry, params(), cfg(merge_in_wg=1), fake)
        assert rc == 1 and "takes no combine kernel" in msg, msg
        rc, msg = run(entry, params(num_splits=16, kv_per_split=32), cfg(merge_in_wg=1), None)
        assert rc == 1 and "the 4 waves of one workgroup" in msg, msg
        rc, msg = run(entry, params(), cfg(merge_in_wg=7), None)
        assert rc == 1 and "merge_in_wg=7" in msg, msg
        rc, msg = run(entry, params(), cfg(merge_in_wg=1, n_rowscales=1), None)
        assert rc == 1 and "rowscale_out[0] is NULL" in msg, msg
    # the last workgroup merges (2): no combine kernel, but both work buffers (partial results, arrival counters)
    rc, msg = run(lib.ae_decode_fwd, params(num_splits=16, kv_per_split=32, partial_o=addr, partial_rs=addr),
                  cfg(merge_in_wg=2), fake)
    assert rc == 1 and "takes no combine kernel" in msg, msg
    rc, msg = run(lib.ae_decode_fwd, params(num_splits=16, kv_per_split=32), cfg(merge_in_wg=2), None)
    assert rc == 1 and "work buffers are NULL" in msg, msg
    rc, msg = run(lib.ae_decode_fwd, params(num_splits=16, kv_per_split=32, partial_o=addr, partial_rs=addr),
                  cfg(merge_in_wg=2), None, ccfg=False)
    assert rc == 1 and "needs combine_cfg" in msg, msg
    rc, msg = run(lib.ae_decode_fwd_noalloc, params(num_splits=16, kv_per_split=32), cfg(merge_in_wg=2), None)
    assert rc == 1 and "needs zeroed arrival counters" in msg, msg
    # without the merge: both work buffers and the combine configuration are required
    rc, msg = run(lib.ae_decode_fwd, params(), cfg(), fake)
    assert rc == 1 and "work buffers are NULL" in msg, msg
    rc, msg = run(lib.ae_decode_fwd, params(partial_o=addr, partial_rs=addr), cfg(), fake, ccfg=False)
    assert rc == 1 and "combine configuration is NULL" in msg, msg


def test_block_table_geometry_is_checked_before_any_launch():
    """mask_mode 2: both prefill launches refuse a table whose blocks do not fit the kernel's tiles - rows that
    neither divide nor are divided by the q tile, columns that are not whole kv tiles, and more table rows per q
    tile than the kernel keeps masks for (ae_tile_cfg.table_rows, the AE_TT_ROWS it was compiled with): such a
    kernel would apply the classes of its last table row to every further row of the q tile."""
    lib = rt.lib()
    fake = ctypes.c_void_p(8)
    buf = ctypes.create_string_buffer(64)
    addr = ctypes.addressof(buf)

    def params(**kw):
        p = rt.AttnParams()
        p.q = p.k = p.v = p.out = p.block_mask = p.partial_o = p.partial_rs = addr
        p.batch, p.heads_q, p.heads_kv, p.seqlen_q, p.seqlen_kv = 1, 8, 8, 256, 1024
        p.mask_b, p.mask_h, p.mask_nq, p.mask_nkv, p.mask_block_m, p.mask_block_n = 1, 1, 8, 16, 32, 64
        p.num_splits, p.kv_per_split = 2, 512
        p.o_stride_h, p.o_stride_s, p.o_stride_b = 64, 8 * 64, 256 * 8 * 64
        for k, v in kw.items():
            setattr(p, k, v)
        return p

    def cfg(**kw):
        c = rt.TileCfg(block_m=128, block_n=64, threads=256, lds_bytes=1024, head_dim=64, head_dim_v=64,
                       elem_bytes=2, n_rowscales=0, mask_mode=2, table_rows=4)
        for k, v in kw.items():
            setattr(c, k, v)
        return c

    def fwd(p, c):
        rc = lib.ae_prefill_fwd(fake, ctypes.byref(p), ctypes.byref(c), None)
        return rc, lib.ae_last_error().decode()

    def split(p, c):
        cc = rt.TileCfg(block_m=1, block_n=p.num_splits, threads=128)
        rc = lib.ae_prefill_split_fwd(fake, fake, ctypes.byref(p), ctypes.byref(c), ctypes.byref(cc), None)
        return rc, lib.ae_last_error().decode()

    for launch in (fwd, split):
        rc, msg = launch(params(), cfg(table_rows=1))            # 128-row tile over 32-row blocks: 4 rows
        assert rc == 1 and "spans 4 rows" in msg and "compiled for 1" in msg, msg
        rc, msg = launch(params(), cfg(table_rows=2))
        assert rc == 1 and "compiled for 2" in msg, msg
        rc, msg = launch(params(mask_block_m=8, mask_nq=32), cfg(table_rows=0))     # 16 rows > the default of 8
        assert rc == 1 and "spans 16 rows" in msg and "compiled for 8" in msg, msg
        rc, msg = launch(params(mask_block_m=48, mask_nq=6), cfg())
        assert rc == 1 and "incompatible with tile" in msg, msg
        rc, msg = launch(params(mask_block_n=96, mask_nkv=11), cfg())
        assert rc == 1 and "not a multiple of the 64-key kv tile" in msg, msg
        rc, msg = launch(params(), cfg(table_rows=-1))
        assert rc == 1 and "table_rows=-1" in msg, msg


def test_misaligned_tensors_are_refused_before_any_launch():
    """The kernels move rows 16 bytes at a time: a tensor that does not start on a 16-byte boundary, or whose
    strides are not multiples of 8 elements, is refused by the argument checks (the Python operators copy such
    views first, core/runtime/hip_rt.py::rows_for_kernels)."""
    lib = rt.lib()
    fake = ctypes.c_void_p(8)
    buf = ctypes.create_string_buffer(256)
    addr = (ctypes.addressof(buf) + 15) & ~15

    def params(**kw):
        p = rt.AttnParams()
        p.q = p.k = p.v = p.out = addr
        p.batch, p.heads_q, p.heads_kv, p.seqlen_q, p.seqlen_kv = 1, 2, 2, 64, 64
        p.q_stride_b = p.k_stride_b = p.v_stride_b = p.o_stride_b = 64 * 2 * 64
        p.q_stride_s = p.k_stride_s = p.v_stride_s = p.o_stride_s = 2 * 64
        p.q_stride_h = p.k_stride_h = p.v_stride_h = p.o_stride_h = 64
        for k, v in kw.items():
            setattr(p, k, v)
        return p

    cfg = rt.TileCfg(block_m=128, block_n=64, threads=256, lds_bytes=1024, head_dim=64, head_dim_v=64,
                     elem_bytes=2, n_rowscales=0, mask_mode=0)
    for bad in (dict(q=addr + 8), dict(out=addr + 2), dict(k_stride_s=2 * 64 + 4), dict(v_stride_h=60)):
        assert lib.ae_prefill_fwd(fake, ctypes.byref(params(**bad)), ctypes.byref(cfg), None) == 1, bad
        msg = lib.ae_last_error().decode()
        assert "16-byte boundary" in msg or "not a multiple of 8" in msg, msg
    bp = rt.AttnBwdParams()
    for name in ("q", "k", "v", "out", "dout", "delta", "dq", "dk", "dv"):
        setattr(bp, name, addr)
    bp.batch, bp.heads_q, bp.heads_kv, bp.seqlen_q, bp.seqlen_kv = 1, 2, 2, 64, 64
    bp.dq = addr + 4
    bcfg = rt.TileCfg(block_m=128, block_n=64, threads=256, lds_bytes=1024, head_dim=64, head_dim_v=64,
                      elem_bytes=2, n_rowscales=0, mask_mode=0)
    assert lib.ae_prefill_bwd(fake, fake, fake, ctypes.byref(bp), ctypes.byref(bcfg), None) == 1
    assert "16-byte boundary" in lib.ae_last_error().decode()


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-GPU behaviour")
def test_no_gpu_is_reported_not_hidden():
    lib = rt.lib()
    assert lib.ae_device_count() == 0
    rc, h = _compile(KERNEL)
    assert rc == 0
    k = ctypes.c_void_p()
    assert lib.ae_module_get_kernel(h, b"ae_probe", ctypes.byref(k)) == 3     # AE_ERR_HIP
    assert b"failed" in lib.ae_last_error()
    lib.ae_module_free(h)
    with pytest.raises(rt.AEError):
        rt.device_info(0)


def test_code_object_cache_is_keyed_by_content(tmp_path, monkeypatch):
    monkeypatch.setenv("AE_CACHE_DIR", str(tmp_path))
    import __graft_entry__ as G
    (template, headers) = [th for th in G.representative_headers() if th[0] == "ae_decode.hip"][0]
    rt._modules.clear()
    m1 = rt.compile_module(template, headers)
    assert not m1.from_cache and len(os.listdir(tmp_path)) == 1
    rt._modules.clear()
    m2 = rt.compile_module(template, headers)
    assert m2.from_cache and m2.code() == m1.code()
    headers2 = dict(headers)
    headers2["ae_config.h"] = headers["ae_config.h"].replace("#define AE_NSPLIT 16", "#define AE_NSPLIT 8")
    m3 = rt.compile_module(template, headers2)
    assert not m3.from_cache and m3.key != m1.key
    rt._modules.clear()


def test_benchmarked_kernels_do_not_spill_registers():
    """The code objects hipRTC builds for the benchmark configurations (and the backward of the causal one) keep
    every value in registers: a kernel that spills pays for it with scratch-memory traffic in every workgroup, and
    an offline hipcc of another ROCm release does not show what this compiler does."""
    import __graft_entry__ as G
    engines = G.benchmark_engines()
    mods = {}
    for name, eng in engines.items():
        op = eng._op
        for key, v in op._variants.items():
            mods[f"{name}{key}"] = v[0]
    bwd = engines["c2_softmax_causal"]._op.backward_op()
    m_dq, m_dkv, _ = bwd._variant(1, False)
    mods["c2_bwd_dq"], mods["c2_bwd_dkv"] = m_dq, m_dkv
    assert len(mods) >= 8
    for name, m in mods.items():
        info = m.kernel_info()
        assert info, name
        for kname, k in info.items():
            assert k[".vgpr_spill_count"] == 0 and k[".sgpr_spill_count"] == 0, (name, kname, k[".vgpr_spill_count"])
            assert k[".private_segment_fixed_size"] == 0, (name, kname)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("causal", [True, False])
def test_prefill_kernels_keep_their_arrays_in_registers(dtype, D, causal):
    """The pipelined and the generic kernel of the softmax prefill, both input types: no scratch memory beyond a few
    spilled single values (some bf16 builds of the pipelined kernel at head dim 128), and never a register tuple in
    scratch memory -- the form of spill that once returned wrong columns (hip_rt.check_spills refuses it).  (A lambda
    of a kernel that the inliner leaves as a function keeps the arrays it captures by reference in scratch memory:
    the larger bf16 builds of the pipelined kernel once ran 30 times slower for it.)"""
    import attn_cases as C
    from core import CustomIO, meta_tensor
    from core.lower.prefill_op import PrefillOp
    meta = (meta_tensor(2, 32, 2048, D, dtype=dtype),) * 3
    args = (meta, CustomIO({}), C.make_scale_score_mod(D ** -0.5), C.causal_mask if causal else None, C.OnlineSoftmax(),
            "-inf")
    base = PrefillOp(*args)
    for t in base._tune_candidates()[:2]:
        op = base if t == base.tiles else PrefillOp(*args, tiles=t)
        for key, (module, _, _) in op._variants.items():
            for kname, k in module.kernel_info().items():
                assert k[".private_segment_fixed_size"] <= 64, (t, key, kname, k[".private_segment_fixed_size"])
            assert module.scratch_accesses()["wide"] == 0, (t, key)
            if dtype == torch.float16:
                assert module.scratch_accesses() == {"single": 0, "wide": 0}, (t, key)


def test_a_kernel_that_spills_registers_is_refused():
    """hip_rt.check_spills: a code object that keeps vector registers in scratch memory is refused after
    compilation when the caller is strict about it (``allow_spills=False``, ``strict_spills``, AE_ALLOW_SPILLS=0) and
    reported with a warning otherwise; ``allow_spills=True`` / AE_ALLOW_SPILLS=1 switch the check off.  The kernel here
    is register-hungry on purpose: 600 values live across a barrier under a launch bound that leaves a wave 128
    registers."""
    src_dir = rt.KERNEL_DIR
    name = "_x_spill_guard_probe.hip"                      # (git-ignored name pattern of scratch kernels)
    path = os.path.join(src_dir, name)
    body = """
#ifndef __HIPCC_RTC__
#include <hip/hip_runtime.h>
#endif
#include "ae_config.h"
extern "C" __global__ __launch_bounds__(1024) void ae_hungry_kernel(float* p) {
  float x[AE_LIVE];
#pragma unroll
  for (int i = 0; i < AE_LIVE; i++) x[i] = p[threadIdx.x + 1024 * i];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < AE_LIVE; i++) p[threadIdx.x + 1024 * ((i * 7) % AE_LIVE)] += x[i] * x[(i * 13) % AE_LIVE];
}
"""
    with open(path, "w") as f:
        f.write(body)

    def small_spill(name):
        """A build that spills, however little (found by raising the number of live values)."""
        for live in (130, 140, 160, 200, 260):
            m = rt.compile_module(name, {"ae_config.h": f"#define AE_LIVE {live}\n"}, use_cache=False, allow_spills=True)
            if m.kernel_info()["ae_hungry_kernel"][".vgpr_spill_count"] > 0:
                return m
        pytest.skip("no spilling build found")
    try:
        small = rt.compile_module(name, {"ae_config.h": "#define AE_LIVE 8\n"}, use_cache=False)
        assert small.kernel_info()["ae_hungry_kernel"][".vgpr_spill_count"] == 0
        big = {"ae_config.h": "#define AE_LIVE 600\n"}
        with pytest.raises(rt.SpillError, match="spills vector registers") as e:
            rt.compile_module(name, big, use_cache=False, allow_spills=False)
        assert "ae_hungry_kernel" in str(e.value) and "allow_spills=True" in str(e.value)
        assert isinstance(e.value, rt.AEError)
        with pytest.raises(rt.SpillError):                       # the family of builds the operators mark
            rt.compile_module(name, big, use_cache=False, strict_spills=True)
        with pytest.warns(RuntimeWarning, match="spills vector registers"):     # the default: reported, not refused
            m = rt.compile_module(name, big, use_cache=False)
        assert m.kernel_info()["ae_hungry_kernel"][".vgpr_spill_count"] > 0 and m.scratch_accesses()["single"] > 0
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("error")
            rt.check_spills(m, name, allow_spills=True)
            os.environ["AE_ALLOW_SPILLS"] = "1"
            try:
                rt.check_spills(m, name)
            finally:
                os.environ["AE_ALLOW_SPILLS"] = "0"
            try:
                with pytest.raises(rt.SpillError):
                    rt.check_spills(m, name)
                with pytest.raises(rt.SpillError):               # ... and with it any spill at all
                    rt.check_spills(small_spill(name), name)
            finally:
                del os.environ["AE_ALLOW_SPILLS"]
    finally:
        os.remove(path)
        rt._modules.clear()


def test_a_prefill_engine_gives_way_to_the_generic_kernel_rather_than_spill(monkeypatch):
    """A build of the software-pipelined kernel that the spill guard refuses (``allow_spills=False``): where that
    kernel was the engine's own choice the engine compiles the generic kernel instead and says so; asked for explicitly
    (``tiles=``, as the tuner does) the refused build is an error, which the tuner passes over.  The case: bf16, head
    dim 128, causal -- a build that spills seven single values, which the guard accepts as it stands and objects to
    here because the test sets its limit on scratch bytes to zero."""
    import attn_cases as C
    from attn_engine import AttentionEngine
    from core import CustomIO, meta_tensor
    from core.lower import lower as L
    from core.lower.prefill_op import PrefillOp
    dtype = torch.bfloat16
    meta = (meta_tensor(2, 32, 4096, 128, dtype=dtype),) * 3
    args = (meta, CustomIO({}), C.make_scale_score_mod(128 ** -0.5), C.causal_mask, C.OnlineSoftmax())
    assert L.choose_prefill_tiles(128, 128, 4096, (0.1, "m", "r"), 64).template == "ae_prefill_pipe.hip"
    accepted = AttentionEngine(*args)
    assert accepted._op.tiles.template == "ae_prefill_pipe.hip"
    (module, _, _), = accepted._op._variants.values()
    acc = module.scratch_accesses()
    assert acc["wide"] == 0 and 0 < acc["single"] < 40
    monkeypatch.setattr(rt, "MAX_SCRATCH_BYTES", 0)
    rt._modules.clear()
    mod = AttentionEngine(*args, allow_spills=False)
    assert mod._op.tiles.template == "ae_prefill.hip" and mod._op.gave_way_to_generic
    assert "#define AE_WAVES_PER_EU 2" in mod.tl_code
    pipe = L.PrefillTiles(template="ae_prefill_pipe.hip", waves_per_eu=1, rows_per_wave=64)
    with pytest.raises(rt.SpillError, match="spills heavily"):
        PrefillOp(*args, "-inf", tiles=pipe, allow_spills=False)
    with pytest.warns(RuntimeWarning, match="spills heavily"):       # the default: reported, and the kernel stays
        assert AttentionEngine(*args)._op.tiles.template == "ae_prefill_pipe.hip"
    forced = AttentionEngine(*args, allow_spills=True)
    assert forced._op.tiles.template == "ae_prefill_pipe.hip"
    # fp16 fits the registers: nothing gives way
    f16 = AttentionEngine((meta_tensor(2, 32, 4096, 128, dtype=torch.float16),) * 3, *args[1:])
    assert f16._op.tiles.template == "ae_prefill_pipe.hip" and not getattr(f16._op, "gave_way_to_generic", False)
    rt._modules.clear()


def test_wide_value_head_builds_are_compiled_strictly(monkeypatch):
    """The configuration whose compiled code once returned a wrong pair of output columns (head dim 256, value head
    dim 512, sliding window, ragged tiles: a 16-register accumulator tuple went through scratch memory and came back
    with a stale register) does not spill as the kernel stands, and PrefillOp compiles that family of builds -- one
    launch over more than 256 value columns -- with the spill check set to refuse: a compiler that spills a tuple
    there again is an error, not a warning."""
    import attn_cases as C
    from core import CustomIO, meta_tensor
    from core.lower.prefill_op import PrefillOp
    seen = []
    real = rt.compile_module

    def spy(template, headers, *a, **kw):
        seen.append((template, kw.get("strict_spills", False)))
        return real(template, headers, *a, **kw)
    monkeypatch.setattr(rt, "compile_module", spy)
    S, D, DV, dt = 100, 256, 512, torch.float16
    meta = (meta_tensor(1, 1, S, D, dtype=dt), meta_tensor(1, 1, S, D, dtype=dt), meta_tensor(1, 1, S, DV, dtype=dt))
    op = PrefillOp(meta, CustomIO({}), C.make_scale_score_mod(D ** -0.5), C.make_sliding_window_mask(70),
                   C.OnlineSoftmax(), "-inf")
    (module, _, _), = op._variants.values()
    assert module.kernel_info()["ae_prefill_kernel"][".vgpr_spill_count"] == 0
    assert op.DV_launch == 512 and seen == [("ae_prefill.hip", True)]
    seen.clear()
    meta = (meta_tensor(1, 1, S, 128, dtype=dt),) * 3
    PrefillOp(meta, CustomIO({}), C.make_scale_score_mod(128 ** -0.5), C.causal_mask, C.OnlineSoftmax(), "-inf")
    assert seen and all(not strict for _, strict in seen)


@pytest.mark.parametrize("mask", [None, "causal", "window"])
@pytest.mark.parametrize("S", [128, 100])
def test_wide_value_heads_do_not_spill(mask, S):
    """Value head dim 512 (256 accumulator registers per lane): the builds keep everything in registers.  Their
    epilogue reads the accumulators block by block through volatile asm statements; as plain copies the compiler
    moved the reads of every block to the front, spilled one block - and in one build (tile table, ragged tiles)
    lost one of the sixteen registers on the way back."""
    import attn_cases as C
    from core import CustomIO, meta_tensor
    from core.lower.prefill_op import PrefillOp
    mask_mod = {None: None, "causal": C.causal_mask, "window": C.make_sliding_window_mask(70)}[mask]
    for D, dtype in ((256, torch.float16), (128, torch.bfloat16)):
        meta = (meta_tensor(1, 1, S, D, dtype=dtype), meta_tensor(1, 1, S, D, dtype=dtype),
                meta_tensor(1, 1, S, 512, dtype=dtype))
        op = PrefillOp(meta, CustomIO({}), C.make_scale_score_mod(D ** -0.5), mask_mod, C.OnlineSoftmax(), "-inf")
        assert op.DV_launch == 512
        for key, (module, _, _) in op._variants.items():
            k = module.kernel_info()["ae_prefill_kernel"]
            assert k[".vgpr_spill_count"] == 0 and k[".private_segment_fixed_size"] == 0, (D, dtype, mask, S, key)
