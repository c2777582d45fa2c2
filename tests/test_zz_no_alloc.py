"""ae_decode_fwd_noalloc (the GQA split-KV decode on the library's built-in work buffer) against
ae_decode_fwd (caller-allocated work buffers), both through the C ABI: the same kernels in the same order,
so out and lse must be bit-identical -- on two calls in a row, the second on a smaller input that leaves
the first call's partials behind in the buffer, and again after the two paths have alternated."""
import math

import pytest
import torch

import attn_cases as C
from attn_engine import AttentionEngine
from core import CustomIO, meta_tensor
from core.runtime import hip_rt as rt

pytestmark = pytest.mark.gpu


def _engine(B, Hq, Hkv, Skv, D, dtype):
    meta = (meta_tensor(B, Hq, 1, D, dtype=dtype), meta_tensor(B, Hkv, Skv, D, dtype=dtype),
            meta_tensor(B, Hkv, Skv, D, dtype=dtype))
    return AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(1 / math.sqrt(D)), mask_mod=None,
                           online_func=C.OnlineSoftmax())


def _both(mod, q, k, v):
    op = mod.attention
    op.static_workspace = False
    out_a = mod(q, k, v).clone()                       # ae_decode_fwd, torch-allocated partial buffers
    lse_a = mod.final_rowscales["lse"].clone()
    op.static_workspace = True
    out_b = mod(q, k, v).clone()                       # ae_decode_fwd_noalloc
    lse_b = mod.final_rowscales["lse"].clone()
    op.static_workspace = False
    return out_a, lse_a, out_b, lse_b


def test_decode_on_the_built_in_work_buffer(cuda_device):
    dtype = torch.float16
    cases = [(8, 32, 8, 4096, 128),      # 32 partials per head: 4.2 MB of the 16 MiB buffer
             (2, 32, 8, 1000, 128),      # smaller, ragged KV: the buffer still holds the first call's partials
             (3, 8, 2, 333, 64),
             # 4 splits = the waves of one workgroup: the allocating path merges inside the workgroup (one launch,
             # no partial buffers), this entry point keeps the merge kernel -- two differently compiled split
             # kernels of one engine, which its kernel cache must keep apart
             (128, 32, 8, 777, 128)]
    for n, (B, Hq, Hkv, Skv, D) in enumerate(cases):
        print(f"case no-alloc decode B{B} Hq{Hq} Hkv{Hkv} Skv{Skv} D{D}", flush=True)
        q, k, v = (t.cuda() for t in C.make_inputs(B, 1, Skv, Hq, Hkv, D, D, dtype, seed=40 + n))
        mod = _engine(B, Hq, Hkv, Skv, D, dtype)
        n_split, _ = mod.attention.plan_splits(B, Hq, Hkv, Skv)
        need = B * Hq * n_split * (D + 1) * 4
        assert need <= rt.NOALLOC_SCRATCH_BYTES, need
        out_a, lse_a, out_b, lse_b = _both(mod, q, k, v)
        assert torch.isfinite(out_a).all() and torch.isfinite(lse_a).all()
        assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b), (B, Hq, Hkv, Skv, D)
        if n_split == mod.attention.N_WAVES:
            assert {k[2] for k in mod.attention._variants} == {True, False}, mod.attention._variants.keys()


def test_decode_too_large_for_the_built_in_work_buffer_is_refused(cuda_device):
    B, Hq, Hkv, Skv, D = 320, 32, 8, 128, 128            # 320*32*4 rows * 129 fp32 = 21 MB > 16 MiB
    dtype = torch.float16
    q, k, v = (t.cuda() for t in C.make_inputs(B, 1, Skv, Hq, Hkv, D, D, dtype, seed=7))
    mod = _engine(B, Hq, Hkv, Skv, D, dtype)
    n_split, _ = mod.attention.plan_splits(B, Hq, Hkv, Skv)
    assert B * Hq * n_split * (D + 1) * 4 > rt.NOALLOC_SCRATCH_BYTES
    mod.attention.static_workspace = True
    with pytest.raises(rt.AEError, match="built-in buffer holds"):
        mod(q, k, v)
    mod.attention.static_workspace = False
    assert torch.isfinite(mod(q, k, v)).all()          # the allocating entry point still takes it
