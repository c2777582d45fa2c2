"""Golden vectors of tests/golden/ (float64 numpy, written by tests/golden/make_golden.py
independently of oracle/): the CPU oracle must reproduce them, and so must the HIP path through
the C-ABI on the fp16 / bf16 cast of the same inputs."""
import os
import sys

import numpy as np
import pytest
import torch

import attn_cases as C
from attn_engine import AttentionEngine
from core import CustomIO, SymbolicTensor, create_block_mask, meta_tensor
from core.transform.core import is_causal_mask, is_less_causal_mask
from oracle import attention_ref as R
from oracle import masks as M

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
sys.path.insert(0, GOLDEN)
from golden_inputs import golden_tensor, qkv  # noqa: E402

OUT_TOL, LSE_TOL = 2e-2, 1e-3        # device bars (fp16 / bf16 storage)
ORACLE_TOL = 2e-5                    # fp32 oracle against float64 vectors


def _load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def _t(*arrays):
    return tuple(torch.from_numpy(a) for a in arrays)


def _maxdiff(a, b):
    return (torch.as_tensor(a).float().cpu() - torch.as_tensor(b).float()).abs().max().item()


# ---------------------------------------------------------------- CPU: oracle against the vectors
def test_oracle_c1_softmax_causal():
    g = _load("c1_softmax_causal.npz")
    q, k, v = _t(*qkv(1, 512, 512, 4, 4, 64, 64, int(g["stream"])))
    out, lse = R.softmax_attention(q, k, v, scale=float(g["scale"]), causal=True)
    assert _maxdiff(out[:, ::int(g["row_stride"])], g["out_rows"]) <= ORACLE_TOL
    assert _maxdiff(lse, g["lse"]) <= ORACLE_TOL


def test_oracle_full_and_window():
    g = _load("softmax_full_and_window.npz")
    q, k, v = _t(*qkv(1, 256, 256, 2, 2, 128, 128, int(g["stream"])))
    out, lse = R.softmax_attention(q, k, v, scale=float(g["scale"]))
    assert _maxdiff(out, g["out"]) <= ORACLE_TOL and _maxdiff(lse, g["lse"]) <= ORACLE_TOL
    mask = torch.from_numpy(M.dense_mask_grid(C.make_sliding_window_mask(int(g["window"])), 1, 2, 256, 256))
    out, lse = R.softmax_attention(q, k, v, scale=float(g["scale"]), mask=mask)
    assert _maxdiff(out, g["out_window"]) <= ORACLE_TOL and _maxdiff(lse, g["lse_window"]) <= ORACLE_TOL


def test_oracle_sigmoid():
    g = _load("sigmoid.npz")
    q, k, v = _t(*qkv(1, 256, 256, 2, 2, 128, 128, int(g["stream"])))
    assert _maxdiff(R.sigmoid_attention(q, k, v, scale=float(g["scale"]), bias=float(g["bias"])), g["out"]) <= ORACLE_TOL
    assert _maxdiff(R.sigmoid_attention(q, k, v, scale=float(g["scale"]), bias=float(g["bias"]), causal=True),
                    g["out_causal"]) <= ORACLE_TOL


def test_oracle_gqa_decode():
    g = _load("gqa_decode.npz")
    q, k, v = _t(*qkv(2, 1, 1000, 32, 8, 128, 128, int(g["stream"])))
    out, lse = R.softmax_attention(q, k, v, scale=float(g["scale"]))
    assert _maxdiff(out, g["out"]) <= ORACLE_TOL and _maxdiff(lse, g["lse"]) <= ORACLE_TOL


def _mla_golden_inputs(stream):
    return _t(golden_tensor((2, 1, 128, 512), stream), golden_tensor((2, 1, 128, 64), stream + 1),
              golden_tensor((2, 300, 1, 512), stream + 2), golden_tensor((2, 300, 1, 64), stream + 3))


def test_oracle_mla_decode():
    g = _load("mla_decode.npz")
    q, q_pe, kv, k_pe = _mla_golden_inputs(int(g["stream"]))
    out, lse = R.mla_decode(q[:, 0], q_pe[:, 0], kv, k_pe, scale=float(g["scale"]))
    assert _maxdiff(out, g["out"][:, 0]) <= ORACLE_TOL and _maxdiff(lse, g["lse"][:, :, 0]) <= ORACLE_TOL


def test_block_mask_known_answers_from_fixture():
    """attention_engine/tests/test_blockmask.py:3-10 at B2 H4 S512 with 128x64 blocks: the host
    block-mask builder and the oracle's brute force both give the hand-typed tables."""
    g = _load("blockmask_kat.npz")
    mods = {"causal": C.causal_mask, "causal_plus_one": C.causal_plus_one_mask,
            "causal_shifted_128": C.causal_shifted_mask}
    for i, name in enumerate(g["names"]):
        mod = mods[str(name)]
        want = torch.from_numpy(g[str(name)])
        got = create_block_mask(mod, 2, 4, 512, 512, "cpu", 128, 64)
        assert torch.equal(got.to(torch.int8).cpu(), want), name
        brute = M.block_any(M.dense_mask_grid(mod, 2, 4, 512, 512), 128, 64)
        assert np.array_equal(brute.astype(np.int8), g[str(name)]), name
        assert bool(is_causal_mask(got, 128, 64)) == bool(g["is_causal"][i]), name
        assert bool(is_less_causal_mask(got, 128, 64)) == bool(g["is_less_causal"][i]), name


# ---------------------------------------------------------------- GPU: HIP path against the vectors
def _prefill(q, k, v, dtype, score_mod, mask_mod, online, customs=None):
    B, S, H, D = q.shape
    meta = (meta_tensor(B, H, S, D, dtype=dtype), meta_tensor(B, k.shape[2], k.shape[1], D, dtype=dtype),
            meta_tensor(B, v.shape[2], v.shape[1], v.shape[3], dtype=dtype))
    return AttentionEngine(meta, customs if customs is not None else CustomIO({}), score_mod=score_mod,
                           mask_mod=mask_mod, online_func=online)


@pytest.mark.gpu
def test_hip_c1_softmax_causal(cuda_device):
    g = _load("c1_softmax_causal.npz")
    q, k, v = (t.half().cuda() for t in _t(*qkv(1, 512, 512, 4, 4, 64, 64, int(g["stream"]))))
    mod = _prefill(q, k, v, torch.float16, C.make_scale_score_mod(float(g["scale"])), C.causal_mask, C.OnlineSoftmax())
    out = mod(q, k, v)
    assert _maxdiff(out[:, ::int(g["row_stride"])], g["out_rows"]) <= OUT_TOL
    assert _maxdiff(mod.final_rowscales["lse"], g["lse"]) <= LSE_TOL


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_hip_full_and_window(cuda_device, dtype):
    g = _load("softmax_full_and_window.npz")
    q, k, v = (t.to(dtype).cuda() for t in _t(*qkv(1, 256, 256, 2, 2, 128, 128, int(g["stream"]))))
    sm = C.make_scale_score_mod(float(g["scale"]))
    mod = _prefill(q, k, v, dtype, sm, None, C.OnlineSoftmax())
    assert _maxdiff(mod(q, k, v), g["out"]) <= OUT_TOL
    assert _maxdiff(mod.final_rowscales["lse"], g["lse"]) <= LSE_TOL
    mod = _prefill(q, k, v, dtype, sm, C.make_sliding_window_mask(int(g["window"])), C.OnlineSoftmax())
    assert _maxdiff(mod(q, k, v), g["out_window"]) <= OUT_TOL
    assert _maxdiff(mod.final_rowscales["lse"], g["lse_window"]) <= LSE_TOL


@pytest.mark.gpu
def test_hip_sigmoid(cuda_device):
    g = _load("sigmoid.npz")
    q, k, v = (t.half().cuda() for t in _t(*qkv(1, 256, 256, 2, 2, 128, 128, int(g["stream"]))))
    bias = torch.tensor([float(g["bias"])], dtype=torch.float32, device="cuda")
    for mask_mod, key in ((None, "out"), (C.causal_mask, "out_causal")):
        customs = CustomIO({"softmax_bias": (1,)})
        mod = _prefill(q, k, v, torch.float16, C.make_sigmoid_score_mod(float(g["scale"])), mask_mod,
                       C.OnlineIdentity(), customs)
        assert _maxdiff(mod(q, k, v, bias), g[key]) <= OUT_TOL


@pytest.mark.gpu
def test_hip_gqa_decode(cuda_device):
    g = _load("gqa_decode.npz")
    q, k, v = (t.half().cuda() for t in _t(*qkv(2, 1, 1000, 32, 8, 128, 128, int(g["stream"]))))
    meta = (meta_tensor(2, 32, 1, 128, dtype=torch.float16), meta_tensor(2, 8, 1000, 128, dtype=torch.float16),
            meta_tensor(2, 8, 1000, 128, dtype=torch.float16))
    mod = AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(float(g["scale"])), mask_mod=None,
                          online_func=C.OnlineSoftmax())
    assert _maxdiff(mod(q, k, v), g["out"]) <= OUT_TOL
    assert _maxdiff(mod.final_rowscales["lse"], g["lse"]) <= LSE_TOL


@pytest.mark.gpu
def test_hip_mla_decode(cuda_device):
    g = _load("mla_decode.npz")
    q, q_pe, kv, k_pe = (t.bfloat16().cuda() for t in _mla_golden_inputs(int(g["stream"])))
    meta = (meta_tensor(2, 128, 1, 576, dtype=torch.bfloat16), meta_tensor(2, 1, 300, 576, dtype=torch.bfloat16),
            meta_tensor(2, 1, 300, 512, dtype=torch.bfloat16))
    mod = AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(float(g["scale"])), mask_mod=None,
                          online_func=C.OnlineSoftmax(), kv_shared=True)
    assert _maxdiff(mod(q, q_pe, kv, k_pe), g["out"]) <= OUT_TOL
    assert _maxdiff(mod.final_rowscales["lse"], g["lse"]) <= LSE_TOL
