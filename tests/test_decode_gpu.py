"""GPU parity of the split-KV decode path (GQA) against the CPU oracle, through
AttentionEngine -> libae_hip.so.  Tolerances: out <= 2e-2, lse <= 1e-3 (natural log, fp32)."""
import math

import pytest
import torch

import attn_cases as C
from attn_engine import AttentionEngine
from core import CustomIO, meta_tensor
from oracle import attention_ref as R

pytestmark = pytest.mark.gpu

OUT_TOL = 2e-2
LSE_TOL = 1e-3


def _decode_engine(B, Hq, Hkv, Skv, D, DV, dtype, score_mod, online, **kw):
    meta = (meta_tensor(B, Hq, 1, D, dtype=dtype), meta_tensor(B, Hkv, Skv, D, dtype=dtype),
            meta_tensor(B, Hkv, Skv, DV, dtype=dtype))
    return AttentionEngine(meta, CustomIO({}), score_mod=score_mod, mask_mod=None, online_func=online, **kw)


@pytest.mark.parametrize("B,Hq,Hkv,Skv,D,dtype", [
    (2, 32, 8, 1024, 128, torch.float16),     # Llama-3.1-8B head layout (BASELINE config 4, short KV)
    (1, 32, 8, 8192, 128, torch.float16),     # attn_script/gqa_inference.py shape
    (3, 8, 2, 1000, 128, torch.bfloat16),     # ragged KV length
    (2, 40, 2, 96, 64, torch.float16),        # 20 heads per group: two head tiles; fewer tiles than waves
    (1, 4, 1, 33, 128, torch.float16),
])
def test_gqa_decode(cuda_device, B, Hq, Hkv, Skv, D, dtype):
    print(f"case gqa decode B{B} Hq{Hq} Hkv{Hkv} Skv{Skv} D{D} {dtype}", flush=True)
    q, k, v = C.make_inputs(B, 1, Skv, Hq, Hkv, D, D, dtype)
    mod = _decode_engine(B, Hq, Hkv, Skv, D, D, dtype, C.make_scale_score_mod(1 / math.sqrt(D)), C.OnlineSoftmax())
    out = mod(q.cuda(), k.cuda(), v.cuda())
    ref, lse = R.softmax_attention(q, k, v, causal=False)
    assert out.shape == (B, 1, Hq, D) and out.dtype == dtype
    assert (out.float().cpu() - ref).abs().max().item() <= OUT_TOL
    assert (mod.final_rowscales["lse"].cpu() - lse).abs().max().item() <= LSE_TOL


def test_gqa_decode_full_size_properties(cuda_device):
    """BASELINE config 4 at full size (B64 Hq32 Hkv8 Skv8192 D128 fp16).  Checked against the oracle
    on two batch entries, and everywhere through linearity in V: decode(q, k, a*v1 + v2) ==
    a*decode(q, k, v1) + decode(q, k, v2) while lse does not depend on V."""
    B, Hq, Hkv, Skv, D = 64, 32, 8, 8192, 128
    dtype = torch.float16
    q, k, v = C.make_inputs(B, 1, Skv, Hq, Hkv, D, D, dtype)
    mod = _decode_engine(B, Hq, Hkv, Skv, D, D, dtype, C.make_scale_score_mod(1 / math.sqrt(D)), C.OnlineSoftmax())
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    out = mod(qc, kc, vc)
    lse = mod.final_rowscales["lse"].clone()
    for b in (0, 63):
        ref, lref = R.softmax_attention(q[b:b + 1], k[b:b + 1], v[b:b + 1], causal=False)
        assert (out[b:b + 1].float().cpu() - ref).abs().max().item() <= OUT_TOL
        assert (lse[b:b + 1].cpu() - lref).abs().max().item() <= LSE_TOL
    v2 = torch.flip(vc, dims=[1])
    out2 = mod(qc, kc, v2)
    assert torch.equal(mod.final_rowscales["lse"], lse)
    out3 = mod(qc, kc, (0.5 * vc + v2))
    assert (out3.float() - (0.5 * out.float() + out2.float())).abs().max().item() <= 1e-2


def test_gqa_decode_sigmoid(cuda_device):
    """A non-softmax decode: identity rowscales, combine() = 1 (plain sum of the partials)."""
    B, Hq, Hkv, Skv, D = 2, 8, 2, 512, 128
    dtype = torch.float16

    def sig(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        return (((score * (1 / math.sqrt(D)) - 6.0) * 0.5).tanh() + 1) * 0.5
    q, k, v = C.make_inputs(B, 1, Skv, Hq, Hkv, D, D, dtype)
    mod = _decode_engine(B, Hq, Hkv, Skv, D, D, dtype, sig, C.OnlineIdentity())
    out = mod(q.cuda(), k.cuda(), v.cuda())
    ref = R.sigmoid_attention(q, k, v, bias=-6.0)
    assert (out.float().cpu() - ref).abs().max().item() <= OUT_TOL
