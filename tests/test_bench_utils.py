"""The example scripts' harness (benchmark/bench_utils.py) keeps the reference's call surface."""
import inspect

import pytest
import torch

import attentionengine_amd  # noqa: F401  (puts attn_engine / core / benchmark on sys.path)
from benchmark import bench_utils


def test_signatures_match_reference_call_sites():
    # attn_script/mha.py:77 `do_bench_attention(mod, B, H, S, D, DV, dtype=torch.bfloat16)`,
    # attn_script/sigmoidattn.py:66 `do_bench_sigmoidattn(mod, B, H, S, D, DV, dtype=..., requires_grad=True)`,
    # attn_script/reluattn.py:63 `do_bench_reluattn(mod, B, H, S, D, DV, dtype=..., requires_grad=True)`.
    p = list(inspect.signature(bench_utils.do_bench_attention).parameters)
    assert p[:7] == ["attn", "B", "H", "S", "D", "DV", "mod"]
    assert {"dtype", "seqlenq", "require_grad", "causal", "groupnum"} <= set(p)
    p = list(inspect.signature(bench_utils.do_bench_sigmoidattn).parameters)
    assert p[:6] == ["attn", "B", "H", "S", "D", "DV"] and {"dtype", "requires_grad"} <= set(p)
    p = list(inspect.signature(bench_utils.do_bench_reluattn).parameters)
    assert p[:6] == ["attn", "B", "H", "S", "D", "DV"] and {"dtype", "causal", "requires_grad"} <= set(p)


def test_check_close_and_print_debug(capsys):
    a = torch.arange(12, dtype=torch.float32).reshape(3, 4) + 1
    b = a.clone()
    assert bench_utils.check_close(a, b)
    b[1, 2] += 1.0
    assert not bench_utils.check_close(a, b)
    bench_utils.print_debug(a, b)
    out = capsys.readouterr().out
    assert "1 elements are not close." in out and "(1, 2)" in out


def test_eager_reference_is_softmax_attention():
    from oracle.attention_ref import softmax_attention
    torch.manual_seed(0)
    q, k, v = torch.randn(2, 16, 4, 8), torch.randn(2, 16, 2, 8), torch.randn(2, 16, 2, 8)
    for causal in (False, True):
        o = bench_utils._eager_attention(q, k, v, 8 ** -0.5, causal, chunk_heads=1)
        ref, _ = softmax_attention(q, k, v, causal=causal)
        assert torch.allclose(o, ref.to(o.dtype), atol=1e-5)


@pytest.mark.gpu
def test_do_bench_attention_runs_a_mha_script(capsys):
    import attn_cases as C
    from attn_engine import AttentionEngine
    from core import CustomIO, meta_tensor
    B, H, S, D = 1, 4, 512, 64
    meta = tuple(meta_tensor(B, H, S, D, dtype=torch.float16) for _ in range(3))
    mod = AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(1 / D ** 0.5),
                          mask_mod=C.causal_mask, online_func=C.OnlineSoftmax())
    lat, tf, lat_ref, _ = bench_utils.do_bench_attention(mod, B, H, S, D, D, dtype=torch.float16)
    out = capsys.readouterr().out
    assert "Max diff" in out and "hip:" in out
    assert lat > 0 and lat_ref > 0 and tf > 0


def _meta3(B, H, S, D, DV, dtype):
    from core import meta_tensor
    return (meta_tensor(B, H, S, D, dtype=dtype), meta_tensor(B, H, S, D, dtype=dtype),
            meta_tensor(B, H, S, DV, dtype=dtype))


def _diff_lines(out):
    """(not-close counts, max diffs) of every print_debug block in the captured text."""
    import re
    bad = [int(m) for m in re.findall(r"Total elements: \d+, Not close elements: (\d+)", out)]
    mx = [float(m) for m in re.findall(r"Max diff: ([0-9.eE+-]+) at index", out)]
    return bad, mx


@pytest.mark.gpu
def test_do_bench_sigmoidattn_runs_the_script_form(capsys):
    """attn_script/sigmoidattn.py through its harness (bench_utils.py:701-788 of the reference): causal
    sigmoid attention with the bias as 4th argument, forward and backward compared with eager torch."""
    import attn_cases as C
    from attn_engine import AttentionEngine
    from core import CustomIO
    B, H, S, D = 1, 4, 256, 64
    mod = AttentionEngine(_meta3(B, H, S, D, D, torch.float16), CustomIO({"softmax_bias": (1,)}),
                          score_mod=C.make_sigmoid_score_mod(), mask_mod=C.causal_mask,
                          online_func=C.OnlineIdentity())
    lat, tf, lat_ref, tf_ref = bench_utils.do_bench_sigmoidattn(mod, B, H, S, D, D, dtype=torch.float16,
                                                                requires_grad=True)
    out = capsys.readouterr().out
    bad, mx = _diff_lines(out)
    assert len(bad) == 4 and len(mx) == 4            # dq, dk, dv, then the forward output
    assert max(bad) == 0, out                       # every element within 1e-2 + 1 % (outputs reach ~50 here)
    assert "hip:" in out and "hip bwd:" in out and "eager torch:" in out
    assert lat > 0 and lat_ref > 0 and tf > 0 and tf_ref > 0


@pytest.mark.gpu
def test_do_bench_reluattn_runs_the_script_form(capsys):
    """attn_script/reluattn.py through its harness (bench_utils.py:949-1022 of the reference), with
    requires_grad=True as the script passes it."""
    import attn_cases as C
    from attn_engine import AttentionEngine
    from core import CustomIO
    B, H, S, D = 2, 3, 256, 64
    mod = AttentionEngine(_meta3(B, H, S, D, D, torch.float16), CustomIO({}),
                          score_mod=C.make_relu_score_mod(1 / D ** 0.5), mask_mod=None,
                          online_func=C.OnlineIdentity())
    lat, tf, lat_ref, tf_ref = bench_utils.do_bench_reluattn(mod, B, H, S, D, D, dtype=torch.float16,
                                                             requires_grad=True)
    out = capsys.readouterr().out
    bad, mx = _diff_lines(out)
    assert len(bad) == 4 and len(mx) == 4
    # relu attention sums ~S/2 positive terms of size ~0.4: fp16 results of size ~10, compared at 1e-2 + 1%
    assert max(bad) <= 4, out
    assert "hip:" in out and "hip bwd:" in out and "eager torch:" in out
    assert lat > 0 and lat_ref > 0 and tf > 0 and tf_ref > 0


@pytest.mark.gpu
def test_do_bench_retention_runs_the_script_form(capsys):
    """attn_script/retention.py through its harness (bench_utils.py:1025-1100 of the reference): the decay
    mask as 4th argument, value head dim twice the key head dim."""
    import attn_cases as C
    from attn_engine import AttentionEngine
    B, H, S, D, DV = 1, 2, 256, 64, 128
    dtype = torch.bfloat16
    mod = AttentionEngine(_meta3(B, H, S, D, DV, dtype), C.retention_custom_inputs(),
                          score_mod=C.retention_score_mod, mask_mod=C.causal_mask,
                          online_func=C.OnlineAbsNorm(), mask_value="0")
    lat, tf, lat_ref, tf_ref = bench_utils.do_bench_retention(mod, B, H, S, D, DV, dtype=dtype)
    out = capsys.readouterr().out
    bad, mx = _diff_lines(out)
    assert len(bad) == 1 and bad[0] == 0, out
    assert "hip:" in out and "eager torch:" in out
    assert lat > 0 and lat_ref > 0 and tf > 0 and tf_ref > 0
