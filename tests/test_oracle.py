"""Pins the CPU oracle (oracle/) without any GPU: closed forms against library routines,
pure-python brute force on tiny inputs, algebraic invariants, and the hand-derived block-mask
known answers for the reference's own mask test cases."""
import math

import numpy as np
import pytest
import torch

import attn_cases as C
from oracle import attention_ref as R
from oracle import masks as M
from oracle.online_interp import combine_partials, online_attention


def _loop_attention(q, k, v, scale, p_fn, causal=False):
    """Pure-python reference: explicit loops over batch, head, query, key."""
    B, Sq, Hq, D = q.shape
    Skv, Hkv, DV = k.shape[1], k.shape[2], v.shape[3]
    G = Hq // Hkv
    out = torch.zeros(B, Sq, Hq, DV, dtype=torch.float64)
    lse = torch.zeros(B, Hq, Sq, dtype=torch.float64)
    for b in range(B):
        for h in range(Hq):
            for i in range(Sq):
                s = []
                for j in range(Skv):
                    if causal and j > i:
                        s.append(-math.inf)
                    else:
                        s.append(sum(float(q[b, i, h, d]) * float(k[b, j, h // G, d]) for d in range(D)) * scale)
                w, l = p_fn(s)
                lse[b, h, i] = l
                for j in range(Skv):
                    if w[j] != 0.0:
                        out[b, i, h] += w[j] * v[b, j, h // G].double()
    return out, lse


def _softmax_weights(s):
    m = max(s)
    e = [math.exp(x - m) if x != -math.inf else 0.0 for x in s]
    z = sum(e)
    return [x / z for x in e], math.log(z) + m


def test_softmax_matches_python_loops():
    q, k, v = C.make_inputs(1, 6, 6, 4, 2, 8, 8, torch.float32, seed=1)
    for causal in (False, True):
        ref, lref = _loop_attention(q, k, v, 1 / math.sqrt(8), _softmax_weights, causal)
        out, lse = R.softmax_attention(q, k, v, causal=causal, compute_dtype=torch.float64)
        assert torch.allclose(out, ref, atol=1e-12)
        assert torch.allclose(lse, lref, atol=1e-12)


@pytest.mark.parametrize("causal", [False, True])
def test_softmax_matches_torch_sdpa(causal):
    """Library cross-check: F.scaled_dot_product_attention on [B,H,S,D] operands."""
    q, k, v = C.make_inputs(2, 96, 96, 4, 4, 32, 32, torch.float32, seed=2)
    out, lse = R.softmax_attention(q, k, v, causal=causal)
    sd = torch.nn.functional.scaled_dot_product_attention(
        q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3), is_causal=causal)
    assert torch.allclose(out, sd.permute(0, 2, 1, 3), atol=2e-6)
    s = torch.einsum("bqhd,bkhd->bhqk", q, k) / math.sqrt(32)
    if causal:
        s = s.masked_fill(~torch.ones(96, 96, dtype=torch.bool).tril(), -math.inf)
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=1e-5)


def test_softmax_gqa_equals_repeated_heads():
    q, k, v = C.make_inputs(1, 40, 40, 8, 2, 16, 16, torch.float32, seed=3)
    out, lse = R.softmax_attention(q, k, v, causal=True)
    kr, vr = k.repeat_interleave(4, dim=2), v.repeat_interleave(4, dim=2)
    out2, lse2 = R.softmax_attention(q, kr, vr, causal=True)
    assert torch.allclose(out, out2, atol=1e-6) and torch.allclose(lse, lse2, atol=1e-6)


def test_softmax_with_all_ones_v_returns_ones():
    """Rows of P sum to one: V = 1 gives out = 1 for every row that sees a key."""
    q, k, _ = C.make_inputs(1, 33, 33, 2, 2, 16, 16, torch.float32, seed=4)
    v = torch.ones(1, 33, 2, 16)
    out, _ = R.softmax_attention(q, k, v, causal=True)
    assert torch.allclose(out, torch.ones_like(out), atol=1e-6)


def test_fully_masked_rows():
    q, k, v = C.make_inputs(1, 8, 8, 1, 1, 4, 4, torch.float32, seed=5)
    mask = torch.ones(8, 8, dtype=torch.bool).tril()
    mask[:3] = False
    out, lse = R.softmax_attention(q, k, v, mask=mask)
    assert torch.equal(out[:, :3], torch.zeros_like(out[:, :3]))
    assert torch.isneginf(lse[..., :3]).all() and torch.isfinite(lse[..., 3:]).all()


def test_sigmoid_and_relu_match_python_loops():
    q, k, v = C.make_inputs(1, 5, 7, 2, 1, 8, 8, torch.float32, seed=6)
    scale, bias = 1 / math.sqrt(8), -1.5
    ref, _ = _loop_attention(q, k, v, scale, lambda s: ([1 / (1 + math.exp(-(x + bias))) for x in s], 0.0))
    assert torch.allclose(R.sigmoid_attention(q, k, v, bias=bias, compute_dtype=torch.float64), ref, atol=1e-12)
    ref, _ = _loop_attention(q, k, v, scale, lambda s: ([max(x, 0.0) for x in s], 0.0))
    assert torch.allclose(R.relu_attention(q, k, v, compute_dtype=torch.float64), ref, atol=1e-12)
    # the script's tanh form is the same function (attn_script/sigmoidattn.py:14-18)
    x = torch.linspace(-20, 20, 401, dtype=torch.float64)
    assert torch.allclose(((x * 0.5).tanh() + 1) * 0.5, torch.sigmoid(x), atol=1e-15)


def test_mla_equals_concatenated_softmax_and_loops():
    g = torch.Generator().manual_seed(7)
    B, H, S, DV, DPE = 2, 6, 9, 8, 4
    q, qpe = torch.randn(B, H, DV, generator=g), torch.randn(B, H, DPE, generator=g)
    kv, kpe = torch.randn(B, S, 1, DV, generator=g), torch.randn(B, S, 1, DPE, generator=g)
    out, lse = R.mla_decode(q, qpe, kv, kpe, compute_dtype=torch.float64)
    qq = torch.cat([q, qpe], -1).unsqueeze(1)
    kk = torch.cat([kv, kpe], -1)
    ref, lref = _loop_attention(qq, kk, kv, 1 / math.sqrt(DV + DPE), _softmax_weights)
    assert torch.allclose(out, ref[:, 0], atol=1e-12) and torch.allclose(lse, lref[:, :, 0], atol=1e-12)


@pytest.mark.parametrize("cuts", [[0, 5, 17, 40], [0, 1, 2, 40], [0, 40], [0, 13, 26, 39, 40]])
def test_merge_of_partials_equals_unsplit(cuts):
    q, k, v = C.make_inputs(2, 1, 40, 4, 2, 16, 16, torch.float32, seed=8)
    full, lfull = R.softmax_attention(q, k, v, compute_dtype=torch.float64)
    po, pl = [], []
    for a, b in zip(cuts[:-1], cuts[1:]):
        o, l = R.softmax_attention(q, k[:, a:b], v[:, a:b], compute_dtype=torch.float64)
        po.append(o[:, 0])
        pl.append(l[:, :, 0])
    o, l = R.merge_partials(torch.stack(po, dim=-2), torch.stack(pl, dim=-1))
    assert torch.allclose(o, full[:, 0], atol=1e-12) and torch.allclose(l, lfull[:, :, 0], atol=1e-12)
    # the traced combine() of the scripts gives the same weights
    on = C.OnlineSoftmax()
    o2 = combine_partials(on, torch.stack(po, 0).reshape(len(po), -1, 16),
                          {"lse": torch.stack(pl, 0).reshape(len(pl), -1)})
    assert torch.allclose(o2.reshape(full[:, 0].shape), full[:, 0], atol=1e-12)


@pytest.mark.parametrize("block_n", [16, 32, 64, 128])
def test_online_interpreter_is_block_size_invariant(block_n):
    q, k, v = C.make_inputs(1, 96, 96, 2, 1, 16, 16, torch.float32, seed=9)
    sm = C.make_scale_score_mod(0.25)
    out, fin = online_attention(q, k, v, sm, C.causal_mask, C.OnlineSoftmax(), block_n=block_n)
    ref, lse = R.softmax_attention(q, k, v, causal=True, compute_dtype=torch.float64)
    assert torch.allclose(out, ref, atol=1e-10) and torch.allclose(fin["lse"], lse, atol=1e-10)


def test_online_interpreter_sigmoid_and_sliding_window():
    q, k, v = C.make_inputs(1, 64, 64, 2, 2, 16, 16, torch.float32, seed=10)
    bias = torch.tensor([-2.0])
    from core import CustomIO
    out, fin = online_attention(q, k, v, C.make_sigmoid_score_mod(0.25), None, C.OnlineIdentity(),
                                custom_fwd_inputs=CustomIO({"softmax_bias": (1,)}), custom_tensors=[bias])
    assert fin == {}
    assert torch.allclose(out, R.sigmoid_attention(q, k, v, scale=0.25, bias=-2.0, compute_dtype=torch.float64),
                          atol=1e-10)
    win = C.make_sliding_window_mask(10)
    out, _ = online_attention(q, k, v, C.make_scale_score_mod(0.25), win, C.OnlineSoftmax(), block_n=16)
    dense = torch.from_numpy(M.dense_mask_grid(win, 1, 2, 64, 64))
    ref, _ = R.softmax_attention(q, k, v, scale=0.25, mask=dense, compute_dtype=torch.float64)
    assert torch.allclose(out, ref, atol=1e-10)


# ---- masks -----------------------------------------------------------------------------------------
def test_grid_mask_equals_python_loop_mask():
    for mm in (C.causal_mask, C.causal_plus_one_mask, C.head_dependent_mask):
        assert np.array_equal(M.dense_mask(mm, 2, 3, 17, 19), M.dense_mask_grid(mm, 2, 3, 17, 19))


# Known answers hand-derived from core/transform/core.py:410-488 for the masks of
# attention_engine/tests/test_blockmask.py:3-10 at B=2, H=4, S=512, 128 x 64 blocks: the LAST non-zero
# kv block of each of the 4 q-block rows (-1 = row empty), is_causal_mask, is_less_causal_mask.
BLOCKMASK_KAT = [
    (C.causal_mask, [1, 3, 5, 7], True, True),
    (C.causal_plus_one_mask, [2, 4, 6, 7], False, False),
    (C.causal_shifted_mask, [-1, 1, 3, 5], False, True),
]


@pytest.mark.parametrize("mask_mod,last,is_causal,is_less", BLOCKMASK_KAT)
def test_block_mask_known_answers(mask_mod, last, is_causal, is_less):
    blocks = M.block_any(M.dense_mask_grid(mask_mod, 2, 4, 512, 512), 128, 64)
    assert blocks.shape == (2, 4, 4, 8)
    expect = np.zeros((4, 8), dtype=np.int8)
    for i, l in enumerate(last):
        expect[i, :l + 1] = 1
    assert np.array_equal(blocks, np.broadcast_to(expect, blocks.shape))
    assert bool(np.array_equal(blocks[0, 0].astype(bool), M.block_causal_pattern(4, 8, 128, 64))) == is_causal
    assert M.no_block_above_diagonal(blocks, 128, 64) == is_less


def test_block_classes_brute_force():
    def mm(b, h, q_idx, kv_idx):          # python-int friendly sliding window
        return (q_idx >= kv_idx) and (q_idx < kv_idx + 20)
    dense = M.dense_mask(mm, 1, 1, 40, 40)
    cls = M.block_classes(dense, 16, 8)
    for i in range(3):
        for j in range(5):
            blk = dense[0, 0, i * 16:(i + 1) * 16, j * 8:(j + 1) * 8]
            want = 0 if not blk.any() else (2 if blk.all() else 1)
            assert cls[0, 0, i, j] == want


def test_retention_closed_form_loops_and_running_form():
    """Retention with a decay mask (bench_utils.py:1062-1067): python loops on a tiny case, and the
    running form of attn_script/retention.py:32-58 (abs-sum, clamp at 1, o_scale = r / r_new) run
    tile by tile through the DAG interpreter telescopes to the same result for any tile width."""
    B, S, H, D, DV = 1, 9, 2, 8, 4
    q, k, v = C.make_inputs(B, S, S, H, H, D, DV, torch.float32, seed=8)
    g = torch.Generator().manual_seed(9)
    # rows both below and above the clamp
    mask = torch.rand(1, H, S, S, generator=g).tril() * torch.linspace(0.01, 3.0, S).view(1, 1, S, 1)
    out, r = R.retention_attention(q, k, v, mask, compute_dtype=torch.float64)
    for h in range(H):
        for i in range(S):
            s = [sum(float(q[0, i, h, d]) * float(k[0, j, h, d]) for d in range(D)) * float(mask[0, h, i, j])
                 for j in range(S)]
            rr = max(sum(abs(x) for x in s), 1.0)
            assert abs(float(r[0, h, i]) - rr) < 1e-9
            for c in range(DV):
                ref = sum(s[j] / rr * float(v[0, j, h, c]) for j in range(S))
                assert abs(float(out[0, i, h, c]) - ref) < 1e-9
    assert (r > 1.0).any() and (r == 1.0).any()
    for bn in (2, 4, 16):
        o2, fin = online_attention(q, k, v, C.retention_score_mod, C.causal_mask, C.OnlineAbsNorm(),
                                   custom_fwd_inputs=C.retention_custom_inputs(), custom_tensors=(mask,),
                                   block_n=bn, mask_value="0")
        assert torch.allclose(o2, out, atol=1e-12) and torch.allclose(fin["r"], r, atol=1e-12)


def test_softmax_gradients_match_autograd():
    """The closed-form backward against torch.autograd through the closed-form forward (fp64), with
    grouped heads, causal and an arbitrary mask with one fully masked row."""
    g = torch.Generator().manual_seed(5)
    B, Sq, Skv, Hq, Hkv, D, DV = 2, 9, 13, 4, 2, 8, 6
    q = torch.randn(B, Sq, Hq, D, generator=g, dtype=torch.float64, requires_grad=True)
    k = torch.randn(B, Skv, Hkv, D, generator=g, dtype=torch.float64, requires_grad=True)
    v = torch.randn(B, Skv, Hkv, DV, generator=g, dtype=torch.float64, requires_grad=True)
    do = torch.randn(B, Sq, Hq, DV, generator=g, dtype=torch.float64)
    mask = torch.rand(B, Hq, Sq, Skv, generator=g) > 0.3
    mask[0, 1, 4] = False
    for kw in (dict(), dict(causal=True), dict(mask=mask), dict(scale=0.37, causal=True)):
        out, _ = R.softmax_attention(q, k, v, compute_dtype=torch.float64, **kw)
        gq, gk, gv = torch.autograd.grad(out, (q, k, v), do)
        dq, dk, dv = R.softmax_attention_grads(q.detach(), k.detach(), v.detach(), do,
                                               compute_dtype=torch.float64, **kw)
        for a, b in ((dq, gq), (dk, gk), (dv, gv)):
            assert torch.allclose(a, b, atol=1e-12, rtol=1e-10)


def test_elementwise_gradients_match_autograd():
    """Closed-form backward of sigmoid and relu attention against torch.autograd through the closed-form
    forwards (fp64)."""
    g = torch.Generator().manual_seed(6)
    B, Sq, Skv, Hq, Hkv, D, DV = 2, 7, 11, 4, 2, 8, 6
    q = torch.randn(B, Sq, Hq, D, generator=g, dtype=torch.float64, requires_grad=True)
    k = torch.randn(B, Skv, Hkv, D, generator=g, dtype=torch.float64, requires_grad=True)
    v = torch.randn(B, Skv, Hkv, DV, generator=g, dtype=torch.float64, requires_grad=True)
    do = torch.randn(B, Sq, Hq, DV, generator=g, dtype=torch.float64)
    for kind, fwd, kw in (("sigmoid", R.sigmoid_attention, dict(bias=-0.7, causal=True, scale=0.4)),
                          ("sigmoid", R.sigmoid_attention, dict(bias=0.3)),
                          ("relu", R.relu_attention, dict(scale=0.3))):
        out = fwd(q, k, v, compute_dtype=torch.float64, **kw)
        gq, gk, gv = torch.autograd.grad(out, (q, k, v), do)
        dq, dk, dv = R.elementwise_attention_grads(q.detach(), k.detach(), v.detach(), do, kind,
                                                   compute_dtype=torch.float64, **kw)
        for a, b in ((dq, gq), (dk, gk), (dv, gv)):
            assert torch.allclose(a, b, atol=1e-12, rtol=1e-10)


def test_retention_gradients_match_autograd_with_a_constant_row_scale():
    """The backward rule of attn_script/retention.py:60-70 treats the saved row scale r as a constant: the
    oracle's closed-form gradients against torch.autograd through out = ((q k^T) * mask / r.detach()) v in
    fp64, with grouped heads and rows on both sides of the clamp (some r = 1, some r > 1).  With r
    differentiated as well, autograd gives something else -- checked, so the test cannot pass vacuously."""
    g = torch.Generator().manual_seed(8)
    B, Sq, Skv, Hq, Hkv, D, DV = 2, 9, 9, 4, 2, 8, 6
    q = torch.randn(B, Sq, Hq, D, generator=g, dtype=torch.float64, requires_grad=True)
    k = torch.randn(B, Skv, Hkv, D, generator=g, dtype=torch.float64, requires_grad=True)
    v = torch.randn(B, Skv, Hkv, DV, generator=g, dtype=torch.float64, requires_grad=True)
    do = torch.randn(B, Sq, Hq, DV, generator=g, dtype=torch.float64)
    mask = (torch.rand(1, Hq, Sq, Skv, generator=g, dtype=torch.float64) * 0.6).tril()
    G = Hq // Hkv

    def forward(detach_r):
        kk = k.repeat_interleave(G, dim=2)
        s = torch.einsum("bshd,bthd->bhst", q, kk) * mask
        r = s.abs().sum(-1, keepdim=True).clamp(min=1.0)
        assert (r == 1.0).any() and (r > 1.0).any()
        p = s / (r.detach() if detach_r else r)
        return torch.einsum("bhst,bthd->bshd", p, v.repeat_interleave(G, dim=2))
    out = forward(True)
    ref_out, _ = R.retention_attention(q.detach(), k.detach(), v.detach(), mask, compute_dtype=torch.float64)
    assert torch.allclose(out, ref_out, atol=1e-12)
    gq, gk, gv = torch.autograd.grad(out, (q, k, v), do)
    dq, dk, dv = R.retention_attention_grads(q.detach(), k.detach(), v.detach(), mask, do,
                                             compute_dtype=torch.float64)
    for a, b in ((dq, gq), (dk, gk), (dv, gv)):
        assert torch.allclose(a, b, atol=1e-12, rtol=1e-10)
    fq, _, _ = torch.autograd.grad(forward(False), (q, k, v), do)
    assert not torch.allclose(fq, gq, atol=1e-6)
