"""GPU parity of the backward of softmax attention: dq, dk, dv from libae_hip.so (through
AttentionEngine and torch.autograd) against the CPU oracle's closed-form gradients on the same seeded
inputs.  The oracle consumes the fp16/bf16-rounded inputs and computes in fp32; a gradient element may
differ by 2e-2 + 1% of the largest magnitude of that gradient (the kernels round p and ds to the input
type before the second products and the results to the input type)."""
import math

import pytest
import torch

import attn_cases as C
from attn_engine import AttentionEngine
from core import CustomIO, meta_tensor
from oracle import attention_ref as R
from oracle import masks as M

pytestmark = pytest.mark.gpu


class OnlineSoftmaxTwoScales(C.OnlineSoftmax):
    """The online softmax of attn_script/mha.py with its reference point and its row sum exported as TWO final row
    scales (instead of their combination lse), and the recompute / backward rules written against both, in the
    protocol of the reference (attn_engine/attn_engine.py:75-93; every final row scale is handed to forward() and
    backward(), core/lower/lower.py:413-453).  The lowering cannot take it for the softmax it has a fixed backward
    for, so both rules are traced; the function it computes is still softmax attention."""

    def __init__(self):
        super().__init__()
        from core import SymbolScalar, Var
        self.final_rowscales = {"m": SymbolScalar("m", Var("0.0")), "r": SymbolScalar("r", Var("0.0"))}

    @staticmethod
    def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
        return o / online_rowscales["r"], {"m": online_rowscales["m"], "r": online_rowscales["r"]}

    @staticmethod
    def forward(scores, final_rowscales, b, h, q_idx, kv_idx):
        return (scores - final_rowscales["m"]).exp() / final_rowscales["r"]

    @staticmethod
    def backward(dp, scores, final_rowscales, doosum_rowscales, b, h, q_idx, kv_idx):
        return scores * (dp - doosum_rowscales)


def _engine(B, H, Hkv, S, D, DV, dtype, mask_mod, scale):
    meta = (meta_tensor(B, H, S, D, dtype=dtype), meta_tensor(B, Hkv, S, D, dtype=dtype),
            meta_tensor(B, Hkv, S, DV, dtype=dtype))
    return AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(scale), mask_mod=mask_mod,
                           online_func=C.OnlineSoftmax())


def _check(got, ref, what, case):
    tol = 2e-2 + 1e-2 * ref.abs().max().item()
    err = (got.float().cpu() - ref).abs().max().item()
    assert math.isfinite(err) and err <= tol, (what, case, err, tol)


def _run(B, H, Hkv, Sq, Skv, D, DV, dtype, mask_mod, causal, seed=3):
    scale = 1 / math.sqrt(D)
    q, k, v = C.make_inputs(B, Sq, Skv, H, Hkv, D, DV, dtype, seed=seed)
    g = torch.Generator().manual_seed(seed + 100)
    do = torch.randn(B, Sq, H, DV, generator=g).to(dtype)
    mod = _engine(B, H, Hkv, Sq, D, DV, dtype, mask_mod, scale)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = mod(qd, kd, vd)
    out.backward(do.cuda())
    dense = None
    if mask_mod is not None and not causal:
        dense = torch.from_numpy(M.dense_mask_grid(mask_mod, B, H, Sq, Skv))
    ref_out, _ = R.softmax_attention(q, k, v, scale=scale, causal=causal, mask=dense)
    assert (out.detach().float().cpu() - ref_out).abs().max().item() <= 2e-2
    dq, dk, dv = R.softmax_attention_grads(q, k, v, do, scale=scale, causal=causal, mask=dense)
    case = (B, H, Hkv, Sq, Skv, D, DV, dtype, causal)
    _check(qd.grad, dq, "dq", case)
    _check(kd.grad, dk, "dk", case)
    _check(vd.grad, dv, "dv", case)
    assert qd.grad.dtype == dtype and kd.grad.shape == k.shape and vd.grad.shape == v.shape


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,H,Hkv,S,D,dtype", [
    (1, 2, 2, 256, 128, torch.float16),
    (2, 4, 4, 512, 64, torch.float16),
    (1, 2, 2, 384, 128, torch.bfloat16),
    (1, 4, 2, 320, 128, torch.float16),      # grouped heads: dk, dv sum over the group
    (1, 2, 1, 200, 64, torch.bfloat16),      # ragged: S not a multiple of any tile
    (1, 1, 1, 77, 128, torch.float16),
])
def test_softmax_backward(cuda_device, B, H, Hkv, S, D, dtype, causal):
    print(f"case bwd B{B} H{H} Hkv{Hkv} S{S} D{D} {dtype} causal={causal}", flush=True)
    _run(B, H, Hkv, S, S, D, D, dtype, C.causal_mask if causal else None, causal)


def test_softmax_backward_headline_shape(cuda_device):
    """The shape bench.py times the backward on (B2 H32 S4096 D128 fp16, causal): every gradient finite,
    and dq, dk, dv of two (batch, head) slices -- which depend on that slice's tensors only -- against the
    oracle's closed-form gradients."""
    B, H, S, D = 2, 32, 4096, 128
    dtype = torch.float16
    scale = 1 / math.sqrt(D)
    q, k, v = C.make_inputs(B, S, S, H, H, D, D, dtype, seed=9)
    do = torch.randn(B, S, H, D, generator=torch.Generator().manual_seed(109)).to(dtype)
    mod = _engine(B, H, H, S, D, D, dtype, C.causal_mask, scale)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    mod(qd, kd, vd).backward(do.cuda())
    for g in (qd.grad, kd.grad, vd.grad):
        assert torch.isfinite(g).all()
    for b, h in ((0, 0), (1, 31)):
        print(f"case backward at the headline shape: oracle on slice b{b} h{h}", flush=True)
        sl = (slice(b, b + 1), slice(None), slice(h, h + 1))
        dq, dk, dv = R.softmax_attention_grads(q[sl], k[sl], v[sl], do[sl], scale=scale, causal=True)
        _check(qd.grad[sl], dq, "dq", (b, h))
        _check(kd.grad[sl], dk, "dk", (b, h))
        _check(vd.grad[sl], dv, "dv", (b, h))


def test_softmax_backward_elementwise_mask_and_dv(cuda_device):
    """A mask that is not causal is applied per element (sliding window: rows see 37 keys), and the
    value head dim may differ from the key head dim."""
    print("case bwd sliding window", flush=True)
    _run(1, 2, 2, 300, 300, 128, 128, torch.float16, C.make_sliding_window_mask(37), False)
    print("case bwd D128 DV64", flush=True)
    _run(1, 2, 1, 256, 256, 128, 64, torch.float16, C.causal_mask, True)
    print("case bwd D64 DV128", flush=True)
    _run(2, 2, 2, 130, 130, 64, 128, torch.bfloat16, None, False)


def test_softmax_backward_skips_masked_tiles(cuda_device):
    """Masks that are not causal come with two tile-class tables (one per launch): tiles without a
    visible element are skipped, partly visible ones test mask_mod per element.  A narrow sliding window
    over a long sequence (most tiles skipped), a mask that depends on the head (one table per head), a
    shifted causal mask with grouped heads."""
    for name, mask_mod, H, Hkv, S in (("window", C.make_sliding_window_mask(100), 2, 2, 700),
                                      ("head", C.head_dependent_mask, 4, 4, 520),
                                      ("shifted", C.causal_shifted_mask, 4, 2, 333)):
        print(f"case bwd tile classes {name}", flush=True)
        _run(1, H, Hkv, S, S, 128, 128, torch.float16, mask_mod, False, seed=11)
        eng = _engine(1, H, Hkv, S, 128, 128, torch.float16, mask_mod, 1 / math.sqrt(128))
        assert eng._op._plan(1, H, S, S, None).mode == 2


def test_backward_tile_classes_of_a_long_sequence(cuda_device):
    """More than 64 streamed items per workgroup (68 q tiles of 64 rows for each of the two q heads of a kv
    head): the kernels read the tile classes 64 items at a time, so this crosses from one set to the next."""
    print("case bwd tile classes, 136 items per kv tile", flush=True)
    _run(1, 2, 1, 4352, 4352, 64, 64, torch.bfloat16, C.make_sliding_window_mask(300), False, seed=13)


def test_backward_odd_shapes_against_oracle(cuda_device):
    """Seeded sweep: ragged sequence lengths (also Sq != Skv without a mask), grouped heads, both head
    dims for keys and values, both dtypes, no mask / causal / sliding window / head-dependent masks."""
    import random
    rng = random.Random(2024)
    masks = [(None, False), (C.causal_mask, True), (C.make_sliding_window_mask(53), False),
             (C.head_dependent_mask, False)]
    for n in range(14):
        hkv = rng.choice([1, 2, 3])
        B, H = rng.choice([1, 2]), hkv * rng.choice([1, 2, 4])
        D, DV = rng.choice([64, 128]), rng.choice([64, 128])
        dtype = torch.float16 if n % 2 == 0 else torch.bfloat16
        mask_mod, causal = masks[n % len(masks)]
        Sq = rng.randint(1, 450)
        Skv = Sq if mask_mod is not None else rng.randint(1, 450)
        print(f"case bwd odd B{B} H{H} Hkv{hkv} Sq{Sq} Skv{Skv} D{D} DV{DV} {dtype} mask {n % len(masks)}", flush=True)
        _run(B, H, hkv, Sq, Skv, D, DV, dtype, mask_mod, causal, seed=300 + n)


def test_sigmoid_and_relu_backward(cuda_device):
    """Graphs whose online function does nothing (attn_script/sigmoidattn.py, reluattn.py): p = f(s),
    ds = dp f'(s) with f' from the symbolic derivative of the traced score_mod; the sigmoid's bias is a
    scalar CustomIO tensor.  Against the oracle's closed-form gradients."""
    g = torch.Generator().manual_seed(9)
    for kind, causal, B, H, Hkv, S, D, dtype in (("sigmoid", True, 1, 2, 2, 300, 128, torch.float16),
                                                 ("sigmoid", False, 2, 4, 2, 256, 64, torch.bfloat16),
                                                 ("relu", False, 1, 3, 3, 200, 64, torch.float16)):
        print(f"case bwd {kind} causal={causal} B{B} H{H} Hkv{Hkv} S{S} D{D} {dtype}", flush=True)
        scale = 1 / math.sqrt(D)
        q, k, v = C.make_inputs(B, S, S, H, Hkv, D, D, dtype, seed=21)
        do = torch.randn(B, S, H, D, generator=g).to(dtype)
        meta = (meta_tensor(B, H, S, D, dtype=dtype), meta_tensor(B, Hkv, S, D, dtype=dtype),
                meta_tensor(B, Hkv, S, D, dtype=dtype))
        if kind == "sigmoid":
            bias = torch.tensor([-math.log(S)], dtype=torch.float32)
            mod = AttentionEngine(meta, CustomIO({"softmax_bias": (1,)}), score_mod=C.make_sigmoid_score_mod(scale),
                                  mask_mod=C.causal_mask if causal else None, online_func=C.OnlineIdentity())
            extra, kw = (bias.cuda(),), dict(bias=bias.item(), causal=causal)
        else:
            mod = AttentionEngine(meta, CustomIO({}), score_mod=C.make_relu_score_mod(scale), mask_mod=None,
                                  online_func=C.OnlineIdentity())
            extra, kw = (), dict()
        qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
        out = mod(qd, kd, vd, *extra)
        out.backward(do.cuda())
        dq, dk, dv = R.elementwise_attention_grads(q, k, v, do, kind, scale=scale, **kw)
        case = (kind, causal, B, H, Hkv, S, D, dtype)
        _check(qd.grad, dq, "dq", case)
        _check(kd.grad, dk, "dk", case)
        _check(vd.grad, dv, "dv", case)


@pytest.mark.parametrize("B,H,Hkv,S,D,DV,dtype", [
    (1, 2, 2, 256, 64, 128, torch.float16),       # value head dim twice the key head dim, as in the script
    (2, 4, 2, 200, 128, 128, torch.bfloat16),     # ragged tiles, grouped heads, batch > 1 against a [1,H,S,S] mask
    (1, 3, 3, 448, 128, 64, torch.float16),
])
def test_retention_backward(cuda_device, B, H, Hkv, S, D, DV, dtype):
    """attn_script/retention.py with its forward() / backward() rules: the traced backward (the saved row
    scale r as a constant, the decay mask read per score and as the derivative of score_mod) against the
    oracle's closed form."""
    print(f"case retention backward B{B} H{H} Hkv{Hkv} S{S} D{D} DV{DV} {dtype}", flush=True)
    q, k, v = C.make_inputs(B, S, S, H, Hkv, D, DV, dtype, seed=21)
    q = (q.float() * (1 / D) ** 0.5).to(dtype)                       # bench_utils.py:1034-1036 of the reference
    g = torch.Generator().manual_seed(22)
    mask = (torch.rand(1, H, S, S, generator=g) * 1.5).tril().to(dtype).contiguous()
    do = torch.randn(B, S, H, DV, generator=g).to(dtype)
    meta = (meta_tensor(B, H, S, D, dtype=dtype), meta_tensor(B, Hkv, S, D, dtype=dtype),
            meta_tensor(B, Hkv, S, DV, dtype=dtype))
    mod = AttentionEngine(meta, C.retention_custom_inputs(), score_mod=C.retention_score_mod,
                          mask_mod=C.causal_mask, online_func=C.OnlineRetention(), mask_value="0")
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = mod(qd, kd, vd, mask.cuda())
    ref, r = R.retention_attention(q, k, v, mask)
    assert (r > 1.0).any() and (r == 1.0).any()
    assert (out.detach().float().cpu() - ref).abs().max().item() <= 2e-2
    out.backward(do.cuda())
    dq, dk, dv = R.retention_attention_grads(q, k, v, mask, do)
    case = (B, H, Hkv, S, D, DV, dtype)
    _check(qd.grad, dq, "dq", case)
    _check(kd.grad, dk, "dk", case)
    _check(vd.grad, dv, "dv", case)


@pytest.mark.parametrize("bm,bn,S,Hkv,dtype", [
    (128, 128, 1024, 3, torch.float16),    # attn_script/blocksparseattn.py's granularity: every backward tile lies in ONE block
    (128, 64, 512, 3, torch.float16),      # the geometry of the reference's tests/test_blockmask.py
    (32, 64, 640, 1, torch.bfloat16),      # finer than the backward's 64- and 128-row tiles: tiles straddle blocks of both
                                           # kinds and test every element against the mask; grouped heads
    (64, 128, 448, 3, torch.float16),      # ragged last tiles of both launches (448 = 3.5 x 128)
])
def test_backward_with_an_external_block_mask(cuda_device, bm, bn, S, Hkv, dtype):
    """attn_script/blocksparseattn.py with gradients (the reference's block-sparse backward,
    blockattn_tl.py:195-470): the user's int8 block mask [B,H,S/bm,S/bn] reaches the two backward launches as
    tile-class tables made from it on the GPU, and tiles that straddle visible and invisible blocks look every
    element up in the mask itself.  Against the oracle's gradients under the expanded dense mask; one q block
    row sees nothing at all (out 0, gradients 0)."""
    print(f"case bwd extern block mask {bm}x{bn} S{S} Hkv{Hkv} {dtype}", flush=True)
    B, H, D = 2, 3, 64
    scale = 1 / math.sqrt(D)
    g = torch.Generator().manual_seed(11)
    nq, nk = -(-S // bm), -(-S // bn)
    blocks = torch.rand(B, H, nq, nk, generator=g) < 0.45
    blocks[..., 0] = True                         # every row sees something ...
    blocks[0, 1, nq - 1] = False                  # ... except one block row of one head
    q, k, v = C.make_inputs(B, S, S, H, Hkv, D, D, dtype, seed=5)
    do = torch.randn(B, S, H, D, generator=g).to(dtype)
    meta = (meta_tensor(B, H, S, D, dtype=dtype), meta_tensor(B, Hkv, S, D, dtype=dtype),
            meta_tensor(B, Hkv, S, D, dtype=dtype))
    mod = AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(scale), mask_mod=None,
                          online_func=C.OnlineSoftmax(), infer_mask=True, extern_block_mask=True,
                          infer_mask_block_M=bm, infer_mask_block_N=bn)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = mod(qd, kd, vd, block_mask=blocks.to(torch.int8).cuda())
    out.backward(do.cuda())
    dense = blocks.repeat_interleave(bm, 2).repeat_interleave(bn, 3)[:, :, :S, :S]
    ref_out, _ = R.softmax_attention(q, k, v, scale=scale, mask=dense)
    assert (out.detach().float().cpu() - ref_out).abs().max().item() <= 2e-2
    dq, dk, dv = R.softmax_attention_grads(q, k, v, do, scale=scale, mask=dense)
    case = (bm, bn, S, Hkv, dtype)
    _check(qd.grad, dq, "dq", case)
    _check(kd.grad, dk, "dk", case)
    _check(vd.grad, dv, "dv", case)
    r0 = (nq - 1) * bm
    assert qd.grad[0, r0:, 1].abs().max().item() == 0.0          # the rows that see nothing
    # a second call with another mask: the tables follow the mask of the call
    blocks2 = torch.ones_like(blocks)
    qd.grad = kd.grad = vd.grad = None
    mod(qd, kd, vd, block_mask=blocks2.to(torch.int8).cuda()).backward(do.cuda())
    dq, dk, dv = R.softmax_attention_grads(q, k, v, do, scale=scale)
    _check(qd.grad, dq, "dq", case + ("all",))
    _check(kd.grad, dk, "dk", case + ("all",))


@pytest.mark.parametrize("mask_name", ["causal", "window", "plus_one", "head_dependent"])
def test_backward_masks_are_bit_exact(cuda_device, mask_name):
    """One-hot probes of the masks the two backward launches apply (tiles skipped by index or by their tile-class
    tables, elements tested where a tile is partly visible), at 4300 positions -- more than 64 streamed items per
    resident tile, so the tables are read in several chunks of ballots, ragged last tiles in both launches -- and
    two q heads per kv head.  Integers, compared exactly:
      * dk / dv launch: the graph out = sum_kv f(s) v with f = 1 on every finite score and 0 on a masked one;
        dO holds one-hot rows (q -> column q mod DV), so dv[kv, j] = dO^T p counts the queries of residue class j
        that see key kv (summed over the group's q heads);
      * dq launch: f(s) = s, so ds = dp on visible scores and 0 on masked ones; with v and dO all equal to the
        first unit vector dp = 1, and K one-hot rows make dq[q, j] = ds K count the visible keys of class j."""
    mask_mod = {"causal": C.causal_mask, "window": C.make_sliding_window_mask(100),
                "plus_one": C.causal_plus_one_mask, "head_dependent": C.head_dependent_mask}[mask_name]
    B, H, Hkv, S, D = 1, 2, 1, 4300, 64
    dtype = torch.float16
    print(f"case bwd mask probe {mask_name}", flush=True)
    dense = torch.from_numpy(M.dense_mask_grid(mask_mod, B, H, S, S)).float()        # [B,H,S,S]
    onehot = torch.zeros(S, D)
    onehot[torch.arange(S), torch.arange(S) % D] = 1.0
    meta = (meta_tensor(B, H, S, D, dtype=dtype), meta_tensor(B, Hkv, S, D, dtype=dtype),
            meta_tensor(B, Hkv, S, D, dtype=dtype))

    def ones_score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        return ((score * 0.001 + 50.0).tanh() + 1.0) * 0.5

    def plain_score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        return score * 1.0

    q, k, v = C.make_inputs(B, S, S, H, Hkv, D, D, dtype)
    # dk / dv launch
    mod = AttentionEngine(meta, CustomIO({}), score_mod=ones_score_mod, mask_mod=mask_mod, online_func=C.OnlineIdentity())
    bwd = mod._op.backward_op()
    assert bwd.kind == 1
    do = onehot.to(dtype).view(1, S, 1, D).expand(B, S, H, D).contiguous()
    out = torch.zeros(B, S, H, D, dtype=dtype)
    _, _, dv = bwd(q.cuda(), k.cuda(), v.cuda(), out.cuda(), None, do.cuda())
    expect = torch.einsum("bhqk,qd->bkd", dense, onehot).view(B, S, Hkv, D)
    assert expect.max().item() >= {"causal": 100, "plus_one": 100, "window": 4, "head_dependent": 5}[mask_name]
    assert torch.equal(dv.float().cpu(), expect), mask_name
    # dq launch
    mod = AttentionEngine(meta, CustomIO({}), score_mod=plain_score_mod, mask_mod=mask_mod, online_func=C.OnlineIdentity())
    bwd = mod._op.backward_op()
    e0 = torch.zeros(D, dtype=dtype)
    e0[0] = 1.0
    kk = onehot.to(dtype).view(1, S, 1, D).expand(B, S, Hkv, D).contiguous()
    vv = e0.view(1, 1, 1, D).expand(B, S, Hkv, D).contiguous()
    do = e0.view(1, 1, 1, D).expand(B, S, H, D).contiguous()
    dq, _, _ = bwd(q.cuda(), kk.cuda(), vv.cuda(), out.cuda(), None, do.cuda())
    expect = torch.einsum("bhqk,kd->bqhd", dense, onehot)
    assert torch.equal(dq.float().cpu(), expect), mask_name


@pytest.mark.parametrize("B,H,Hkv,S,D,dtype,causal", [
    (1, 2, 2, 256, 64, torch.float16, False),
    (2, 4, 2, 333, 128, torch.bfloat16, True),      # grouped heads, ragged tiles, causal
    (1, 3, 1, 200, 64, torch.float16, True),
])
def test_traced_backward_with_two_final_row_scales(cuda_device, B, H, Hkv, S, D, dtype, causal):
    """An online function with TWO final row scales whose forward() / backward() rules read both: the rules are
    traced (no fixed gradient applies), the backward launches carry both row scales per q row, and since the
    function is softmax attention written differently its gradients must be those of the oracle
    (softmax_attention_grads, pinned by float64 autograd).  The exported scales themselves: m + log r = lse."""
    print(f"case two row scales B{B} H{H} Hkv{Hkv} S{S} D{D} {dtype} causal={causal}", flush=True)
    scale = 1 / math.sqrt(D)
    q, k, v = C.make_inputs(B, S, S, H, Hkv, D, D, dtype, seed=13)
    do = torch.randn(B, S, H, D, generator=torch.Generator().manual_seed(113)).to(dtype)
    meta = (meta_tensor(B, H, S, D, dtype=dtype), meta_tensor(B, Hkv, S, D, dtype=dtype),
            meta_tensor(B, Hkv, S, D, dtype=dtype))
    mod = AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(scale),
                          mask_mod=C.causal_mask if causal else None, online_func=OnlineSoftmaxTwoScales())
    bwd = mod._op.backward_op()
    assert bwd.kind == 2 and bwd.rowscale_names == ["m", "r"] and bwd.n_rs == 2
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = mod(qd, kd, vd)
    out.backward(do.cuda())
    ref_out, lse = R.softmax_attention(q, k, v, scale=scale, causal=causal)
    assert (out.detach().float().cpu() - ref_out).abs().max().item() <= 2e-2
    m, r = mod.final_rowscales["m"].cpu(), mod.final_rowscales["r"].cpu()
    assert (m + r.log() - lse).abs().max().item() <= 1e-3
    dq, dk, dv = R.softmax_attention_grads(q, k, v, do, scale=scale, causal=causal)
    case = (B, H, Hkv, S, D, dtype, causal)
    _check(qd.grad, dq, "dq", case)
    _check(kd.grad, dk, "dk", case)
    _check(vd.grad, dv, "dv", case)


def test_backward_of_other_graphs_is_refused(cuda_device):
    """An online function that keeps row scales of its own but defines no forward() / backward() rules
    (here: the running sum of |s| without them) has no backward.  Its forward still runs on tensors that
    require gradients, with the result of the plain call; the missing rule is reported by .backward(), where the
    reference reports it."""
    B, H, S, D = 1, 2, 128, 64
    meta = (meta_tensor(B, H, S, D, dtype=torch.float16),) * 3
    mod = AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(0.125), mask_mod=None,
                          online_func=C.OnlineAbsNorm())
    q, k, v = (t.cuda() for t in C.make_inputs(B, S, S, H, H, D, D, torch.float16))
    plain = mod(q, k, v)
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = mod(qg, kg, vg)
    assert out.requires_grad and torch.equal(out.detach(), plain)
    with pytest.raises(NotImplementedError, match="no backward for this engine"):
        out.sum().backward()
    assert qg.grad is None
