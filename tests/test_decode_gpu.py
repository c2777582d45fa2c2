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


@pytest.mark.parametrize("B,Hq,Hkv,Skv,D,dtype", [
    (64, 16, 4, 500, 64, torch.float16),       # ragged kv, fewer keys in the last waves' tiles
    (64, 40, 2, 160, 128, torch.bfloat16),     # 20 heads per group: a full and a partly filled head tile
    (256, 8, 1, 40, 128, torch.float16),       # two tiles for four waves: two partial results are empty
])
def test_gqa_decode_merged_in_the_workgroup(cuda_device, monkeypatch, B, Hq, Hkv, Skv, D, dtype):
    """Launches with one workgroup per (batch, kv head, head tile) merge their waves' partial results in LDS and
    write out themselves (one launch, no work buffers): against the oracle, and bit for bit against the same
    launch followed by the merge kernel (attn_gqa_decode_tl.py:224-266)."""
    print(f"case merged gqa decode B{B} Hq{Hq} Hkv{Hkv} Skv{Skv} D{D} {dtype}", flush=True)
    q, k, v = C.make_inputs(B, 1, Skv, Hq, Hkv, D, D, dtype)
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    res = {}
    for merge in ("1", "0"):
        monkeypatch.setenv("AE_DECODE_MERGE_IN_WG", merge)
        mod = _decode_engine(B, Hq, Hkv, Skv, D, D, dtype, C.make_scale_score_mod(1 / math.sqrt(D)), C.OnlineSoftmax())
        op = mod.attention
        n_split, _ = op.plan_splits(B, Hq, Hkv, Skv)
        assert n_split == op.N_WAVES and op.merges_in_workgroup(n_split) == (merge == "1")
        res[merge] = (mod(qc, kc, vc).clone(), mod.final_rowscales["lse"].clone())
    assert torch.equal(res["1"][0], res["0"][0]) and torch.equal(res["1"][1], res["0"][1])
    for b in (0, B - 1):
        ref, lse = R.softmax_attention(q[b:b + 1], k[b:b + 1], v[b:b + 1], causal=False)
        assert (res["1"][0][b:b + 1].float().cpu() - ref).abs().max().item() <= OUT_TOL
        assert (res["1"][1][b:b + 1].cpu() - lse).abs().max().item() <= LSE_TOL


@pytest.mark.parametrize("B,Hq,Hkv,Skv,D,dtype,kind", [
    (1, 32, 8, 8192, 128, torch.float16, "softmax"),     # attn_script/gqa_inference.py shape: 8 workgroups a kv head
    (2, 40, 2, 4001, 64, torch.bfloat16, "softmax"),     # two head tiles (one partly filled), ragged kv
    (1, 16, 8, 2048, 128, torch.float16, "softmax"),     # two q heads a kv head: 14 of a tile's 16 rows are padding
    (2, 8, 2, 3000, 128, torch.float16, "sigmoid"),      # no row scales: the partial results are summed
])
def test_gqa_decode_merged_by_the_last_workgroup(cuda_device, monkeypatch, B, Hq, Hkv, Skv, D, dtype, kind):
    """Small batches spread one kv axis over several workgroups; the workgroup that counts itself in last merges
    all partial results (one launch).  Bit for bit equal to the split launch followed by the merge kernel
    (attn_gqa_decode_tl.py:224-266), on 300 launches that alternate between two inputs (a merge that read another
    launch's partial results, or that ran before the last partial result was visible, would differ), and again
    as replays of a captured HIP graph with eager work between them."""
    print(f"case last-workgroup gqa decode B{B} Hq{Hq} Hkv{Hkv} Skv{Skv} D{D} {dtype} {kind}", flush=True)

    def sig(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        return (((score * (1 / math.sqrt(D)) - 6.0) * 0.5).tanh() + 1) * 0.5
    score_mod, online = ((C.make_scale_score_mod(1 / math.sqrt(D)), C.OnlineSoftmax()) if kind == "softmax"
                         else (sig, C.OnlineIdentity()))
    inputs = [tuple(t.cuda() for t in C.make_inputs(B, 1, Skv, Hq, Hkv, D, D, dtype, seed=s)) for s in (0, 1)]

    def rowscale(mod):
        return mod.final_rowscales["lse"].clone() if kind == "softmax" else torch.zeros(1)
    monkeypatch.setenv("AE_DECODE_MERGE_LAST", "0")
    two = _decode_engine(B, Hq, Hkv, Skv, D, D, dtype, score_mod, online)
    n_split, _ = two.attention.plan_splits(B, Hq, Hkv, Skv)
    assert n_split > two.attention.N_WAVES and two.attention._merge_mode(n_split) == 0
    want = []
    for q, k, v in inputs:
        want.append((two(q, k, v).clone(), rowscale(two)))
    assert not torch.equal(want[0][0], want[1][0])
    monkeypatch.setenv("AE_DECODE_MERGE_LAST", "1")
    one = _decode_engine(B, Hq, Hkv, Skv, D, D, dtype, score_mod, online)
    assert one.attention._merge_mode(n_split) == 2
    got = []
    for it in range(300):
        q, k, v = inputs[it & 1]
        got.append((one(q, k, v), rowscale(one)))
    torch.cuda.synchronize()
    for it, (o, r) in enumerate(got):
        assert torch.equal(o, want[it & 1][0]), f"launch {it}: out differs"
        assert torch.equal(r.cpu(), want[it & 1][1].cpu()), f"launch {it}: row scale differs"
    if kind == "softmax":
        q, k, v = (t.cpu() for t in inputs[0])
        ref, lse = R.softmax_attention(q, k, v, causal=False)
        assert (want[0][0].float().cpu() - ref).abs().max().item() <= OUT_TOL
        assert (want[0][1].cpu() - lse).abs().max().item() <= LSE_TOL
    # under a HIP graph: the work buffers are the operator's (allocated by the first call on the stream, outside the
    # capture), the arrival counters are back at zero after every launch
    side = torch.cuda.Stream()
    q, k, v = (t.clone() for t in inputs[0])
    with torch.cuda.stream(side):
        one(q, k, v)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out_g = one(q, k, v)
        out_g2 = one(q, k, v)          # two launches in one graph share the buffers, one after the other
    for rep in range(6):
        for dst, src in zip((q, k, v), inputs[rep & 1]):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, want[rep & 1][0]) and torch.equal(out_g2, want[rep & 1][0]), f"replay {rep}"
        assert torch.equal(one(*inputs[1]), want[1][0])        # eager work between the replays


@pytest.mark.parametrize("B,Hq,Hkv,Skv,dtype", [
    (64, 32, 8, 777, torch.float16),       # one workgroup per (batch, kv head): merged in the workgroup
    (2, 32, 8, 4100, torch.bfloat16),      # kv axis over several workgroups: merged by the last one
])
def test_gqa_decode_head_dim_256(cuda_device, B, Hq, Hkv, Skv, dtype):
    """Head dim 256 (the kernel is built for one wave per SIMD there: at two it spills 85 registers): against the
    oracle on every batch entry."""
    D = 256
    print(f"case gqa decode D256 B{B} Hq{Hq} Hkv{Hkv} Skv{Skv} {dtype}", flush=True)
    q, k, v = C.make_inputs(B, 1, Skv, Hq, Hkv, D, D, dtype, seed=5)
    mod = _decode_engine(B, Hq, Hkv, Skv, D, D, dtype, C.make_scale_score_mod(1 / math.sqrt(D)), C.OnlineSoftmax())
    (module, _, _, src), = mod.attention._variants.values()
    assert "#define AE_WAVES_PER_EU 1" in src
    assert module.kernel_info()["ae_decode_split_kernel"].get(".vgpr_spill_count", 0) == 0
    out = mod(q.cuda(), k.cuda(), v.cuda())
    ref, lse = R.softmax_attention(q, k, v, causal=False)
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


def _mla_inputs(B, H, G, S, DV, DPE, dtype, seed=0):
    """q, q_pe, kv, k_pe generated on the CPU in that order."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, 1, H, DV, generator=g).to(dtype)
    q_pe = torch.randn(B, 1, H, DPE, generator=g).to(dtype)
    kv = torch.randn(B, S, G, DV, generator=g).to(dtype)
    k_pe = torch.randn(B, S, G, DPE, generator=g).to(dtype)
    return q, q_pe, kv, k_pe


def _mla_engine(B, H, G, S, D, DV, dtype, scale, **kw):
    meta = (meta_tensor(B, H, 1, D, dtype=dtype), meta_tensor(B, G, S, D, dtype=dtype),
            meta_tensor(B, G, S, DV, dtype=dtype))
    return AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(scale), mask_mod=None,
                           online_func=C.OnlineSoftmax(), kv_shared=True, **kw)


@pytest.mark.parametrize("B,S", [(2, 4096), (40, 600)])      # several splits with the merge kernel / one split
def test_mla_decode_as_nodes_of_a_hip_graph(cuda_device, B, S):
    """MLA decode captured into a HIP graph and replayed on changing inputs: every replay equals the eager call, bit
    for bit, with eager work between the replays."""
    H, D, DV, dtype = 128, 576, 512, torch.bfloat16
    print(f"case mla decode in a graph B{B} S{S}", flush=True)
    mod = _mla_engine(B, H, 1, S, D, DV, dtype, 1 / math.sqrt(192))
    inputs = [tuple(t.cuda() for t in _mla_inputs(B, H, 1, S, DV, D - DV, dtype, seed=s)) for s in (11, 12)]
    want = [(mod(*a).clone(), mod.final_rowscales["lse"].clone()) for a in inputs]
    assert not torch.equal(want[0][0], want[1][0])
    side = torch.cuda.Stream()
    args = [t.clone() for t in inputs[0]]
    with torch.cuda.stream(side):
        mod(*args)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out_g = mod(*args)
        lse_g = mod.final_rowscales["lse"]
    for rep in range(5):
        for dst, src in zip(args, inputs[rep & 1]):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, want[rep & 1][0]) and torch.equal(lse_g, want[rep & 1][1]), f"replay {rep}"
        assert torch.equal(mod(*inputs[1]), want[1][0])


@pytest.mark.parametrize("B,H,G,S,dtype", [
    (2, 128, 1, 512, torch.bfloat16),     # DeepSeek-V3 head layout (BASELINE config 5, short KV)
    (1, 128, 1, 4096, torch.bfloat16),    # attn_script/mla_decode.py shape, one batch entry -> many splits
    (3, 16, 1, 200, torch.float16),       # fewer heads than a workgroup covers, ragged KV
    (2, 64, 2, 96, torch.bfloat16),       # two latent heads
])
@pytest.mark.parametrize("kernel,template", [("", "ae_mla_decode_ws.hip"), ("generic", "ae_mla_decode.hip")])
def test_mla_decode_tl_convention(cuda_device, monkeypatch, B, H, G, S, dtype, kernel, template):
    """Both kernel templates: the wave-specialised one chosen for scaled softmax and the generic one
    (any functor graph), forced through AE_MLA_KERNEL."""
    D, DV = 576, 512
    scale = 1 / math.sqrt(192)            # BASELINE config 5 scale
    print(f"case mla B{B} H{H} G{G} S{S} {dtype} kernel={kernel or 'default'}", flush=True)
    monkeypatch.setenv("AE_MLA_KERNEL", kernel)
    q, q_pe, kv, k_pe = _mla_inputs(B, H, G, S, DV, D - DV, dtype)
    mod = _mla_engine(B, H, G, S, D, DV, dtype, scale)
    out = mod(q.cuda(), q_pe.cuda(), kv.cuda(), k_pe.cuda())
    assert mod.attention.template == template
    ref, lse = R.mla_decode(q[:, 0], q_pe[:, 0], kv, k_pe, scale=scale)
    assert out.shape == (B, 1, H, DV) and out.dtype == dtype
    assert (out[:, 0].float().cpu() - ref).abs().max().item() <= OUT_TOL
    assert (mod.final_rowscales["lse"][:, :, 0].cpu() - lse).abs().max().item() <= LSE_TOL


@pytest.mark.parametrize("kernel,template", [("", "ae_mla_decode_ws.hip"), ("generic", "ae_mla_decode.hip")])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("S,late_keys", [(1024, False), (1000, False), (1531, True)])
def test_mla_decode_long_single_split_loop(cuda_device, monkeypatch, kernel, template, dtype, S, late_keys):
    """The plan the benchmark runs at B128 H128 S4096 is ONE split per workgroup and a loop over many kv
    tiles that writes out / lse directly, without the merge pass.  Forced here on a small shape
    (target_workgroups = 1): 32 to 48 tiles per workgroup with a ragged last tile, so the LDS stage ring
    wraps many times, the hand-off between score and value waves runs a long loop, and -- with keys that
    score far above everything before them late in the sequence -- the lazy reference moves and O is
    rescaled in the middle of it."""
    D, DV, B, H, G = 576, 512, 2, 128, 1
    scale = 1 / math.sqrt(192)
    print(f"case mla long loop S{S} {dtype} kernel={kernel or 'default'} late_keys={late_keys}", flush=True)
    monkeypatch.setenv("AE_MLA_KERNEL", kernel)
    q, q_pe, kv, k_pe = _mla_inputs(B, H, G, S, DV, D - DV, dtype, seed=17)
    if late_keys:
        # (only the rope part of the keys is scaled: the latent part is also V, and outputs beyond ~4 do
        # not fit bf16's 8 bits inside the 2e-2 bar)
        k_pe = k_pe.float()
        k_pe[:, 700:703] *= 12.0          # a jump for every head ...
        k_pe[:, 1200:] *= 4.0             # ... and a second level that stays
        k_pe = k_pe.to(dtype)
    mod = _mla_engine(B, H, G, S, D, DV, dtype, scale)
    mod.attention.target_workgroups = 1       # read by plan_splits at call time
    n_split, per = mod.attention.plan_splits(B, H, G, S)
    assert n_split == 1 and per >= S and per // mod.attention.BLOCK_N >= 2 * mod.attention.WS_STAGES
    out = mod(q.cuda(), q_pe.cuda(), kv.cuda(), k_pe.cuda())
    assert mod.attention.template == template
    ref, lse = R.mla_decode(q[:, 0], q_pe[:, 0], kv, k_pe, scale=scale)
    assert torch.isfinite(out).all()
    assert (out[:, 0].float().cpu() - ref).abs().max().item() <= OUT_TOL
    got = mod.final_rowscales["lse"][:, :, 0].cpu()
    assert ((got - lse).abs() <= LSE_TOL + 2e-6 * lse.abs()).all()


def test_mla_decode_full_size(cuda_device):
    """BASELINE config 5 at full size (B128 H128 one latent head, D576 DV512, Skv4096, bf16, scale
    1/sqrt(192)) with the plan the benchmark times: one split, 128 tiles per workgroup.  Oracle on batch
    entries 0, 127 and two seeded others; everything finite; lse independent of which batch slot a
    sequence sits in (entry 5 is a copy of entry 77)."""
    D, DV, B, H, G, S = 576, 512, 128, 128, 1, 4096
    dtype = torch.bfloat16
    scale = 1 / math.sqrt(192)
    q, q_pe, kv, k_pe = _mla_inputs(B, H, G, S, DV, D - DV, dtype, seed=5)
    for t in (q, q_pe, kv, k_pe):
        t[5] = t[77]
    mod = _mla_engine(B, H, G, S, D, DV, dtype, scale)
    n_split, per = mod.attention.plan_splits(B, H, G, S)
    assert (n_split, per) == (1, S)                 # what bench.py's c5_mla_decode launches
    out = mod(q.cuda(), q_pe.cuda(), kv.cuda(), k_pe.cuda())
    lse = mod.final_rowscales["lse"][:, :, 0]
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    assert torch.equal(out[5], out[77]) and torch.equal(lse[5], lse[77])
    import random
    picks = [0, 127] + random.Random(8).sample(range(1, 127), 2)
    for b in picks:
        print(f"case mla full size: oracle on batch entry {b}", flush=True)
        ref, lref = R.mla_decode(q[b:b + 1, 0], q_pe[b:b + 1, 0], kv[b:b + 1], k_pe[b:b + 1], scale=scale)
        assert (out[b:b + 1, 0].float().cpu() - ref).abs().max().item() <= OUT_TOL, b
        assert (lse[b:b + 1].cpu() - lref).abs().max().item() <= LSE_TOL, b


def test_mla_decode_cute_convention(cuda_device):
    """mod(q [B,1,H,576], paged kv cache [B*S/64, 64, 1, 576]) -> (out, lse), as in
    attn_script/mla_decode_cute.py:286-303; lse checked with the script's cos-diff bound (107-113)."""
    B, H, G, S, D, DV = 2, 128, 1, 1024, 576, 512
    dtype = torch.bfloat16
    scale = 1 / math.sqrt(D)
    q, q_pe, kv, k_pe = _mla_inputs(B, H, G, S, DV, D - DV, dtype, seed=3)
    mod = _mla_engine(B, H, G, S, D, DV, dtype, scale, backend="cute")
    q_full = torch.cat([q, q_pe], -1)
    cache = torch.cat([kv, k_pe], -1).reshape(B * S // 64, 64, G, D).contiguous()
    out, lse = mod(q_full.cuda(), cache.cuda())
    ref, lref = R.mla_decode(q[:, 0], q_pe[:, 0], kv, k_pe, scale=scale)
    assert (out[:, 0].float().cpu() - ref).abs().max().item() <= OUT_TOL
    x, y = lse[:, :, 0].double().cpu(), lref.double()
    cos_diff = 1 - 2 * (x * y).sum().item() / max((x * x + y * y).sum().item(), 1e-12)
    assert cos_diff < 1e-5
    assert (x - y).abs().max().item() <= LSE_TOL


@pytest.mark.parametrize("kernel", ["ws", "generic"])
@pytest.mark.parametrize("dtype,B,H,page,lens,target", [
    (torch.bfloat16, 3, 128, 64, [1000, 37, 640], 256),    # split launch; entry 1 leaves most splits without a key
    (torch.float16, 2, 16, 32, [513, 2048], 1),            # one split, long loop, ragged tails, 16 of 64 head rows
    (torch.bfloat16, 2, 64, 128, [128, 1], 8),             # pages larger than a tile, a one-token entry
    (torch.float16, 4, 64, 64, [700, 0, 64, 257], 64),     # split launch with an empty entry, entries of one split
                                                           # (they write `out` themselves) and merged ones
])
def test_mla_decode_paged_cache(cuda_device, monkeypatch, kernel, dtype, B, H, page, lens, target):
    """mod(q, kv_cache, block_table=..., cache_seqlens=...): pages in a shuffled order, every batch entry
    with its own length (cute_template_kvshared/flash_api.cpp:61-72, kernels/params.h:33-36).  Unused
    table entries hold an out-of-range page number and unused pages NaN, so a read beyond an entry's
    length shows."""
    print(f"case mla paged {kernel} {dtype} B{B} H{H} page{page} lens{lens} target{target}", flush=True)
    if kernel == "generic":
        monkeypatch.setenv("AE_MLA_KERNEL", "generic")
    G, D, DV = 1, 576, 512
    scale = 1 / math.sqrt(D)
    max_pages = -(-max(lens) // page) + 1
    n_pages = B * max_pages + 3
    g = torch.Generator().manual_seed(11)
    perm = torch.randperm(n_pages, generator=g)
    table = torch.full((B, max_pages), n_pages + 7, dtype=torch.int32)
    cache = torch.full((n_pages, page, G, D), float("nan"), dtype=dtype)
    q, q_pe, kv, k_pe = _mla_inputs(B, H, G, max_pages * page, DV, D - DV, dtype, seed=5)
    dense = torch.cat([kv, k_pe], -1)
    used = 0
    for b in range(B):
        for j in range(-(-lens[b] // page)):
            pg = int(perm[used]); used += 1
            table[b, j] = pg
            cache[pg] = dense[b, j * page:(j + 1) * page]
    # rows of the last used page beyond the entry's length stay finite (any value): the kernels may load
    # them, they must not let them reach the result
    mod = _mla_engine(B, H, G, max_pages * page, D, DV, dtype, scale, backend="cute")
    mod.attention.target_workgroups = target
    out, lse = mod(torch.cat([q, q_pe], -1).cuda(), cache.cuda(), block_table=table.cuda(),
                   cache_seqlens=torch.tensor(lens, dtype=torch.int32).cuda())
    assert out.shape == (B, 1, H, DV) and lse.shape == (B, H, 1)
    for b in range(B):
        n = lens[b]
        if n == 0:      # no key at all: zeros, lse -inf (cute_template/flash_fwd_kernel.h:180-183 of the reference)
            assert (out[b] == 0).all() and (lse[b] == float("-inf")).all()
            continue
        ref, lref = R.mla_decode(q[b:b + 1, 0], q_pe[b:b + 1, 0], kv[b:b + 1, :n], k_pe[b:b + 1, :n], scale=scale)
        assert (out[b:b + 1, 0].float().cpu() - ref).abs().max().item() <= OUT_TOL, b
        assert (lse[b:b + 1, :, 0].cpu() - lref).abs().max().item() <= LSE_TOL, b
    # the same engine still reads a dense cache when no table is given
    n0 = -(-max(lens) // page) * page
    out2, _ = mod(torch.cat([q, q_pe], -1).cuda(), dense[:, :n0].reshape(-1, page, G, D).contiguous().cuda())
    ref, _ = R.mla_decode(q[:, 0], q_pe[:, 0], kv[:, :n0], k_pe[:, :n0], scale=scale)
    assert (out2[:, 0].float().cpu() - ref).abs().max().item() <= OUT_TOL


def test_decode_split_counts_are_tuned_and_recorded(cuda_device, tmp_path):
    """tune=True for the decode engines (the reference tunes num_split whenever it builds the MLA decode kernel,
    mla_decode_tl.py:13-24, 308-319): the first call of a shape measures the planned split count, its half and its
    multiples on the caller's tensors, records the fastest under the problem keys and uses it from then on; every
    candidate computes the same result (checked here through the oracle on the winner and through the records)."""
    import json
    f = str(tmp_path / "splits.json")
    # MLA, paged cache with very different lengths
    B, H, G, D, DV, page, dtype = 8, 128, 1, 576, 512, 64, torch.bfloat16
    lens = [2048, 64, 300, 1, 1024, 77, 512, 1999]
    scale = 1 / math.sqrt(D)
    max_pages = -(-max(lens) // page)
    q, q_pe, kv, k_pe = _mla_inputs(B, H, G, max_pages * page, DV, D - DV, dtype, seed=9)
    cache = torch.cat([kv, k_pe], -1).reshape(B * max_pages, page, G, D).contiguous()
    table = torch.arange(B * max_pages, dtype=torch.int32).reshape(B, max_pages)
    args = (torch.cat([q, q_pe], -1).cuda(), cache.cuda())
    kw = dict(block_table=table.cuda(), cache_seqlens=torch.tensor(lens, dtype=torch.int32).cuda())
    mod = _mla_engine(B, H, G, max_pages * page, D, DV, dtype, scale, backend="cute", tune=True, tune_file=f)
    out, lse = mod(*args, **kw)
    op = mod.attention
    key = (B, H, G, max_pages * page)
    assert len(op.tune_times) >= 3 and op._tuned[key] in op.tune_times
    assert op.tune_times[op._tuned[key]] == min(op.tune_times.values())
    (rec,) = json.load(open(f))
    assert rec == {"batch": B, "heads": H, "seq_len": max_pages * page, "dim": D, "dimv": DV,
                   "tuned_config": [op._tuned[key]]}
    for b in range(B):
        n = lens[b]
        ref, lref = R.mla_decode(q[b:b + 1, 0], q_pe[b:b + 1, 0], kv[b:b + 1, :n], k_pe[b:b + 1, :n], scale=scale)
        assert (out[b:b + 1, 0].float().cpu() - ref).abs().max().item() <= OUT_TOL, b
        assert (lse[b:b + 1, :, 0].cpu() - lref).abs().max().item() <= LSE_TOL, b
    again = _mla_engine(B, H, G, max_pages * page, D, DV, dtype, scale, backend="cute", tune=True, tune_file=f)
    out2, lse2 = again(*args, **kw)
    assert again.attention.tune_times is None and again.attention._tuned[key] == op._tuned[key]
    assert torch.equal(out, out2) and torch.equal(lse, lse2)

    # GQA decode: same file, another problem
    B, Hq, Hkv, Skv, D = 4, 32, 8, 4096, 128
    qg, kg, vg = C.make_inputs(B, 1, Skv, Hq, Hkv, D, D, torch.float16)
    gqa = _decode_engine(B, Hq, Hkv, Skv, D, D, torch.float16, C.make_scale_score_mod(1 / math.sqrt(D)),
                         C.OnlineSoftmax(), tune=True, tune_file=f)
    og = gqa(qg.cuda(), kg.cuda(), vg.cuda())
    ref, lref = R.softmax_attention(qg, kg, vg, causal=False)
    assert (og.float().cpu() - ref).abs().max().item() <= OUT_TOL
    assert (gqa.final_rowscales["lse"].cpu() - lref).abs().max().item() <= LSE_TOL
    assert len(gqa.attention.tune_times) >= 2
    recs = json.load(open(f))
    assert len(recs) == 2 and recs[1]["tuned_config"] == [gqa.attention._tuned[(B, Hq, Hkv, Skv)]]


def _mha_decode_engine(B, H, Sq, Skv, D, dtype, online, mask_mod=None):
    meta = (meta_tensor(B, H, Sq, D, dtype=dtype), meta_tensor(B, H, Skv, D, dtype=dtype),
            meta_tensor(B, H, Skv, D, dtype=dtype))
    return AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(1 / math.sqrt(D)),
                           mask_mod=mask_mod, online_func=online)


@pytest.mark.parametrize("B,H,Sq,Skv,D,dtype", [
    (1, 32, 128, 8192, 128, torch.float16),   # attn_script/mha_inference.py shape
    (2, 4, 5, 1000, 128, torch.float16),      # q rows and kv length that are no multiple of any tile
    (1, 2, 64, 4096, 64, torch.bfloat16),
    (2, 3, 1, 300, 128, torch.float16),       # one query token, as many heads as kv heads
])
def test_mha_decode_split_kv(cuda_device, B, H, Sq, Skv, D, dtype):
    """A few query tokens against a long KV with as many kv heads as q heads: the kv axis is split
    over workgroups and merged with OnlineFunc.combine (attn_engine.py:273-290 and
    core/template/tl_template/attn/attn_decode_tl.py:47-205 of the reference)."""
    print(f"case mha decode B{B} H{H} Sq{Sq} Skv{Skv} D{D} {dtype}", flush=True)
    q, k, v = C.make_inputs(B, Sq, Skv, H, H, D, D, dtype)
    mod = _mha_decode_engine(B, H, Sq, Skv, D, dtype, C.OnlineSoftmax())
    n_split, per = mod.attention.plan_splits(B, H, Sq, Skv)
    assert n_split > 1 and n_split * per >= Skv and (n_split - 1) * per < Skv
    out = mod(q.cuda(), k.cuda(), v.cuda())
    ref, lse = R.softmax_attention(q, k, v, causal=False)
    assert out.shape == (B, Sq, H, D) and out.dtype == dtype
    assert (out.float().cpu() - ref).abs().max().item() <= OUT_TOL
    got = mod.final_rowscales["lse"]
    assert got.shape == (B, H, Sq)
    assert (got.cpu() - lse).abs().max().item() <= LSE_TOL


def test_mha_decode_matches_unsplit(cuda_device):
    """Merge invariant: the split-KV result equals the same engine run without splitting."""
    B, H, Sq, Skv, D, dtype = 1, 8, 32, 2048, 128, torch.float16
    q, k, v = C.make_inputs(B, Sq, Skv, H, H, D, D, dtype)
    mod = _mha_decode_engine(B, H, Sq, Skv, D, dtype, C.OnlineSoftmax())
    out = mod(q.cuda(), k.cuda(), v.cuda())
    lse = mod.final_rowscales["lse"].clone()
    mod.attention.split_kv = False
    out1 = mod(q.cuda(), k.cuda(), v.cuda())
    assert (out.float() - out1.float()).abs().max().item() <= 2e-3
    assert (lse - mod.final_rowscales["lse"]).abs().max().item() <= 1e-4


def test_decode_odd_shapes_against_oracle(cuda_device):
    """Seeded sweep over decode shapes: one key, fewer keys than a tile, KV lengths no tile divides,
    group sizes 2..24, head dims 64 / 128 / 256, both dtypes."""
    import random
    rng = random.Random(4321)
    cases = [(1, 2, 1, 1, 64), (2, 4, 2, 31, 128), (1, 24, 1, 4097, 128), (1, 6, 3, 257, 256), (3, 16, 8, 95, 64)]
    for _ in range(8):
        hkv = rng.choice([1, 2, 4])
        cases.append((rng.choice([1, 2, 5]), hkv * rng.choice([2, 3, 4, 8]), hkv, rng.randint(1, 3000),
                      rng.choice([64, 128])))
    for n, (B, Hq, Hkv, Skv, D) in enumerate(cases):
        dtype = torch.float16 if n % 2 == 0 else torch.bfloat16
        print(f"case odd decode B{B} Hq{Hq} Hkv{Hkv} Skv{Skv} D{D} {dtype}", flush=True)
        q, k, v = C.make_inputs(B, 1, Skv, Hq, Hkv, D, D, dtype, seed=100 + n)
        mod = _decode_engine(B, Hq, Hkv, Skv, D, D, dtype, C.make_scale_score_mod(1 / math.sqrt(D)), C.OnlineSoftmax())
        out = mod(q.cuda(), k.cuda(), v.cuda())
        ref, lse = R.softmax_attention(q, k, v, causal=False)
        assert torch.isfinite(out).all()
        assert (out.float().cpu() - ref).abs().max().item() <= OUT_TOL, (B, Hq, Hkv, Skv, D)
        assert (mod.final_rowscales["lse"].cpu() - lse).abs().max().item() <= LSE_TOL, (B, Hq, Hkv, Skv, D)


def test_mla_odd_shapes_against_oracle(cuda_device):
    """Seeded sweep over MLA decode shapes: head counts below and above a workgroup's 64, several latent
    heads, KV lengths from one token to lengths no tile divides, both dtypes, split and unsplit."""
    import random
    rng = random.Random(99)
    D, DV = 576, 512
    scale = 1 / math.sqrt(192)
    cases = [(1, 1, 1, 1), (1, 7, 1, 33), (2, 96, 1, 1023), (1, 160, 2, 130), (5, 64, 1, 64)]
    for _ in range(5):
        g = rng.choice([1, 2])
        cases.append((rng.choice([1, 3]), g * rng.choice([8, 40, 128]), g, rng.randint(1, 2500)))
    for n, (B, H, G, S) in enumerate(cases):
        dtype = torch.bfloat16 if n % 2 == 0 else torch.float16
        print(f"case odd mla B{B} H{H} G{G} S{S} {dtype}", flush=True)
        q, q_pe, kv, k_pe = _mla_inputs(B, H, G, S, DV, D - DV, dtype, seed=300 + n)
        mod = _mla_engine(B, H, G, S, D, DV, dtype, scale)
        out = mod(q.cuda(), q_pe.cuda(), kv.cuda(), k_pe.cuda())
        ref = torch.empty(B, H, DV)
        lse = torch.empty(B, H)
        hg = H // G
        for g in range(G):      # the oracle takes one latent head at a time
            r, l = R.mla_decode(q[:, 0, g * hg:(g + 1) * hg], q_pe[:, 0, g * hg:(g + 1) * hg], kv[:, :, g:g + 1],
                                k_pe[:, :, g:g + 1], scale=scale)
            ref[:, g * hg:(g + 1) * hg], lse[:, g * hg:(g + 1) * hg] = r, l
        assert torch.isfinite(out).all()
        assert (out[:, 0].float().cpu() - ref).abs().max().item() <= OUT_TOL, (B, H, G, S)
        assert (mod.final_rowscales["lse"][:, :, 0].cpu() - lse).abs().max().item() <= LSE_TOL, (B, H, G, S)


def test_decode_and_prefill_replay_from_a_hip_graph(cuda_device):
    """The launches go to the caller's stream and nothing but torch allocates, so a call can be captured into
    a HIP graph (serving loops do that for their decode step) and replayed on new contents of the same buffers.
    Every replay is checked against the eager result, with eager work between the replays."""
    B, Hq, Hkv, Skv, D = 4, 32, 8, 2048, 128
    dtype = torch.float16
    meta = (meta_tensor(B, Hq, 1, D, dtype=dtype), meta_tensor(B, Hkv, Skv, D, dtype=dtype),
            meta_tensor(B, Hkv, Skv, D, dtype=dtype))
    dec = AttentionEngine(meta, CustomIO({}), C.make_scale_score_mod(1 / math.sqrt(D)), None, C.OnlineSoftmax())
    S = 512
    pre = AttentionEngine((meta_tensor(1, 4, S, D, dtype=dtype),) * 3, CustomIO({}),
                          C.make_scale_score_mod(1 / math.sqrt(D)), C.causal_mask, C.OnlineSoftmax())
    q, k, v = (t.cuda() for t in C.make_inputs(B, 1, Skv, Hq, Hkv, D, D, dtype, seed=1))
    pq, pk, pv = (t.cuda() for t in C.make_inputs(1, S, S, 4, 4, D, D, dtype, seed=2))
    dec(q, k, v), pre(pq, pk, pv)                      # compile and warm up outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        dec(q, k, v), pre(pq, pk, pv)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_d = dec(q, k, v)
        out_p = pre(pq, pk, pv)
    for step in range(3):
        g = torch.Generator().manual_seed(10 + step)
        q.copy_(torch.randn(q.shape, generator=g).to(dtype))
        k.copy_(torch.randn(k.shape, generator=g).to(dtype))
        pq.copy_(torch.randn(pq.shape, generator=g).to(dtype))
        graph.replay()
        torch.cuda.synchronize()
        got_d, got_p = out_d.clone(), out_p.clone()
        ref_d, ref_p = dec(q, k, v), pre(pq, pk, pv)   # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got_d, ref_d), step
        assert torch.equal(got_p, ref_p), step
    ref, _ = R.softmax_attention(q.cpu(), k.cpu(), v.cpu(), causal=False)
    assert (got_d.float().cpu() - ref).abs().max().item() <= OUT_TOL
