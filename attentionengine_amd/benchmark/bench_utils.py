"""Benchmark / comparison harness the example scripts call.

Drop-in counterpart of attention_engine/benchmark/bench_utils.py: same
function names, arguments and printed quantities for ``do_bench`` (14-99), ``check_close``
(133-155), ``print_debug`` (158-192), ``do_bench_attention`` (1179-1360),
``do_bench_sigmoidattn`` (701-788) and ``do_bench_reluattn`` (949-1022).  Inputs are generated
exactly as there (``torch.cuda.manual_seed(0)``, ``torch.randn`` on the device in the order
q, k, v, do), FLOP counts use the reference's formulas (1185-1186), and the comparison reference
is the reference's own eager fallback (1250-1275: grouped einsum, ``tril`` mask to -inf,
``softmax(scores * scale)``, einsum), run on the GPU with torch.

Not carried over: the external-library baselines (flash_attn, FA3, flash_sigmoid, flashinfer) --
not installable here.  ``require_grad=True`` checks dq, dk, dv against autograd through the eager
reference and times the backward for softmax, sigmoid and relu attention; the retention harness accepts
it and skips the backward with a note.
"""
from __future__ import annotations


import torch
import torch.nn.functional as F


def do_bench(fn, warmup=25, rep=100, _n_warmup=0, _n_repeat=0, grad_to_none=None, quantiles=None,
             fast_flush=True, return_mode="mean"):
    """Mean (or min/max/median) runtime of ``fn`` in milliseconds, measured with device events
    around back-to-back calls: ``warmup`` / ``rep`` are time budgets in ms from which the call
    counts are derived with a 5-call estimate, as in the reference."""
    assert return_mode in ("min", "max", "mean", "median")
    fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(5):
        fn()
    end.record()
    torch.cuda.synchronize()
    estimate_ms = start.elapsed_time(end) / 5
    n_warmup = _n_warmup if _n_warmup > 0 else max(1, int(warmup / max(estimate_ms, 1e-6)))
    n_repeat = _n_repeat if _n_repeat > 0 else max(1, int(rep / max(estimate_ms, 1e-6)))
    for _ in range(n_warmup):
        fn()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for i in range(n_repeat):
        if grad_to_none is not None:
            for x in grad_to_none:
                x.grad = None
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    times = torch.tensor([s.elapsed_time(e) for s, e in zip(starts, ends)], dtype=torch.float)
    if quantiles is not None:
        ret = torch.quantile(times, torch.tensor(quantiles, dtype=torch.float)).tolist()
        return ret[0] if len(ret) == 1 else ret
    return getattr(torch, return_mode)(times).item()


def check_close(o, O_ref, rtol=1e-3, atol=1e-3):
    """True if every element is within atol OR rtol; prints the share that is not."""
    abs_err = torch.abs(o - O_ref)
    rel_err = abs_err / (torch.abs(O_ref) + 1e-6)
    ok = (abs_err < atol) | (rel_err < rtol)
    bad = (~ok).sum().item()
    print(f"{bad / o.numel() * 100:.2f}% of the elements are not close.")
    if bad:
        print("Error elements:")
        for idx in torch.nonzero(~ok, as_tuple=False)[:10]:
            t = tuple(idx.cpu().numpy())
            print(f"Index: {t}, Reference: {O_ref[t]}, Library: {o[t]}")
    return bool(torch.all(ok))


def print_debug(o, O_ref, rtol=1e-3, atol=1e-3, save_file=False):
    """Prints mismatch counts and the largest absolute / relative differences."""
    close = torch.isclose(o, O_ref, rtol=rtol, atol=atol)
    total, bad = o.numel(), (~close).sum().item()
    print(f"{bad} elements are not close.")
    print(f"{bad / total * 100:.2f}% of the elements are not close.")
    print(f"Total elements: {total}, Not close elements: {bad}")
    diff = (o - O_ref).abs()
    i = torch.unravel_index(diff.argmax(), o.shape)
    print(f"Max diff: {diff.max().item()} at index {tuple(int(x) for x in i)}")
    print(f"Reference: {O_ref[i]}")
    print(f"Library: {o[i]}")
    print(torch.allclose(o, O_ref, rtol=rtol, atol=atol))
    rel = diff / O_ref.abs()
    i = torch.unravel_index(rel.argmax(), o.shape)
    print(f"Max rel diff: {rel.max().item()} at index {tuple(int(x) for x in i)}")
    print(f"Reference: {O_ref[i]}")
    print(f"Library: {o[i]}")
    if save_file:
        for name, t in (("o_ref.txt", O_ref), ("o.txt", o)):
            with open(name, "w") as f:
                for idx, element in enumerate(t.cpu()):
                    f.write(f"{idx}: {element}\n")


def _eager_attention(query, key, value, softmax_scale, causal, chunk_heads=None):
    """The reference's eager fallback (bench_utils.py:1250-1275), evaluated in fp32 and in chunks of
    kv heads so the [B, heads, Sq, Skv] score tensor stays bounded."""
    B, Sq, Hq, D = query.shape
    Skv, Hkv = key.shape[1], key.shape[2]
    G = Hq // Hkv
    out = torch.empty(B, Sq, Hq, value.shape[-1], dtype=query.dtype, device=query.device)
    if chunk_heads is None:
        budget = 1 << 28  # score elements per chunk
        chunk_heads = max(1, min(Hkv, budget // max(1, B * G * Sq * Skv)))
    mask = None
    if causal:
        mask = torch.ones(Sq, Skv, device=query.device, dtype=torch.bool).tril()
    for h0 in range(0, Hkv, chunk_heads):
        h1 = min(Hkv, h0 + chunk_heads)
        q = query[:, :, h0 * G:h1 * G].float().reshape(B, Sq, h1 - h0, G, D)
        scores = torch.einsum("bshgd,bthd->bhgst", q, key[:, :, h0:h1].float())
        if mask is not None:
            scores = scores.masked_fill(~mask, float("-inf"))
        attention = F.softmax(scores * softmax_scale, dim=-1)
        o = torch.einsum("bhgst,bthd->bshgd", attention, value[:, :, h0:h1].float())
        out[:, :, h0 * G:h1 * G] = o.reshape(B, Sq, (h1 - h0) * G, -1).to(query.dtype)
    return out


def _report(name, latency_ms, flops):
    print("{}: {:.2f} ms".format(name, latency_ms))
    print("tflops: {:.2f}".format(flops / latency_ms * 1e-9))


def _check_and_time_backward(o, do, leaves, eager_one_head, bwd_flops, name="hip bwd"):
    """``o.backward(do)`` against autograd through an eager fp32 reference evaluated one (batch, kv head)
    group at a time (the full score tensor of the headline shapes does not fit twice), then its timing.
    ``leaves`` = (query, key, value) with requires_grad; ``eager_one_head(q, k, v)`` -> out for slices
    [1, S, g, D], [1, S, 1, D], [1, S, 1, DV] in fp32."""
    query, key, value = leaves
    o.backward(do, retain_graph=True)
    got = [t.grad.clone() for t in leaves]
    for t in leaves:
        t.grad = None
    want = [torch.zeros_like(t) for t in leaves]
    g = query.shape[2] // key.shape[2]
    for b0 in range(query.shape[0]):
        for h0 in range(key.shape[2]):
            qs = query[b0:b0 + 1, :, h0 * g:(h0 + 1) * g].detach().float().requires_grad_(True)
            ks = key[b0:b0 + 1, :, h0:h0 + 1].detach().float().requires_grad_(True)
            vs = value[b0:b0 + 1, :, h0:h0 + 1].detach().float().requires_grad_(True)
            eager_one_head(qs, ks, vs).backward(do[b0:b0 + 1, :, h0 * g:(h0 + 1) * g].float())
            want[0][b0:b0 + 1, :, h0 * g:(h0 + 1) * g] = qs.grad.to(query.dtype)
            want[1][b0:b0 + 1, :, h0:h0 + 1] = ks.grad.to(key.dtype)
            want[2][b0:b0 + 1, :, h0:h0 + 1] = vs.grad.to(value.dtype)
    for a_, b_ in zip(got, want):
        print_debug(a_, b_, rtol=1e-2, atol=1e-2)
    latency = do_bench(lambda: o.backward(do, retain_graph=True), warmup=50, rep=100)
    _report(name, latency, bwd_flops)
    return latency


def do_bench_attention(attn, B, H, S, D, DV, mod=None, dtype=torch.float16, seqlenq=None,
                       require_grad=False, causal=True, groupnum=None):
    """Softmax attention (MHA / GQA / decode): correctness print-out against the eager reference,
    then forward timing; with ``require_grad`` also dq/dk/dv against autograd through the eager
    reference and backward timing (bench_utils.py:1179-1360; backward flops 4*B*H*S^2*DV + 6*B*H*S^2*D,
    halved when causal, 1199-1201).  Returns (latency_ms, tflops, latency_ref_ms, tflops_ref)."""
    seqlenq = S if seqlenq is None else seqlenq
    groupnum = H if groupnum is None else groupnum
    tflops = 2 * B * H * seqlenq * S * D + 2 * B * H * seqlenq * S * DV
    tflops = tflops * 0.5 if causal else tflops
    bwd_tflops = (4 * B * H * seqlenq * S * DV + 6 * B * H * seqlenq * S * D) * (0.5 if causal else 1.0)
    torch.cuda.manual_seed(0)
    device = "cuda"
    query = torch.randn(B, seqlenq, H, D, device=device, dtype=dtype, requires_grad=require_grad)
    key = torch.randn(B, S, groupnum, D, device=device, dtype=dtype, requires_grad=require_grad)
    value = torch.randn(B, S, groupnum, DV, device=device, dtype=dtype, requires_grad=require_grad)
    do = torch.randn(B, seqlenq, H, DV, device=device, dtype=dtype)

    o = attn(query, key, value)
    scale = (1 / D) ** 0.5
    if require_grad:
        o.backward(do, retain_graph=True)
        dQ, dK, dV = query.grad.clone(), key.grad.clone(), value.grad.clone()
        query.grad = key.grad = value.grad = None
    with torch.no_grad():
        o_ref = _eager_attention(query, key, value, scale, causal)
    print_debug(o, o_ref)
    if require_grad:
        # autograd through the eager reference, one (batch, head) group at a time (the full score
        # tensor of the headline shape does not fit twice)
        gq, gk, gv = torch.zeros_like(query), torch.zeros_like(key), torch.zeros_like(value)
        g = H // groupnum
        for b0 in range(B):
            for h0 in range(groupnum):
                qs = query[b0:b0 + 1, :, h0 * g:(h0 + 1) * g].detach().float().requires_grad_(True)
                ks = key[b0:b0 + 1, :, h0:h0 + 1].detach().float().requires_grad_(True)
                vs = value[b0:b0 + 1, :, h0:h0 + 1].detach().float().requires_grad_(True)
                _eager_attention(qs, ks, vs, scale, causal).backward(do[b0:b0 + 1, :, h0 * g:(h0 + 1) * g].float())
                gq[b0:b0 + 1, :, h0 * g:(h0 + 1) * g] = qs.grad.to(dtype)
                gk[b0:b0 + 1, :, h0:h0 + 1] = ks.grad.to(dtype)
                gv[b0:b0 + 1, :, h0:h0 + 1] = vs.grad.to(dtype)
        print_debug(dQ, gq)
        print_debug(dK, gk)
        print_debug(dV, gv)

    with torch.no_grad():
        latency = do_bench(lambda: attn(query, key, value), warmup=50, rep=100)
        _report("hip", latency, tflops)
        latency_ref = do_bench(lambda: _eager_attention(query, key, value, scale, causal), warmup=50, rep=100)
        _report("eager torch", latency_ref, tflops)
    if require_grad:
        latency_bwd = do_bench(lambda: o.backward(do, retain_graph=True), warmup=50, rep=100)
        _report("hip bwd", latency_bwd, bwd_tflops)
    return latency, tflops / latency * 1e-9, latency_ref, tflops / latency_ref * 1e-9


def do_bench_sigmoidattn(attn, B, H, S, D, DV, dtype=torch.float16, requires_grad=False, causal=True):
    """Sigmoid attention of attn_script/sigmoidattn.py: out = sum_kv sigmoid(s + bias) v under a
    causal mask, ``softmax_bias`` an fp32 tensor of shape [1] passed as the 4th argument
    (bench_utils.py:723-729)."""
    tflops = (2 * B * H * S * S * D + 2 * B * H * S * S * DV) * (0.5 if causal else 1.0)
    torch.cuda.manual_seed(0)
    device = "cuda"
    query = torch.randn(B, S, H, D, device=device, dtype=dtype, requires_grad=requires_grad)
    key = torch.randn(B, S, H, D, device=device, dtype=dtype, requires_grad=requires_grad)
    value = torch.randn(B, S, H, DV, device=device, dtype=dtype, requires_grad=requires_grad)
    do = torch.randn(B, S, H, DV, device=device, dtype=dtype)
    softmax_bias = 0.1 * torch.randn(1, device=device, dtype=torch.float32)

    o = attn(query, key, value, softmax_bias)
    if requires_grad:
        def one_head(qs, ks, vs):
            sc = torch.einsum("bqhd,bkhd->bhqk", qs, ks)
            pr = torch.sigmoid(sc + softmax_bias)
            if causal:
                pr = pr.masked_fill(~torch.ones(S, S, device=device, dtype=torch.bool).tril(), 0.0)
            return torch.einsum("bhqk,bkhd->bqhd", pr, vs)
        _check_and_time_backward(o, do, (query, key, value), one_head, 2.5 * tflops)
        query, key, value = query.detach(), key.detach(), value.detach()

    def ref():
        out = torch.empty_like(o)
        mask = torch.ones(S, S, device=device, dtype=torch.bool).tril() if causal else None
        for h0 in range(0, H, 4):
            s = torch.einsum("bqhd,bkhd->bhqk", query[:, :, h0:h0 + 4].float(), key[:, :, h0:h0 + 4].float())
            p = torch.sigmoid(s + softmax_bias)
            if mask is not None:
                p = p.masked_fill(~mask, 0.0)
            out[:, :, h0:h0 + 4] = torch.einsum("bhqk,bkhd->bqhd", p, value[:, :, h0:h0 + 4].float()).to(dtype)
        return out
    print_debug(o, ref(), rtol=1e-2, atol=1e-2)
    latency = do_bench(lambda: attn(query, key, value, softmax_bias), warmup=50, rep=100)
    _report("hip", latency, tflops)
    latency_ref = do_bench(ref, warmup=50, rep=100)
    _report("eager torch", latency_ref, tflops)
    return latency, tflops / latency * 1e-9, latency_ref, tflops / latency_ref * 1e-9


def do_bench_reluattn(attn, B, H, S, D, DV, dtype=torch.float16, causal=False, requires_grad=False):
    """ReLU attention of attn_script/reluattn.py; reference = bench_utils.py:979-984."""
    tflops = (2 * B * H * S * S * D + 2 * B * H * S * S * DV) * (0.5 if causal else 1.0)
    torch.cuda.manual_seed(0)
    device = "cuda"
    query = torch.randn(B, S, H, D, device=device, dtype=dtype, requires_grad=requires_grad)
    key = torch.randn(B, S, H, D, device=device, dtype=dtype, requires_grad=requires_grad)
    value = torch.randn(B, S, H, DV, device=device, dtype=dtype, requires_grad=requires_grad)
    do = torch.randn(B, S, H, DV, device=device, dtype=dtype)

    o = attn(query, key, value)
    if requires_grad:
        def one_head(qs, ks, vs):
            pr = F.relu(torch.einsum("bqhd,bkhd->bhqk", qs, ks) / (D ** 0.5))
            if causal:
                pr = pr.masked_fill(~torch.ones(S, S, device=device, dtype=torch.bool).tril(), 0.0)
            return torch.einsum("bhqk,bkhd->bqhd", pr, vs)
        _check_and_time_backward(o, do, (query, key, value), one_head, 2.5 * tflops)
        query, key, value = query.detach(), key.detach(), value.detach()

    def ref_program():
        qk = torch.einsum("bqhd,bkhd->bhqk", query, key) / (D ** 0.5)
        qk = F.relu(qk)
        if causal:
            qk = qk.masked_fill(~torch.ones(S, S, device=device, dtype=torch.bool).tril(), 0.0)
        return torch.einsum("bhqk,bkhd->bqhd", qk, value)
    print_debug(o, ref_program(), rtol=1e-2, atol=1e-2)
    latency = do_bench(lambda: attn(query, key, value), warmup=50, rep=100)
    _report("hip", latency, tflops)
    latency_ref = do_bench(ref_program, warmup=50, rep=100)
    _report("eager torch", latency_ref, tflops)
    return latency, tflops / latency * 1e-9, latency_ref, tflops / latency_ref * 1e-9


def do_bench_retention(attn, B, H, S, D, DV, dtype=torch.bfloat16):
    """Retention with a decay-mask input (attn_script/retention.py); inputs, reference and flop
    count as bench_utils.py:1025-1100 of the reference: q scaled by D^-0.5, mask = rand.tril()."""
    tflops = (2 * B * H * S * S * D + 2 * B * H * S * S * DV) * 0.5
    torch.cuda.manual_seed(0)
    device = "cuda"
    query = torch.randn(B, S, H, D, device=device, dtype=dtype) * ((1 / D) ** 0.5)
    key = torch.randn(B, S, H, D, device=device, dtype=dtype)
    value = torch.randn(B, S, H, DV, device=device, dtype=dtype)
    torch.randn(B, S, H, DV, device=device, dtype=dtype)
    mask = torch.rand(1, H, S, S, device=device, dtype=dtype).tril().contiguous()

    o = attn(query, key, value, mask)

    def ref_program():
        qk = torch.einsum("bqhd,bkhd->bhqk", query, key)
        qkm = qk * mask
        r = qkm.abs().sum(dim=-1, keepdim=True).clamp(min=1.0)
        return torch.einsum("bhqk,bkhd->bqhd", qkm / r, value).to(dtype)
    print_debug(o, ref_program(), rtol=1e-2, atol=1e-2)
    latency = do_bench(lambda: attn(query, key, value, mask), warmup=50, rep=100)
    _report("hip", latency, tflops)
    latency_ref = do_bench(ref_program, warmup=50, rep=100)
    _report("eager torch", latency_ref, tflops)
    return latency, tflops / latency * 1e-9, latency_ref, tflops / latency_ref * 1e-9
