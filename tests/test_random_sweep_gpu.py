"""Seeded random sweeps over shapes, dtypes, masks, graphs and tile configurations, each case against the CPU
oracle on the same inputs (out <= 2e-2, lse <= 1e-3; gradients as in test_prefill_bwd_gpu.py).  The fixed suites
test the shapes someone thought of; a sweep like this one found a build (value head dim 512, tile table, ragged
tiles) whose compiled code lost a register."""
import math
import os
import random

import pytest
import torch

import attn_cases as C
from attn_engine import AttentionEngine
from core import CustomIO, meta_tensor
from core.lower.prefill_op import PrefillOp
from oracle import attention_ref as R
from oracle import masks as M

pytestmark = pytest.mark.gpu


def _mask(name, window=70):
    return {None: None, "causal": C.causal_mask, "window": C.make_sliding_window_mask(window),
            "head": C.head_dependent_mask, "shifted": C.causal_shifted_mask}[name]


@pytest.mark.parametrize("seed", [1, 2])
def test_prefill_forward_sweep(cuda_device, seed):
    """Every head dim class (direct-to-LDS: 64 ... 256 x 64 ... 512; register-staged: the others), softmax /
    sigmoid / relu graphs, no mask / causal / sliding window, grouped heads, one of the tile configurations the
    tuner may pick chosen at random."""
    rng = random.Random(seed)
    for case in range(40):
        D = rng.choice([64, 80, 96, 112, 128, 160, 192, 224, 256])
        DV = rng.choice([64, 128, 256, 512] if D in (64, 128, 256) else [64, 96, 128, 160, 256])
        dt = rng.choice([torch.float16, torch.bfloat16])
        B, Hkv, G = rng.choice([1, 2]), rng.choice([1, 2, 3]), rng.choice([1, 1, 2, 4])
        H = Hkv * G
        S = rng.choice([1, 31, 64, 100, 128, 257, 333, 512, 640])
        mask = rng.choice([None, "causal", "window", "causal"])
        kind = rng.choice(["softmax", "softmax", "sigmoid", "relu"])
        mask_mod = _mask(mask)
        q, k, v = C.make_inputs(B, S, S, H, Hkv, D, DV, dt, seed=case + 1000 * seed)
        meta = (meta_tensor(B, H, S, D, dtype=dt), meta_tensor(B, Hkv, S, D, dtype=dt),
                meta_tensor(B, Hkv, S, DV, dtype=dt))
        scale = 1 / math.sqrt(D)
        mk = None if mask_mod is None else mask_mod(0, 0, torch.arange(S)[:, None], torch.arange(S)[None, :])[None, None]
        extra, lse = (), None
        if kind == "softmax":
            args = (meta, CustomIO({}), C.make_scale_score_mod(scale), mask_mod, C.OnlineSoftmax(), "-inf")
            ref, lse = R.softmax_attention(q, k, v, mask=mk)
        else:
            s = torch.einsum("bqhd,bkhd->bhqk", q.float(), k.float().repeat_interleave(G, 2)) * scale
            if kind == "sigmoid":
                bias = torch.tensor([-math.log(max(S, 2))])
                args = (meta, CustomIO({"softmax_bias": (1,)}), C.make_sigmoid_score_mod(scale), mask_mod,
                        C.OnlineIdentity(), "-inf")
                extra, p = (bias.cuda(),), torch.sigmoid(s + bias.item())
            else:
                args = (meta, CustomIO({}), C.make_relu_score_mod(scale), mask_mod, C.OnlineIdentity(), "-inf")
                p = torch.relu(s)
            if mk is not None:
                p = p * mk
            ref = torch.einsum("bhqk,bkhd->bqhd", p, v.float().repeat_interleave(G, 2))
        base = PrefillOp(*args)
        t = rng.choice(base._tune_candidates())
        print(f"case {case}: B{B} H{H}/{Hkv} S{S} D{D} DV{DV} {dt} {kind} {mask} {t.template} bn{t.block_n} "
              f"w{t.waves_per_eu}", flush=True)
        op = base if t == base.tiles else PrefillOp(*args, tiles=t)
        out = op(q.cuda(), k.cuda(), v.cuda(), *extra, *([op.block_mask] if op.block_mask is not None else []))
        tol = 2e-2 * max(1.0, ref.abs().max().item() / 4)      # unnormalised graphs: relative to the output's size
        assert (out.float().cpu() - ref).abs().max().item() <= tol
        if lse is not None:
            got, fin = op.final_rowscales["lse"].cpu(), torch.isfinite(lse)
            assert (got[fin] - lse[fin]).abs().max().item() <= 1e-3 if fin.any() else True
            assert torch.equal(got[~fin], lse[~fin])


def test_prefill_backward_sweep(cuda_device):
    rng = random.Random(7)
    for case in range(30):
        D, DV = rng.choice([64, 128]), rng.choice([64, 128])
        dt = rng.choice([torch.float16, torch.bfloat16])
        B, Hkv, G = rng.choice([1, 2]), rng.choice([1, 2]), rng.choice([1, 2, 3])
        H = Hkv * G
        S = rng.choice([1, 33, 64, 100, 128, 200, 257, 384, 520])
        mask = rng.choice([None, "causal", "window", "head", "shifted"])
        mask_mod = _mask(mask, rng.choice([40, 100, 300]))
        scale = 1 / math.sqrt(D)
        print(f"case {case}: B{B} H{H}/{Hkv} S{S} D{D} DV{DV} {dt} {mask}", flush=True)
        q, k, v = C.make_inputs(B, S, S, H, Hkv, D, DV, dt, seed=case + 7000)
        do = torch.randn(B, S, H, DV, generator=torch.Generator().manual_seed(case + 5)).to(dt)
        meta = (meta_tensor(B, H, S, D, dtype=dt), meta_tensor(B, Hkv, S, D, dtype=dt),
                meta_tensor(B, Hkv, S, DV, dtype=dt))
        mod = AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(scale), mask_mod=mask_mod,
                              online_func=C.OnlineSoftmax())
        qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
        mod(qd, kd, vd).backward(do.cuda())
        causal = mask == "causal"
        dense = None
        if mask_mod is not None and not causal:
            dense = torch.from_numpy(M.dense_mask_grid(mask_mod, B, H, S, S))
        for name, got, want in zip(("dq", "dk", "dv"), (qd.grad, kd.grad, vd.grad),
                                   R.softmax_attention_grads(q, k, v, do, scale=scale, causal=causal, mask=dense)):
            err = (got.float().cpu() - want).abs().max().item()
            assert math.isfinite(err) and err <= 2e-2 + 1e-2 * want.abs().max().item(), (name, err)


def test_decode_sweep(cuda_device, monkeypatch):
    """GQA decode, split-KV decode with several query tokens, and MLA decode over a paged cache with shuffled
    pages, per-entry lengths (empty entries too), page sizes, split counts and both MLA kernels."""
    rng = random.Random(11)
    for case in range(40):
        kind = rng.choice(["gqa", "gqa", "mha_split"])
        dt = rng.choice([torch.float16, torch.bfloat16])
        D = rng.choice([64, 128])
        DV = D if kind == "mha_split" else rng.choice([64, 128])
        B = rng.choice([1, 2, 3, 7])
        if kind == "gqa":
            Hkv, G, Sq = rng.choice([1, 2, 4]), rng.choice([2, 4, 8, 20]), 1
            Hq = Hkv * G
        else:
            Hq = Hkv = rng.choice([1, 2, 5])
            Sq = rng.choice([1, 5, 64, 128])
        Skv = rng.choice([33, 96, 300, 1000, 1024, 2049, 4096])
        if kind == "mha_split" and Sq >= Skv:
            Skv = 4096
        tw = rng.choice([1, 16, 64, 512, 2048])
        print(f"case {case}: {kind} {dt} B{B} Hq{Hq} Hkv{Hkv} Sq{Sq} Skv{Skv} D{D} DV{DV} target{tw}", flush=True)
        q, k, v = C.make_inputs(B, Sq, Skv, Hq, Hkv, D, DV, dt, seed=case + 31)
        meta = (meta_tensor(B, Hq, Sq, D, dtype=dt), meta_tensor(B, Hkv, Skv, D, dtype=dt),
                meta_tensor(B, Hkv, Skv, DV, dtype=dt))
        mod = AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(1 / math.sqrt(D)), mask_mod=None,
                              online_func=C.OnlineSoftmax())
        mod.attention.target_workgroups = tw
        out = mod(q.cuda(), k.cuda(), v.cuda())
        ref, lse = R.softmax_attention(q, k, v, causal=False)
        assert (out.float().cpu() - ref).abs().max().item() <= 2e-2
        assert (mod.final_rowscales["lse"].cpu() - lse).abs().max().item() <= 1e-3
    D, DV, G = 576, 512, 1
    scale = 1 / math.sqrt(D)
    for case in range(30):
        dt = rng.choice([torch.float16, torch.bfloat16])
        B, H, page = rng.choice([1, 2, 3, 5]), rng.choice([16, 64, 128]), rng.choice([32, 64, 128])
        maxlen = rng.choice([64, 200, 700, 1500])
        lens = [rng.choice([0, 1, rng.randint(1, maxlen), maxlen]) for _ in range(B)]
        if max(lens) == 0:
            lens[0] = 5
        target, kernel = rng.choice([1, 8, 64, 256]), rng.choice(["ws", "ws", "generic"])
        monkeypatch.setenv("AE_MLA_KERNEL", "generic" if kernel == "generic" else "")
        max_pages = -(-max(lens) // page) + rng.choice([0, 1])
        n_pages = B * max_pages + 2
        g = torch.Generator().manual_seed(case + 77)
        perm = torch.randperm(n_pages, generator=g)
        table = torch.full((B, max_pages), n_pages + 5, dtype=torch.int32)
        cache = torch.full((n_pages, page, G, D), float("nan"), dtype=dt)
        q = torch.randn(B, 1, H, D, generator=g).to(dt)
        dense = torch.randn(B, max_pages * page, G, D, generator=g).to(dt)
        used = 0
        for b in range(B):
            for j in range(-(-lens[b] // page)):
                pg = int(perm[used])
                used += 1
                table[b, j] = pg
                cache[pg] = dense[b, j * page:(j + 1) * page]
        print(f"case {case}: mla {kernel} {dt} B{B} H{H} page{page} lens{lens} target{target}", flush=True)
        meta = (meta_tensor(B, H, 1, D, dtype=dt), meta_tensor(B, G, max_pages * page, D, dtype=dt),
                meta_tensor(B, G, max_pages * page, DV, dtype=dt))
        mod = AttentionEngine(meta, CustomIO({}), score_mod=C.make_scale_score_mod(scale), mask_mod=None,
                              online_func=C.OnlineSoftmax(), kv_shared=True, backend="cute")
        mod.attention.target_workgroups = target
        out, lse = mod(q.cuda(), cache.cuda(), block_table=table.cuda(),
                       cache_seqlens=torch.tensor(lens, dtype=torch.int32).cuda())
        for b in range(B):
            n = lens[b]
            if n == 0:
                assert (out[b] == 0).all() and (lse[b] == float("-inf")).all()
                continue
            ref, lref = R.mla_decode(q[b:b + 1, 0, :, :DV], q[b:b + 1, 0, :, DV:], dense[b:b + 1, :n, :, :DV],
                                     dense[b:b + 1, :n, :, DV:], scale=scale)
            assert (out[b:b + 1, 0].float().cpu() - ref).abs().max().item() <= 2e-2, b
            assert (lse[b:b + 1, :, 0].cpu() - lref).abs().max().item() <= 1e-3, b
