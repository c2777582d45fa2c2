"""Closed-form CPU references (fp32 or fp64 torch on the host).  Test infrastructure only.

Each function restates one eager reference of microsoft/AttentionEngine and says which:
runtime layouts are the reference's, q [B,Sq,Hq,D], k [B,Skv,Hkv,D], v [B,Skv,Hkv,DV],
out [B,Sq,Hq,DV], lse [B,Hq,Sq].
"""
from __future__ import annotations

import math

import torch


def _grouped_scores(q, k, compute_dtype):
    """QK^T with grouped heads: q head h uses kv head h // (Hq/Hkv).  Returns [B,Hkv,G,Sq,Skv].

    Follows the fallback ``flash_attn_func`` of attention_engine/benchmark/bench_utils.py:1250-1262
    (rearrange 'b s (h g) d -> b s g h d', einsum '... -> b g h s t')."""
    B, Sq, Hq, D = q.shape
    _, Skv, Hkv, _ = k.shape
    assert Hq % Hkv == 0
    G = Hq // Hkv
    qg = q.to(compute_dtype).reshape(B, Sq, Hkv, G, D)
    return torch.einsum("bshgd,bthd->bhgst", qg, k.to(compute_dtype))


def _apply_p(p, v, compute_dtype):
    """P [B,Hkv,G,Sq,Skv] times V [B,Skv,Hkv,DV] -> [B,Sq,Hq,DV] (bench_utils.py:1272-1274)."""
    B, Hkv, G, Sq, _ = p.shape
    out = torch.einsum("bhgst,bthd->bshgd", p, v.to(compute_dtype))
    return out.reshape(B, Sq, Hkv * G, v.shape[-1])


def _mask_to_grouped(mask, B, Hkv, G, Sq, Skv):
    """bool mask broadcastable to [B,Hq,Sq,Skv] -> [B,Hkv,G,Sq,Skv]."""
    m = mask
    while m.dim() < 4:
        m = m.unsqueeze(0)
    m = m.expand(B, Hkv * G, Sq, Skv)
    return m.reshape(B, Hkv, G, Sq, Skv)


def softmax_attention(q, k, v, scale=None, causal=False, mask=None, compute_dtype=torch.float32):
    """softmax(mask(QK^T) * scale) V and lse = logsumexp(mask(QK^T) * scale).

    Restates bench_utils.py:1250-1275: scores = einsum; if causal, ``tril`` mask -> -inf (1263-1269);
    ``softmax(scores * softmax_scale)`` (1270-1271); einsum with V (1272-1274).  lse restates
    attn_script/mla_decode_cute.py:102 (``attn_weight.logsumexp(-1)``) = log(r) + m of the
    OnlineSoftmax epilogue (attn_script/mha.py:66-72).  ``mask`` (bool, True = visible) replaces
    the causal mask for block-sparse / sliding-window cases (attn_script/blocksparseattn.py:129-135).
    Rows with no visible key give out = 0, lse = -inf.
    """
    B, Sq, Hq, D = q.shape
    Skv, Hkv = k.shape[1], k.shape[2]
    G = Hq // Hkv
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    s = _grouped_scores(q, k, compute_dtype)
    if causal:
        tril = torch.ones(Sq, Skv, dtype=torch.bool).tril()
        s = s.masked_fill(~tril, float("-inf"))
    if mask is not None:
        s = s.masked_fill(~_mask_to_grouped(mask, B, Hkv, G, Sq, Skv), float("-inf"))
    s = s * scale
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse.unsqueeze(-1).clamp(min=-3.0e38))
    p = torch.where(torch.isfinite(lse).unsqueeze(-1), p, torch.zeros_like(p))
    out = _apply_p(p, v, compute_dtype)
    return out, lse.reshape(B, Hq, Sq)


def softmax_attention_grads(q, k, v, do, scale=None, causal=False, mask=None, compute_dtype=torch.float32):
    """Gradients (dq, dk, dv) of ``softmax_attention`` for the output gradient ``do`` [B,Sq,Hq,DV].

    Restates the backward the reference generates for attn_script/mha.py: recompute
    p = exp(s*scale - lse) (OnlineSoftmax.forward, mha.py:75-78), dv = p^T do, dp = do v^T,
    ds = p * (dp - rowsum(do * o)) (OnlineSoftmax.backward, mha.py:80-84, with the
    ``doosum`` row scale of flashattn_bwd_preprocess, attn_tl.py:196-221), score_mod's derivative
    (the constant ``scale``), dq = ds k, dk = ds^T q (attn_tl.py:330-420); grouped heads sum into their
    kv head.  Pinned in tests/test_oracle.py against torch.autograd through ``softmax_attention``.
    """
    B, Sq, Hq, D = q.shape
    Skv, Hkv = k.shape[1], k.shape[2]
    G = Hq // Hkv
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    s = _grouped_scores(q, k, compute_dtype)
    vis = torch.ones(B, Hkv, G, Sq, Skv, dtype=torch.bool)
    if causal:
        vis = vis & torch.ones(Sq, Skv, dtype=torch.bool).tril()
    if mask is not None:
        vis = vis & _mask_to_grouped(mask, B, Hkv, G, Sq, Skv)
    s = s.masked_fill(~vis, float("-inf")) * scale
    lse = torch.logsumexp(s, dim=-1, keepdim=True)
    p = torch.where(torch.isfinite(lse), torch.exp(s - lse.clamp(min=-3.0e38)), torch.zeros_like(s))
    dog = do.to(compute_dtype).reshape(B, Sq, Hkv, G, -1)                 # [B,Sq,Hkv,G,DV]
    vf = v.to(compute_dtype)
    dv = torch.einsum("bhgst,bshgd->bthd", p, dog)
    dp = torch.einsum("bshgd,bthd->bhgst", dog, vf)
    delta = (dp * p).sum(-1, keepdim=True)                                 # = rowsum(do * o)
    ds = p * (dp - delta) * scale
    dq = torch.einsum("bhgst,bthd->bshgd", ds, k.to(compute_dtype)).reshape(B, Sq, Hq, D)
    dk = torch.einsum("bhgst,bshgd->bthd", ds, q.to(compute_dtype).reshape(B, Sq, Hkv, G, D))
    return dq, dk, dv


def sigmoid_attention(q, k, v, scale=None, bias=0.0, causal=False, compute_dtype=torch.float32):
    """out = sum_kv sigmoid(QK^T * scale + bias) V, no normalisation.

    The reference has no eager sigmoid reference (bench_utils.py:736-744 compares against the
    external ``flash_sigmoid`` package only); this is the closed form of attn_script/sigmoidattn.py:
    14-18 (``((score + bias) * 0.5).tanh() + 1) * 0.5`` == sigmoid(score + bias)) with the score
    scaling of the benchmark configuration applied first.  Masked positions contribute 0.
    """
    B, Sq, Hq, D = q.shape
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    s = _grouped_scores(q, k, compute_dtype) * scale + bias
    p = torch.sigmoid(s)
    if causal:
        tril = torch.ones(Sq, k.shape[1], dtype=torch.bool).tril()
        p = p.masked_fill(~tril, 0.0)
    return _apply_p(p, v, compute_dtype)


def relu_attention(q, k, v, scale=None, compute_dtype=torch.float32):
    """out = relu(QK^T / sqrt(D)) V (restates bench_utils.py:979-984)."""
    D = q.shape[-1]
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    p = torch.relu(_grouped_scores(q, k, compute_dtype) * scale)
    return _apply_p(p, v, compute_dtype)


def elementwise_attention_grads(q, k, v, do, kind, scale=None, bias=0.0, causal=False,
                                compute_dtype=torch.float32):
    """Gradients (dq, dk, dv) of ``sigmoid_attention`` (kind "sigmoid") and ``relu_attention`` (kind
    "relu"): out = sum_kv f(s) v has dv = p^T do, ds = (do v^T) * f'(s), dq = ds k, dk = ds^T q -- what the
    reference's backward computes for attn_script/sigmoidattn.py and reluattn.py, whose online function
    passes scores and dp through (``OnlineIdentity.forward/backward``) and whose f' comes from the symbolic
    derivative of score_mod (core/transform/core.py:119-199).  relu' is 0 at 0.  Pinned in
    tests/test_oracle.py against torch.autograd through the two forward functions."""
    B, Sq, Hq, D = q.shape
    Skv, Hkv = k.shape[1], k.shape[2]
    G = Hq // Hkv
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    s = _grouped_scores(q, k, compute_dtype) * scale
    if kind == "sigmoid":
        p = torch.sigmoid(s + bias)
        dpds = p * (1.0 - p) * scale
    elif kind == "relu":
        p = torch.relu(s)
        dpds = (s > 0).to(compute_dtype) * scale
    else:
        raise ValueError(kind)
    if causal:
        tril = torch.ones(Sq, Skv, dtype=torch.bool).tril()
        p = p.masked_fill(~tril, 0.0)
        dpds = dpds.masked_fill(~tril, 0.0)
    dog = do.to(compute_dtype).reshape(B, Sq, Hkv, G, -1)
    dv = torch.einsum("bhgst,bshgd->bthd", p, dog)
    ds = torch.einsum("bshgd,bthd->bhgst", dog, v.to(compute_dtype)) * dpds
    dq = torch.einsum("bhgst,bthd->bshgd", ds, k.to(compute_dtype)).reshape(B, Sq, Hq, D)
    dk = torch.einsum("bhgst,bshgd->bthd", ds, q.to(compute_dtype).reshape(B, Sq, Hkv, G, D))
    return dq, dk, dv


def retention_attention(q, k, v, mask, compute_dtype=torch.float32):
    """Retention with a decay mask: s = (QK^T) * mask, out = (s / max(sum_kv |s|, 1)) V, r = that
    clamped row sum (restates ``ref_program`` of bench_utils.py:1062-1067; the running form of
    attn_script/retention.py:32-58 telescopes to it).  mask [1|B, Hq, Sq, Skv]; returns
    (out [B,Sq,Hq,DV], r [B,Hq,Sq])."""
    B, Sq, Hq, _ = q.shape
    Hkv = k.shape[2]
    s = _grouped_scores(q, k, compute_dtype)                          # [B,Hkv,G,Sq,Skv]
    m = mask.to(compute_dtype).expand(B, Hq, Sq, k.shape[1]).reshape(B, Hkv, Hq // Hkv, Sq, k.shape[1])
    s = s * m
    r = s.abs().sum(dim=-1, keepdim=True).clamp(min=1.0)
    return _apply_p(s / r, v, compute_dtype), r.reshape(B, Hq, Sq)


def retention_attention_grads(q, k, v, mask, do, compute_dtype=torch.float32):
    """Gradients (dq, dk, dv) the reference's backward produces for attn_script/retention.py: recompute
    p = (s * mask) / r with the SAVED row scale r (OnlineRetention.forward, retention.py:60-63),
    dv = p^T do, dp = do v^T, dscores = dp / r (OnlineRetention.backward, retention.py:65-70: r is a
    constant there, its dependence on the scores is not differentiated), score_mod's derivative (the mask,
    retention.py:14-16), dq = ds k, dk = ds^T q.  Pinned in tests/test_oracle.py against torch.autograd
    through ``retention_attention``'s formula with r detached."""
    B, Sq, Hq, D = q.shape
    Skv, Hkv = k.shape[1], k.shape[2]
    G = Hq // Hkv
    m = mask.to(compute_dtype).expand(B, Hq, Sq, Skv).reshape(B, Hkv, G, Sq, Skv)
    s = _grouped_scores(q, k, compute_dtype) * m
    r = s.abs().sum(dim=-1, keepdim=True).clamp(min=1.0)
    p = s / r
    dog = do.to(compute_dtype).reshape(B, Sq, Hkv, G, -1)
    dv = torch.einsum("bhgst,bshgd->bthd", p, dog)
    dp = torch.einsum("bshgd,bthd->bhgst", dog, v.to(compute_dtype))
    ds = dp / r * m
    dq = torch.einsum("bhgst,bthd->bshgd", ds, k.to(compute_dtype)).reshape(B, Sq, Hq, D)
    dk = torch.einsum("bhgst,bshgd->bthd", ds, q.to(compute_dtype).reshape(B, Sq, Hkv, G, D))
    return dq, dk, dv


def mla_decode(q, q_pe, kv, k_pe, scale=None, compute_dtype=torch.float32):
    """MLA decode: K = [kv | k_pe], V = kv, one latent kv head shared by all q heads.

    q [B,Hq,DV], q_pe [B,Hq,DPE], kv [B,Skv,Hkv,DV], k_pe [B,Skv,Hkv,DPE] -> (out [B,Hq,DV],
    lse [B,Hq]).  Restates ``ref_program`` of core/template/tl_template/attn/mla_decode_tl.py:266-306
    (concat, einsum, softmax(scores / sqrt(dim + pe_dim)), einsum with kv); lse as in
    attn_script/mla_decode_cute.py:88-105.  ``scale`` defaults to the reference's 1/sqrt(D+DPE).
    """
    D = q.shape[-1] + q_pe.shape[-1]
    scale = 1.0 / math.sqrt(D) if scale is None else scale
    query = torch.cat([q, q_pe], dim=-1).unsqueeze(1)      # [B,1,Hq,D]
    key = torch.cat([kv, k_pe], dim=-1)                     # [B,Skv,Hkv,D]
    out, lse = softmax_attention(query, key, kv, scale=scale, compute_dtype=compute_dtype)
    return out[:, 0], lse[:, :, 0]


def merge_partials(partial_o, partial_lse):
    """Split-KV merge: partial_o [..., n_split, DV] (each normalised within its split),
    partial_lse [..., n_split] natural log -> (o [..., DV], lse [...]).

    Restates ``combine`` of attn_script/gqa_inference.py:73-81 (lse_max, sum exp(lse - lse_max),
    lse_sum = log(sum) + lse_max, o_scale = exp(lse - lse_sum)) and the accumulation loop of
    core/template/tl_template/attn/attn_decode_tl.py:184-189."""
    lse_max = partial_lse.max(dim=-1, keepdim=True).values
    lse_max = torch.where(torch.isfinite(lse_max), lse_max, torch.zeros_like(lse_max))
    w = torch.exp(partial_lse - lse_max)
    lse = torch.log(w.sum(dim=-1, keepdim=True)) + lse_max
    o_scale = torch.exp(partial_lse - lse)
    o = (partial_o * o_scale.unsqueeze(-1)).sum(dim=-2)
    return o, lse.squeeze(-1)
