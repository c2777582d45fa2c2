"""Brute-force mask evaluation on the host.  Test infrastructure only.

``dense_mask`` calls ``mask_mod(b, h, q_idx, kv_idx)`` on the full index grid; ``block_any`` /
``block_classes`` restate ``_convert_mask_to_block_mask`` of
attention_engine/core/transform/core.py:410-453 (a block is set when ANY element is visible;
"full" when all are); ``block_causal_pattern`` / ``no_block_above_diagonal`` restate
``is_causal_mask`` (455-470) and ``is_less_causal_mask`` (472-488).  Written with numpy so that
it shares no code with the product's torch implementation.
"""
from __future__ import annotations

import numpy as np


def dense_mask(mask_mod, B, H, Sq, Skv):
    """bool ndarray [B,H,Sq,Skv] by calling mask_mod on python ints (slow; tiny shapes only)
    -- the pure-python ground truth."""
    out = np.zeros((B, H, Sq, Skv), dtype=bool)
    for b in range(B):
        for h in range(H):
            for q in range(Sq):
                for kv in range(Skv):
                    out[b, h, q, kv] = bool(mask_mod(b, h, q, kv))
    return out


def dense_mask_grid(mask_mod, B, H, Sq, Skv):
    """Same mask evaluated on broadcast index grids (fast).  The grids are torch tensors because
    mask_mods may call torch.logical_and (attn_script/sparseattn.py:18-19)."""
    import torch
    b = torch.arange(B).reshape(B, 1, 1, 1)
    h = torch.arange(H).reshape(1, H, 1, 1)
    q = torch.arange(Sq).reshape(1, 1, Sq, 1)
    kv = torch.arange(Skv).reshape(1, 1, 1, Skv)
    m = torch.as_tensor(mask_mod(b, h, q, kv)).to(torch.bool)
    return np.broadcast_to(m.numpy(), (B, H, Sq, Skv)).copy()


def _block_counts(mask, bm, bn):
    B, H, Sq, Skv = mask.shape
    nq, nk = -(-Sq // bm), -(-Skv // bn)
    padded = np.zeros((B, H, nq * bm, nk * bn), dtype=np.int64)
    padded[:, :, :Sq, :Skv] = mask
    return padded.reshape(B, H, nq, bm, nk, bn).sum(axis=(3, 5))


def block_any(mask, bm, bn):
    """int8 [B,H,ceil(Sq/bm),ceil(Skv/bn)]: 1 where any element of the block is visible."""
    return (_block_counts(mask, bm, bn) > 0).astype(np.int8)


def block_classes(mask, bm, bn):
    """int8 tile classes: 0 = nothing visible, 1 = partly visible, 2 = every in-range element
    visible."""
    vis = _block_counts(mask, bm, bn)
    tot = _block_counts(np.ones_like(mask), bm, bn)
    return np.where(vis == 0, 0, np.where(vis == tot, 2, 1)).astype(np.int8)


def block_causal_pattern(nq, nk, bm, bn):
    """Block (i, j) of q_idx >= kv_idx is non-empty iff (i+1)*bm > j*bn."""
    i = np.arange(nq).reshape(nq, 1)
    j = np.arange(nk).reshape(1, nk)
    return (i + 1) * bm > j * bn


def no_block_above_diagonal(blocks, bm, bn):
    """True iff every block with (i+1)*bm - 1 < j*bn is empty."""
    nq, nk = blocks.shape[-2:]
    i = np.arange(nq).reshape(nq, 1)
    j = np.arange(nk).reshape(1, nk)
    above = (i + 1) * bm - 1 < j * bn
    return bool(np.all(blocks[..., above] == 0))
