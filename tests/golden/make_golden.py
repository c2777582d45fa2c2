"""Writes the fixtures in this folder.  Run:  python tests/golden/make_golden.py

The reference's own tests hold no golden vectors (they print differences), so these vectors are
computed here, independently of ``oracle/``, from what the mathematics fixes:

* attention outputs in float64 numpy with explicit per-(batch, head) loops over the textbook
  formulas (softmax / logsumexp / logistic function), never touching the oracle's code, so a
  dropped term, wrong grouping or wrong mask orientation in the oracle shows up as a mismatch;
* block-mask tables typed in by hand from the rule of core/transform/core.py:410-488 applied to
  the three masks of attention_engine/tests/test_blockmask.py:3-10 (B2 H4 S512, 128x64 blocks).

Inputs are not stored: golden_inputs.py derives them from an integer hash of the element index
(values k/64, exact in fp16 and bf16), so the fixtures hold expected outputs only.  C1 keeps every
third query row to stay small.
"""
import os

import numpy as np

from golden_inputs import golden_tensor, qkv

HERE = os.path.dirname(os.path.abspath(__file__))


def _attend(q, k, v, weight_fn, visible):
    """q [B,Sq,Hq,D], k [B,Skv,Hkv,D], v [B,Skv,Hkv,DV]; head h reads kv head h // (Hq/Hkv).
    weight_fn(scores[Sq,Skv], visible[Sq,Skv]) -> (weights, per-row statistic)."""
    B, Sq, Hq, _ = q.shape
    Hkv = k.shape[2]
    out = np.zeros((B, Sq, Hq, v.shape[-1]), np.float64)
    stat = np.zeros((B, Hq, Sq), np.float64)
    for b in range(B):
        for h in range(Hq):
            g = h // (Hq // Hkv)
            s = q[b, :, h].astype(np.float64) @ k[b, :, g].astype(np.float64).T
            w, st = weight_fn(s, visible(b, h))
            out[b, :, h] = w @ v[b, :, g].astype(np.float64)
            stat[b, h] = st
    return out.astype(np.float32), stat.astype(np.float32)


def _softmax(scale):
    def fn(s, vis):
        s = np.where(vis, s * scale, -np.inf)
        m = s.max(-1, keepdims=True)
        e = np.exp(s - m)
        z = e.sum(-1, keepdims=True)
        return e / z, (np.log(z) + m)[:, 0]
    return fn


def _logistic(scale, bias):
    def fn(s, vis):
        w = 1.0 / (1.0 + np.exp(-(s * scale + bias)))
        return np.where(vis, w, 0.0), np.zeros(s.shape[0])
    return fn


def _causal(Sq, Skv):
    vis = np.arange(Sq)[:, None] >= np.arange(Skv)[None, :]
    return lambda b, h: vis


def _all(Sq, Skv):
    vis = np.ones((Sq, Skv), bool)
    return lambda b, h: vis


def main():
    # C1: B1 H4 S512 D64 causal softmax, score * 1/8; rows 0, 3, 6, ... of the output are kept.
    q, k, v = qkv(1, 512, 512, 4, 4, 64, 64, stream=10)
    out, lse = _attend(q, k, v, _softmax(0.125), _causal(512, 512))
    np.savez_compressed(os.path.join(HERE, "c1_softmax_causal.npz"), out_rows=out[:, ::3], lse=lse,
                        row_stride=np.int32(3), scale=np.float32(0.125), stream=np.int32(10))

    # non-causal softmax and a sliding-window mask (window 96), D128
    q, k, v = qkv(1, 256, 256, 2, 2, 128, 128, stream=20)
    out, lse = _attend(q, k, v, _softmax(128 ** -0.5), _all(256, 256))
    i, j = np.arange(256)[:, None], np.arange(256)[None, :]
    win = (i >= j) & (i < j + 96)
    out_w, lse_w = _attend(q, k, v, _softmax(128 ** -0.5), lambda b, h: win)
    np.savez_compressed(os.path.join(HERE, "softmax_full_and_window.npz"), out=out, lse=lse,
                        out_window=out_w, lse_window=lse_w, window=np.int32(96),
                        scale=np.float32(128 ** -0.5), stream=np.int32(20))

    # C3 form: sigmoid(s / sqrt(D) + bias), bias = -ln(Skv), non-causal and causal
    q, k, v = qkv(1, 256, 256, 2, 2, 128, 128, stream=30)
    bias = -np.log(256.0)
    out, _ = _attend(q, k, v, _logistic(128 ** -0.5, bias), _all(256, 256))
    out_c, _ = _attend(q, k, v, _logistic(128 ** -0.5, bias), _causal(256, 256))
    np.savez_compressed(os.path.join(HERE, "sigmoid.npz"), out=out, out_causal=out_c, bias=np.float32(bias),
                        scale=np.float32(128 ** -0.5), stream=np.int32(30))

    # C4 form: GQA decode, one query token, Hq 32 over Hkv 8, ragged Skv (not a multiple of any tile)
    q, k, v = qkv(2, 1, 1000, 32, 8, 128, 128, stream=40)
    out, lse = _attend(q, k, v, _softmax(128 ** -0.5), _all(1, 1000))
    np.savez_compressed(os.path.join(HERE, "gqa_decode.npz"), out=out, lse=lse, scale=np.float32(128 ** -0.5),
                        stream=np.int32(40))

    # C5 form: MLA decode, keys = latent(512) || rope(64), values = latent; scale 1/sqrt(192)
    B, H, Skv = 2, 128, 300
    qn, qr = golden_tensor((B, 1, H, 512), 50), golden_tensor((B, 1, H, 64), 51)
    kv, kr = golden_tensor((B, Skv, 1, 512), 52), golden_tensor((B, Skv, 1, 64), 53)
    out, lse = _attend(np.concatenate([qn, qr], -1), np.concatenate([kv, kr], -1), kv,
                       _softmax(192 ** -0.5), _all(1, Skv))
    np.savez_compressed(os.path.join(HERE, "mla_decode.npz"), out=out, lse=lse, scale=np.float32(192 ** -0.5),
                        stream=np.int32(50))

    # Block-mask known answers, typed by hand: for each mask, per q-block row (4 rows of 128) the
    # number of leading visible kv blocks (8 columns of 64); block (i, j) is set iff any element
    # of it is visible.  q_idx >= kv_idx: row i sees kv < 128(i+1)       -> 2(i+1) blocks.
    # q_idx + 1 >= kv_idx: row i also sees kv = 128(i+1)                  -> 2(i+1)+1, capped at 8.
    # q_idx - 128 >= kv_idx: row i sees kv <= 128 i - 1                    -> 2 i blocks.
    lead = {"causal": [2, 4, 6, 8], "causal_plus_one": [3, 5, 7, 8], "causal_shifted_128": [0, 2, 4, 6]}
    tables = {}
    for name, counts in lead.items():
        t = np.zeros((2, 4, 4, 8), np.int8)
        for i, c in enumerate(counts):
            t[:, :, i, :c] = 1
        tables[name] = t
    np.savez_compressed(os.path.join(HERE, "blockmask_kat.npz"),
                        is_causal=np.array([True, False, False]), is_less_causal=np.array([True, False, True]),
                        names=np.array(list(lead)), **tables)


if __name__ == "__main__":
    main()
