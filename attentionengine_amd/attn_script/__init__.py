"""User-level definitions of the reference's example scripts -- score_mod / mask_mod / OnlineFunc
written the way a user of the API writes them -- shared by the benchmark, the build step and the tests
(attn_script/mha.py:17-84, sigmoidattn.py:10-53, reluattn.py:12-45, gqa_inference.py:22-102,
sparseattn.py:18-19, blocksparseattn.py:18-19, attention_engine/tests/test_blockmask.py:3-10)."""
import math

import torch

from attn_engine import OnlineFunc
from core import CustomIO, SymbolScalar, Var


def causal_mask(b, h, q_idx, kv_idx):
    return q_idx >= kv_idx


def causal_plus_one_mask(b, h, q_idx, kv_idx):
    return q_idx + 1 >= kv_idx


def causal_shifted_mask(b, h, q_idx, kv_idx):
    return q_idx - 128 >= kv_idx


def make_sliding_window_mask(window):
    def sliding_window_mask(b, h, q_idx, kv_idx):
        return torch.logical_and(q_idx >= kv_idx, q_idx < kv_idx + window)
    return sliding_window_mask


def head_dependent_mask(b, h, q_idx, kv_idx):
    # window grows with the head index: exercises b/h inside mask_mod
    return (q_idx >= kv_idx) & (q_idx - kv_idx <= 64 * (h + 1) + 32 * b)


def make_scale_score_mod(scale):
    def score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        return score * scale
    return score_mod


def make_sigmoid_score_mod(scale=None):
    def score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        softmax_bias = custom_fwd_inputs.input_tensors["softmax_bias"]
        if scale is not None:
            score = score * scale
        score = score + softmax_bias
        score = ((score * 0.5).tanh() + 1) * 0.5
        return score
    return score_mod


def make_relu_score_mod(scale):
    def score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        return (score * scale).max(0)
    return score_mod


def make_alibi_score_mod(scale, slope):
    # uses q_idx / kv_idx / h inside score_mod
    def score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        return score * scale - (q_idx - kv_idx).abs() * ((h + 1) * slope)
    return score_mod


class OnlineSoftmax(OnlineFunc):
    def __init__(self):
        online_rowscales = {
            "m": SymbolScalar("m", Var("-inf")),
            "r": SymbolScalar("r", Var("0.0")),
        }
        final_rowscales = {"lse": SymbolScalar("lse", Var("0.0"))}
        super().__init__(online_rowscales, final_rowscales, CustomIO())

    @staticmethod
    def online_fwd(scores, online_rowscales, b, h, q_idx):
        m, r = online_rowscales["m"], online_rowscales["r"]
        m_new = m.max(scores.get_reduce("max"))
        scale_tmp = (m - m_new).exp()
        r = r * scale_tmp
        scores = (scores - m_new).exp()
        r = r + scores.get_reduce("sum")
        return scores, {"m": m_new, "r": r}, scale_tmp

    @staticmethod
    def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
        o_new = o / online_rowscales["r"]
        lse = (online_rowscales["r"]).log() + online_rowscales["m"]
        return o_new, {"lse": lse}

    @staticmethod
    def combine(final_rowscales):
        lse = final_rowscales["lse"]
        lse_max = lse.get_reduce("max")
        row_sum = (lse - lse_max).exp()
        row_sum_sum = row_sum.get_reduce("sum")
        lse_sum = row_sum_sum.log() + lse_max
        return (lse - lse_sum).exp()


class OnlineIdentity(OnlineFunc):
    def __init__(self):
        super().__init__({}, {}, CustomIO())

    @staticmethod
    def online_fwd(scores, online_rowscales, b, h, q_idx):
        return scores, online_rowscales, SymbolScalar("o_scale", Var("1"))

    @staticmethod
    def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
        return o, {}


class OnlineAbsNorm(OnlineFunc):
    """Retention-style normalisation by the running abs-sum (attn_script/retention.py:40-70),
    without its decay-mask input: out = (sum_kv s v) / max(sum_kv |s|, 1)."""

    def __init__(self):
        super().__init__({"r_wo_clamp": SymbolScalar("r_wo_clamp", Var("0.0")),
                          "r": SymbolScalar("r", Var("0.0"))},
                         {"r": SymbolScalar("r", Var("0.0"))}, CustomIO())

    @staticmethod
    def online_fwd(scores, online_rowscales, b, h, q_idx):
        r_wo_clamp, r = online_rowscales["r_wo_clamp"], online_rowscales["r"]
        r_wo_clamp = r_wo_clamp + scores.get_reduce("abssum")
        r_new = r_wo_clamp.max(1.0)
        o_scale = r / r_new
        scores = scores / r_new
        return scores, {"r_wo_clamp": r_wo_clamp, "r": r_new}, o_scale

    @staticmethod
    def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
        return o, {"r": online_rowscales["r"]}


class OnlineRetention(OnlineAbsNorm):
    """attn_script/retention.py:19-70 in full: the abs-sum normalisation above plus the recompute and
    backward rules of its backward pass (the row scale is treated as a constant there, as in the script)."""

    @staticmethod
    def forward(scores, final_rowscales, b, h, q_idx, kv_idx):
        return scores / final_rowscales["r"]

    @staticmethod
    def backward(dp, scores, final_rowscales, doosum_rowscales, b, h, q_idx, kv_idx):
        return dp / final_rowscales["r"]


def retention_score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
    """attn_script/retention.py:14-16: the scores times a decay mask given as a [1,H,S,S] input."""
    return score * custom_fwd_inputs.input_tensors["mask"]


def retention_custom_inputs():
    return CustomIO({"mask": (1, "heads", "seq_len", "seq_len_kv")})


def make_inputs(B, Sq, Skv, Hq, Hkv, D, DV, dtype, seed=0):
    """Seeded inputs generated on the CPU in the order q, k, v (fp32 randn, then rounded to
    ``dtype``) so oracle, CPU baseline and GPU kernel see identical values."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Sq, Hq, D, generator=g, dtype=torch.float32).to(dtype)
    k = torch.randn(B, Skv, Hkv, D, generator=g, dtype=torch.float32).to(dtype)
    v = torch.randn(B, Skv, Hkv, DV, generator=g, dtype=torch.float32).to(dtype)
    return q, k, v
