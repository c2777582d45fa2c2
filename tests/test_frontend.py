"""CPU tests of the host side: symbolic tracer, mask utilities (product code vs the oracle's brute
force), mask_mod lowering, functor emission + hipRTC compilation (no GPU needed), engine dispatch
and error behaviour."""
import math

import numpy as np
import pytest
import torch

import attn_cases as C
from attn_engine import AttentionEngine, OnlineFunc
from core import CustomIO, SymbolicArray, SymbolScalar, Var, create_block_mask, create_mask, meta_tensor
from core.lower import lower as L
from core.lower.lower_decode import lower_combine
from core.lower.mask import lower_mask_mod, plan_mask
from core.transform.core import (SymbolicConst, create_block_idx, is_causal_mask, is_less_causal_mask)
from oracle import masks as M


# ---- tracer ---------------------------------------------------------------------------------------
def test_tracer_builds_the_softmax_graph():
    """Node sequence of OnlineSoftmax.online_fwd as traced from attn_script/mha.py:47-63."""
    on = C.OnlineSoftmax()
    scores = SymbolicArray("scores", Var("scores"), shape_idx=["block_M", "block_N"])
    b = h = q = SymbolScalar("b", Var("b"))
    s2, rows, o_scale = on.online_fwd(scores, on.online_rowscales, b, h, q)
    assert s2.code.type == "Exp" and s2.prev[0].code.type == "Sub"
    assert s2.shape_idx == ["block_M", "block_N"]
    m_new = rows["m"]
    assert m_new.code.type == "Max" and m_new.prev[1].code.type == "ReduceMax"
    assert m_new.prev[1].shape_idx == ["block_M"] and m_new.prev[1].varname == "scores_max_0"
    assert rows["r"].code.type == "Add" and rows["r"].prev[1].code.type == "ReduceSum"
    assert o_scale.code.type == "Exp" and o_scale.prev[0].prev[1] is m_new
    # naming rule <varname>[_<suffix>]_<use count>
    assert m_new.varname == "m_0"


def test_python_numbers_become_constants_on_either_side():
    x = SymbolScalar("x", Var("x"))
    y = (x * 2 + 1.5) / 3
    assert y.code.type == "Div" and isinstance(y.prev[1], SymbolicConst) and y.prev[1].code.value == 3
    z = 1 - x
    assert z.code.type == "Sub" and z.prev[0].code.type == "Const" and z.prev[1] is x
    with pytest.raises(TypeError):
        x + "a"


def test_customio_declares_symbolic_tensors():
    io = CustomIO({"softmax_bias": (1,), "slopes": ("heads",)})
    assert io.input_tensors["softmax_bias"].shape_idx == ["1"]
    assert io.input_tensors["slopes"].shape_idx == ["heads"]


# ---- masks (product) vs brute force (oracle) --------------------------------------------------------
@pytest.mark.parametrize("mask_mod", [C.causal_mask, C.causal_plus_one_mask, C.causal_shifted_mask,
                                      C.make_sliding_window_mask(100), C.head_dependent_mask])
def test_create_mask_and_block_mask_match_brute_force(mask_mod):
    B, H, S = 2, 4, 512
    dense = create_mask(mask_mod, B, H, S, S, device="cpu")
    ref = M.dense_mask_grid(mask_mod, B, H, S, S)
    assert dense.dtype == torch.bool and np.array_equal(dense.numpy(), ref)
    blocks = create_block_mask(mask_mod, B, H, S, S, "cpu", 128, 64)
    assert blocks.dtype == torch.int8 and np.array_equal(blocks.numpy(), M.block_any(ref, 128, 64))
    assert bool(is_causal_mask(blocks, 128, 64)) == bool(
        np.array_equal(np.broadcast_to(M.block_causal_pattern(4, 8, 128, 64), blocks.shape), blocks.numpy().astype(bool)))
    assert bool(is_less_causal_mask(blocks, 128, 64)) == M.no_block_above_diagonal(blocks.numpy(), 128, 64)
    idx = create_block_idx(mask_mod, B, H, S, S, "cpu", 128, 64)
    assert idx.shape == (int(blocks.sum()), 4)


def test_block_mask_known_answers_of_the_reference_test_script():
    """attention_engine/tests/test_blockmask.py:3-27 prints these; values hand-derived."""
    for mask_mod, last, causal, less in [(C.causal_mask, [1, 3, 5, 7], True, True),
                                         (C.causal_plus_one_mask, [2, 4, 6, 7], False, False),
                                         (C.causal_shifted_mask, [-1, 1, 3, 5], False, True)]:
        blocks = create_block_mask(mask_mod, 2, 4, 512, 512, "cpu", 128, 64)
        for i, l in enumerate(last):
            assert blocks[0, 0, i].tolist() == [1] * (l + 1) + [0] * (7 - l)
        assert bool(is_causal_mask(blocks, 128, 64)) == causal
        assert bool(is_less_causal_mask(blocks, 128, 64)) == less


def test_ragged_block_mask_pads_with_invisible():
    blocks = create_block_mask(C.causal_mask, 1, 1, 200, 200, "cpu", 128, 64)
    assert blocks.shape == (1, 1, 2, 4)
    assert blocks[0, 0].tolist() == [[1, 1, 0, 0], [1, 1, 1, 1]]


def test_mask_plan_classes_match_oracle():
    for mask_mod in (C.causal_plus_one_mask, C.make_sliding_window_mask(100), C.head_dependent_mask):
        lm = lower_mask_mod(mask_mod)
        plan = plan_mask(mask_mod, lm, 2, 4, 300, 300, 128, 64, chunk_rows=128)
        assert plan.mode == 2
        mb, mh = (2 if lm.uses_b else 1), (4 if lm.uses_h else 1)
        ref = M.block_classes(M.dense_mask_grid(mask_mod, mb, mh, 300, 300), 128, 64)
        assert np.array_equal(plan.table.numpy(), ref)
    lm = lower_mask_mod(C.causal_mask)
    assert plan_mask(C.causal_mask, lm, 2, 4, 300, 300, 128, 64).mode == 1
    assert not lm.uses_b and not lm.uses_h
    assert lower_mask_mod(C.head_dependent_mask).uses_h


def test_mask_mod_lowering_text_and_unsupported_ops():
    lm = lower_mask_mod(C.make_sliding_window_mask(256))
    assert "n_ge" in lm.body and "(bool)(n_ge) & (bool)(n_lt)" in lm.body and "return (bool)" in lm.body

    def bad(b, h, q_idx, kv_idx):
        return torch.sin(q_idx) > kv_idx
    with pytest.raises(NotImplementedError):
        lower_mask_mod(bad)


# ---- functor emission -----------------------------------------------------------------------------
def test_emitted_softmax_functors():
    lf = L.trace_functors(C.make_scale_score_mod(0.125), C.causal_mask, C.OnlineSoftmax(), CustomIO({}),
                          torch.float16)
    assert lf.rowstate_fields == ["m", "r"] and lf.rowstate_init == ["-1e38f", "0.0f"]
    assert lf.final_rowscale_names == ["lse"] and not lf.o_scale_one
    body = lf.online_fwd_body
    assert "ae_row_sum<N>" in body
    # affine folding: the score scale is applied to the row maximum (one multiply per row) and
    # folded with log2(e) into the exponent, one fma + exp2 per element, no separate scaling pass
    assert "ae_row_max<N>(s) * 0.125f" in body
    assert f"ae_exp2(__builtin_fmaf(s[e], {0.125 * 1.4426950408889634!r}f" in body
    assert "s[e] * 0.125f" not in body
    # the graph is recognised as the online softmax: thresholded (lazy) running maximum
    assert "> 5.545177444479562f) ?" in body and "ae_max(st.m" not in body
    assert "frs[0]" in lf.epilogue_body and "ae_log(st.r)" in lf.epilogue_body
    src = L.render_functors(lf)
    for name in ("ae_score_mod", "ae_online_fwd", "ae_epilogue", "ae_mask_mod", "ae_rowstate_init"):
        assert name in src


def test_emitted_identity_and_custom_scalar():
    lf = L.trace_functors(C.make_sigmoid_score_mod(0.1), None, C.OnlineIdentity(),
                          CustomIO({"softmax_bias": (1,)}), torch.float16)
    assert lf.o_scale_one and lf.rowstate_fields == [] and lf.final_rowscale_names == []
    assert lf.customs[0].name == "softmax_bias" and lf.customs[0].torch_dtype == torch.float32
    # ((x*0.5).tanh() + 1) * 0.5 is the logistic function: one exp2 and one reciprocal per score
    assert "ae_rcp(1.0f + ae_exp2(__builtin_fmaf(s[e], -0.14426950" in lf.online_fwd_body
    assert "ae_tanh" not in lf.online_fwd_body and "cust.softmax_bias" in lf.online_fwd_body


def test_affine_of_tanh_forms():
    """a*tanh(x)+b with literal constants: the logistic special case, the general case, and a bare
    tanh (sigmoid script form attn_script/sigmoidattn.py:14-18; tanh semantics tl_gen.py:113-117)."""
    def lower(f):
        return L.trace_functors(f, None, C.OnlineIdentity(), CustomIO({}), torch.float16).online_fwd_body
    gen = lower(lambda s, c, b, h, q, kv: 3.0 - (s * 0.25).tanh() * 2.0)           # a = -2, b = 3
    assert "__builtin_fmaf(ae_rcp(ae_exp2(s[e] * 0.72134752" in gen and ", 4.0f, 1.0f)" in gen
    bare = lower(lambda s, c, b, h, q, kv: (s * 0.25).tanh())
    assert "ae_tanh" in bare
    # the rewritten forms agree with the definition
    import math
    for x in (-30.0, -2.0, -0.1, 0.0, 0.3, 5.0, 40.0):
        e = 2.0 ** (2 * 0.25 * x * 1.4426950408889634)
        assert abs((1.0 / (e + 1.0)) * 4.0 + 1.0 - (3.0 - 2.0 * math.tanh(0.25 * x))) < 1e-12
        assert abs(1.0 / (1.0 + 2.0 ** (-x * 1.4426950408889634)) - 0.5 * (math.tanh(0.5 * x) + 1)) < 1e-12


def test_unsupported_graphs_raise():
    class Bad(OnlineFunc):
        def __init__(self):
            super().__init__({"m": SymbolScalar("m", Var("banana"))}, {}, CustomIO())
    with pytest.raises(NotImplementedError):
        L.trace_functors(None, None, Bad(), CustomIO({}), torch.float16)
    with pytest.raises(NotImplementedError):   # an unknown dimension name in a custom input's shape
        L.trace_functors(lambda s, c, b, h, q, kv: s * c.input_tensors["x"], None, C.OnlineIdentity(),
                         CustomIO({"x": (1, "channels")}), torch.float16)


def test_custom_input_with_a_kv_dimension_is_read_per_score():
    """The retention decay mask (attn_script/retention.py:14-16, lower.py:590-597 of the reference):
    a [1,H,S,S] input is indexed by the lane's row once and by kv position inside the tile loop."""
    lf = L.trace_functors(C.retention_score_mod, C.causal_mask, C.OnlineAbsNorm(), C.retention_custom_inputs(),
                          torch.float16, mask_value="0")
    text = L.render_functors(lf)
    assert lf.customs[0].per_kv and lf.customs[0].torch_dtype == torch.float16
    assert "const ae_elem* mask_row;" in text and "p.custom[0]" in text
    assert "(int64_t)(ctx.h) * (1 * (int64_t)p.seqlen_kv * (int64_t)p.seqlen_q)" in text   # [1, heads, seq_len, seq_len_kv]
    assert "*(const ae_elem4*)src" in text and "ctx.kv_base + ae_kv_off(4 * g)" in text
    assert "(s[e] * cm_mask[e])" in text and "ae_row_abssum<N>" in text
    with pytest.raises(NotImplementedError):   # ... but not in the epilogue, which has no kv position
        class Epi(C.OnlineIdentity):
            @staticmethod
            def online_fwd_epilogue(o, rs, b, h, q_idx):
                return o, {}
        bad = Epi()
        cio = C.retention_custom_inputs()
        bad.online_fwd_epilogue = staticmethod(lambda o, rs, b, h, q_idx: (o * cio.input_tensors["mask"], {}))
        L.trace_functors(None, None, bad, cio, torch.float16)


def test_combine_lowering_finds_the_merged_lse():
    text = lower_combine(C.OnlineSoftmax(), ["lse"])
    assert "ae_arr_max<AE_NSPLIT>(rs[0])" in text and "ae_arr_sum<AE_NSPLIT>" in text
    assert "merged[0] = cb" in text and "nanf" not in text
    text = lower_combine(C.OnlineIdentity(), [])
    assert "w[e] = 1.0f" in text


# ---- engine construction compiles through hipRTC without a GPU ---------------------------------------
def _meta(B, Hq, Hkv, Sq, Skv, D, DV, dt):
    return (meta_tensor(B, Hq, Sq, D, dtype=dt), meta_tensor(B, Hkv, Skv, D, dtype=dt),
            meta_tensor(B, Hkv, Skv, DV, dtype=dt))


def test_engine_dispatch_and_compile_on_cpu():
    from core.lower.lower_decode import GQADecodeOp, MLADecodeOp
    from core.lower.prefill_op import PrefillOp
    sm = C.make_scale_score_mod(0.1)
    pre = AttentionEngine(_meta(1, 2, 2, 256, 256, 64, 64, torch.float16), CustomIO({}), sm, C.causal_mask,
                          C.OnlineSoftmax())
    assert isinstance(pre._op, PrefillOp) and "#define AE_MASK_MODE 1" in pre.tl_code
    assert pre.block_mask is None     # exactly block-causal -> dense template in the reference
    win = AttentionEngine(_meta(1, 2, 2, 512, 512, 64, 64, torch.bfloat16), CustomIO({}), sm,
                          C.make_sliding_window_mask(128), C.OnlineSoftmax())
    assert "#define AE_MASK_MODE 2" in win.tl_code and "#define AE_DTYPE_BF16 1" in win.tl_code
    assert win.block_mask.shape == (1, 2, 4, 4) and win.block_mask.dtype == torch.int8
    dec = AttentionEngine(_meta(2, 32, 8, 1, 1024, 128, 128, torch.float16), CustomIO({}), sm, None,
                          C.OnlineSoftmax())
    assert isinstance(dec._op, GQADecodeOp) and "ae_combine" in dec.tl_code
    mla = AttentionEngine(_meta(2, 128, 1, 1, 512, 576, 512, torch.bfloat16), CustomIO({}), sm, None,
                          C.OnlineSoftmax(), kv_shared=True)
    assert isinstance(mla._op, MLADecodeOp)
    gqa = AttentionEngine(_meta(1, 8, 2, 256, 256, 64, 64, torch.float16), CustomIO({}), sm, C.causal_mask,
                          C.OnlineSoftmax())
    assert isinstance(gqa._op, PrefillOp)
    # MHA decode (attn_script/mha_inference.py): a few query tokens against a long KV -> split-KV prefill
    mhad = AttentionEngine(_meta(1, 32, 32, 128, 8192, 128, 128, torch.float16), CustomIO({}), sm, None,
                           C.OnlineSoftmax())
    assert isinstance(mhad._op, PrefillOp) and mhad._op.split_kv
    assert mhad._op.plan_splits(1, 32, 128, 8192) == (8, 1024)
    assert mhad._op.plan_splits(2, 4, 5, 1000) == (16, 64)       # never an empty split, whole tiles
    assert "#define AE_NSPLIT 8" in mhad.tl_code and "ae_combine" in mhad.tl_code
    # tuner / backend arguments of the reference scripts are accepted
    AttentionEngine(_meta(1, 2, 2, 128, 128, 64, 64, torch.float16), CustomIO({}), sm, C.causal_mask,
                    C.OnlineSoftmax(), tune=True, tune_file="x.json", tune_bwd=True, backend="cute")
    # identity online function may be None (reference CuTe scripts)
    AttentionEngine(_meta(1, 2, 2, 128, 128, 64, 64, torch.float16), CustomIO({}), C.make_relu_score_mod(0.1),
                    None, None)


def test_engine_error_behaviour():
    sm = C.make_scale_score_mod(0.1)
    with pytest.raises(KeyError):       # unsupported dtype, as attn_engine.py:225-228 / 304
        AttentionEngine(_meta(1, 2, 2, 128, 128, 64, 64, torch.float32), CustomIO({}), sm, None, C.OnlineSoftmax())
    with pytest.raises(AssertionError):  # decode asserts q_len == 1 (attn_engine.py:255)
        AttentionEngine(_meta(1, 8, 2, 4, 1024, 64, 64, torch.float16), CustomIO({}), sm, None, C.OnlineSoftmax())
    # an online function without combine() cannot merge KV splits: the same shape runs unsplit
    unsplit = AttentionEngine(_meta(1, 2, 2, 128, 1024, 64, 64, torch.float16), CustomIO({}), sm, None,
                              C.OnlineIdentity())
    assert not unsplit._op.split_kv and unsplit._op.plan_splits(1, 2, 128, 1024) == (1, 1024)
    with pytest.raises(ValueError):
        AttentionEngine(_meta(1, 2, 2, 128, 128, 64, 64, torch.float16), CustomIO({}), sm, None,
                        C.OnlineSoftmax(), backend="triton")
    mod = AttentionEngine(_meta(1, 2, 2, 128, 128, 64, 64, torch.float16), CustomIO({}), sm, None, C.OnlineSoftmax())
    q = torch.zeros(1, 128, 2, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="no CPU path"):   # the product never falls back to the CPU
        mod(q, q, q)


def test_lazy_maximum_only_for_the_online_softmax():
    """The thresholded running maximum is applied only when the traced graph is provably the online
    softmax; a function that exports m itself keeps the exact update."""
    from attn_engine import OnlineFunc

    class SoftmaxExportingMax(C.OnlineSoftmax):
        @staticmethod
        def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
            o_new = o / online_rowscales["r"]
            return o_new, {"m": online_rowscales["m"] + 0.0}
    lf = L.trace_functors(C.make_scale_score_mod(0.125), None, SoftmaxExportingMax(), CustomIO({}), torch.float16)
    assert "ae_max(st.m" in lf.online_fwd_body and "5.545" not in lf.online_fwd_body
    lf = L.trace_functors(C.make_scale_score_mod(0.125), None, C.OnlineAbsNorm(), CustomIO({}), torch.float16)
    assert "5.545" not in lf.online_fwd_body


def test_softmax_specialisation_needs_the_exact_graph():
    """Kernels that hard-code exp(c*S - m) (pipelined prefill, wave-specialised MLA decode, the softmax
    backward) may only be chosen for the online softmax OF the modified scores.  Near misses -- another
    function of the scores inside exp, another quantity inside the running maximum, other initial
    values -- stay reference-point invariant (lazy maximum allowed) but must run the generated functor."""
    from attn_engine import OnlineFunc
    sm = C.make_scale_score_mod(0.125)
    assert L.trace_functors(sm, None, C.OnlineSoftmax(), CustomIO({}), torch.float16).softmax == (0.125, "m", "r")

    class TwiceInsideExp(C.OnlineSoftmax):
        @staticmethod
        def online_fwd(scores, online_rowscales, b, h, q_idx):
            m, r = online_rowscales["m"], online_rowscales["r"]
            m_new = m.max(scores.get_reduce("max"))
            scale_tmp = (m - m_new).exp()
            p = (scores * 2.0 - m_new).exp()
            return p, {"m": m_new, "r": r * scale_tmp + p.get_reduce("sum")}, scale_tmp

    class AbsInsideMax(C.OnlineSoftmax):
        @staticmethod
        def online_fwd(scores, online_rowscales, b, h, q_idx):
            m, r = online_rowscales["m"], online_rowscales["r"]
            m_new = m.max(scores.abs().get_reduce("max"))
            scale_tmp = (m - m_new).exp()
            p = (scores - m_new).exp()
            return p, {"m": m_new, "r": r * scale_tmp + p.get_reduce("sum")}, scale_tmp

    class StartsAtZero(C.OnlineSoftmax):
        def __init__(self):
            OnlineFunc.__init__(self, {"m": SymbolScalar("m", Var("0.0")), "r": SymbolScalar("r", Var("0.0"))},
                                {"lse": SymbolScalar("lse", Var("0.0"))}, CustomIO())

    for near_miss in (TwiceInsideExp(), AbsInsideMax(), StartsAtZero()):
        lf = L.trace_functors(sm, None, near_miss, CustomIO({}), torch.float16)
        assert lf.softmax is None, type(near_miss).__name__
        # ... and the generic kernel is what the engine then compiles, even on chip-filling shapes
        tiles = L.choose_prefill_tiles(128, 128, seqlen_q=4096, softmax=lf.softmax, batch_heads=64)
        assert tiles.template == "ae_prefill.hip"
    src = L.render_functors(L.trace_functors(sm, None, TwiceInsideExp(), CustomIO({}), torch.float16))
    assert "0.3606737" in src                    # the functor carries the user's factor: 0.125 * 2 * log2(e)
    # no backward is derived for them either: the softmax gradient is only valid for the exact graph
    from core.lower.prefill_bwd_op import PrefillBwdOp
    from core.lower.prefill_op import PrefillOp
    for near_miss in (TwiceInsideExp(), AbsInsideMax()):
        op = PrefillOp(_meta(1, 2, 2, 256, 256, 64, 64, torch.float16), CustomIO({}), sm, None, near_miss, "-inf")
        with pytest.raises(NotImplementedError):
            PrefillBwdOp(op, sm, near_miss, CustomIO({}))


def test_softmax_proof_takes_the_guarded_division_of_the_sparse_attention_script():
    """attn_script/sparseattn.py:66-72 divides by r + 1e-30.  A row with a visible key has r >= 1 whatever the lagging
    reference, so a constant of at most 1e-20 leaves r unchanged in fp32 and the graph is still the online softmax;
    a constant that can change r (or anything else in the denominator) is not."""
    sm = C.make_scale_score_mod(0.125)

    def guarded(c, wrong_side=False):
        class Guarded(C.OnlineSoftmax):
            @staticmethod
            def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
                r = online_rowscales["r"]
                den = (c + r) if wrong_side else (r + c)
                return o / den, {"lse": r.log() + online_rowscales["m"]}
        return Guarded()
    for c in (1e-30, 1e-20, 0.0):
        assert L.trace_functors(sm, None, guarded(c), CustomIO({}), torch.float16).softmax == (0.125, "m", "r"), c
    assert L.trace_functors(sm, None, guarded(1e-30, wrong_side=True), CustomIO({}), torch.float16).softmax is not None
    for c in (1e-6, 1.0, -1e-30):
        lf = L.trace_functors(sm, None, guarded(c), CustomIO({}), torch.float16)
        assert lf.softmax is None and "5.545" not in lf.online_fwd_body, c      # neither specialised nor lazy
    src = L.render_functors(L.trace_functors(sm, None, guarded(1e-30), CustomIO({}), torch.float16))
    assert "1e-30" in src or "1.0e-30" in src or "9.99999" in src        # the user's epilogue runs as written


def test_shapes_broadcast_by_name():
    q = SymbolScalar("q_idx", Var("q_idx"), shape_idx=["block_M"])
    kv = SymbolScalar("kv_idx", Var("kv_idx"), shape_idx=["block_N"])
    assert (q - kv).shape_idx == ["block_M", "block_N"]
    assert (kv - q).shape_idx == ["block_M", "block_N"]
    s = SymbolicArray("s", Var("s"), shape_idx=["block_M", "block_N"])
    assert (s - q).shape_idx == ["block_M", "block_N"] and (q * 2).shape_idx == ["block_M"]
    assert s.get_reduce("max").shape_idx == ["block_M"]


def test_symbolic_derivative_matches_autograd():
    """core.transform.autodiff.derivative on traced elementwise graphs (every node type the tracer has),
    evaluated by the oracle's graph interpreter, against torch.autograd of the same function."""
    from core.transform.autodiff import derivative
    from oracle.online_interp import evaluate
    x = torch.linspace(-2.3, 2.7, 41, dtype=torch.float64)
    cases = [
        (lambda s: ((s * 0.125 + 0.3) * 0.5).tanh() * 0.5 + 0.5, lambda t: torch.sigmoid(t * 0.125 + 0.3)),
        (lambda s: (s * 0.7).max(0), lambda t: torch.relu(t * 0.7)),
        (lambda s: (s * s + 1.5).log() / (s.exp() + 2.0), lambda t: torch.log(t * t + 1.5) / (torch.exp(t) + 2.0)),
        (lambda s: (s * 0.4).exp2() - (s * s + 1.0).log2() - s.abs() * 0.25 + (-s) * 0.1,
         lambda t: torch.exp2(t * 0.4) - torch.log2(t * t + 1.0) - t.abs() * 0.25 - t * 0.1),
        (lambda s: 3.0 / (s * s + 1.0) + (2.0 - s) * s, lambda t: 3.0 / (t * t + 1.0) + (2.0 - t) * t),
    ]
    for traced_fn, torch_fn in cases:
        s = SymbolScalar("scores", Var("scores"), shape_idx=[])
        y = traced_fn(s)
        dy = derivative(y, s)
        got = evaluate(dy, {id(s): x})
        t = x.clone().requires_grad_(True)
        (want,) = torch.autograd.grad(torch_fn(t).sum(), t)
        got = got if isinstance(got, torch.Tensor) else torch.full_like(x, float(got))
        assert torch.allclose(got.expand_as(want), want, atol=1e-12, rtol=1e-10)
    # no dependence -> zero
    s, c = SymbolScalar("scores", Var("scores"), shape_idx=[]), SymbolScalar("c", Var("c"), shape_idx=[])
    assert float(evaluate(derivative(c * 2.0, s), {id(c): 1.0})) == 0.0


def test_elementwise_backward_lowering():
    """The backward functors of sigmoid / relu attention are emitted; online functions that keep row
    scales, non-scalar custom inputs and non-identity forward/backward rules are refused."""
    from core.lower.prefill_bwd_op import lower_elementwise_backward
    src = lower_elementwise_backward(C.make_sigmoid_score_mod(0.125), C.OnlineIdentity(),
                                     CustomIO({"softmax_bias": (1,)}), torch.float16)
    assert "ae_bwd_pd" in src and "cust.softmax_bias" in src and "p.custom[0]" in src
    src = lower_elementwise_backward(C.make_relu_score_mod(0.125), C.OnlineIdentity(), CustomIO({}), torch.float16)
    assert "> 0.0f ?" in src
    with pytest.raises(NotImplementedError):
        lower_elementwise_backward(C.make_scale_score_mod(0.125), C.OnlineAbsNorm(), CustomIO({}), torch.float16)
    with pytest.raises(NotImplementedError):
        lower_elementwise_backward(C.retention_score_mod, C.OnlineIdentity(), C.retention_custom_inputs(),
                                   torch.float16)


def test_inferred_block_mask_granularity_does_not_reach_the_kernel():
    """infer_mask_block_M/N only shape the block mask kept on mod.block_mask (lower.py:721-738 of the
    reference); the kernel classifies its own tiles from mask_mod, so a granularity that no kv tile fits
    (96 keys against 64-key tiles) is harmless, and handing the engine such a mask from outside is refused
    instead of skipping visible keys."""
    from core.lower.prefill_op import PrefillOp
    op = PrefillOp(_meta(1, 2, 2, 384, 384, 64, 64, torch.float16), CustomIO({}), C.make_scale_score_mod(0.125),
                   C.make_sliding_window_mask(100), C.OnlineSoftmax(), "-inf", infer_mask=True,
                   infer_mask_block_M=128, infer_mask_block_N=96)
    assert op.block_mask is not None and op.block_mask.shape == (1, 2, 3, 4)
    plan = op._plan(1, 2, 384, 384, device=None)
    assert (plan.block_m, plan.block_n) == (op.tiles.block_m, op.tiles.block_n)


def test_traced_backward_of_an_online_function_with_its_own_row_scale():
    """attn_script/retention.py: OnlineFunc.forward / backward are traced into ae_bwd_pd2 together with the
    derivative of score_mod (the decay mask, read per score); an online function that keeps row scales
    without defining them gets no backward."""
    from core.lower.prefill_bwd_op import lower_traced_backward
    src, names = lower_traced_backward(C.retention_score_mod, C.OnlineRetention(), C.retention_custom_inputs(),
                                       torch.float16)
    assert names == ["r"] and "ae_bwd_pd2" in src
    assert "p.custom[0]" in src and "p.seqlen_kv" in src          # the mask element of (head, q, kv)
    body = src.split("ae_bwd_pd2", 2)[-1]
    assert "const float (&rs)[1]" in body and "rs[0]" in body and "cv_mask" in body and "dp" in body
    with pytest.raises(NotImplementedError, match="forward"):
        lower_traced_backward(C.retention_score_mod, C.OnlineAbsNorm(), C.retention_custom_inputs(), torch.float16)


def test_traced_backward_reads_every_final_row_scale():
    """An online function with two final row scales whose forward() / backward() read both (the reference hands
    every final row scale to them, core/lower/lower.py:413-453): both arrive in the functor, in declaration order."""
    from core.lower.prefill_bwd_op import lower_traced_backward

    class TwoScales(C.OnlineSoftmax):
        def __init__(self):
            super().__init__()
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
    src, names = lower_traced_backward(C.make_scale_score_mod(0.125), TwoScales(), CustomIO({}), torch.float16)
    assert names == ["m", "r"]
    body = src.split("ae_bwd_pd2", 2)[-1]
    assert "const float (&rs)[2]" in body and "rs[0]" in body and "rs[1]" in body and "doosum" in body
    lf = L.trace_functors(C.make_scale_score_mod(0.125), None, TwoScales(), CustomIO({}), torch.float16)
    assert lf.softmax is None and lf.final_rowscale_names == ["m", "r"]     # not the graph with the fixed backward


def test_symbol_backward_leaves_gradient_expressions_on_the_leaves():
    """SymbolScalar.backward (core/transform/core.py:119-199 of the reference): after
    ``f(x, y).backward(g)`` the leaves carry g * df/dx and g * df/dy as traced expressions; evaluated by the
    oracle's graph interpreter against torch.autograd."""
    from oracle.online_interp import evaluate
    x = SymbolScalar("x", Var("x"), shape_idx=[])
    y = SymbolScalar("y", Var("y"), shape_idx=[])
    g = SymbolScalar("g", Var("g"), shape_idx=[])
    f = (x * y + x.exp()) / (y * y + 2.0) - (x * 0.5).tanh()
    f.backward(g)
    assert x.grad is not None and y.grad is not None
    xv = torch.linspace(-1.5, 1.2, 17, dtype=torch.float64).requires_grad_(True)
    yv = torch.linspace(0.3, 2.1, 17, dtype=torch.float64).requires_grad_(True)
    gv = torch.linspace(-0.7, 0.9, 17, dtype=torch.float64)
    ref = (xv * yv + xv.exp()) / (yv * yv + 2.0) - (xv * 0.5).tanh()
    gx, gy = torch.autograd.grad(ref, (xv, yv), gv)
    env = {id(x): xv.detach(), id(y): yv.detach(), id(g): gv}
    assert torch.allclose(evaluate(x.grad, env), gx, atol=1e-12)
    assert torch.allclose(evaluate(y.grad, env), gy, atol=1e-12)


def test_elementwise_graphs_are_recognised():
    """out = sum_kv f(s) v (no row state, no reduction over the tile, no kv index): the functor may be applied
    to any subset of a tile, which is what lets the software-pipelined kernel call it pairwise."""
    import attn_script as C
    from core.lower import lower as L
    f16 = torch.float16
    sig = L.trace_functors(C.make_sigmoid_score_mod(0.125), None, C.OnlineIdentity(),
                           CustomIO({"softmax_bias": (1,)}), f16)
    relu = L.trace_functors(C.make_relu_score_mod(0.125), C.causal_mask, C.OnlineIdentity(), CustomIO({}), f16)
    soft = L.trace_functors(C.make_scale_score_mod(0.125), None, C.OnlineSoftmax(), CustomIO({}), f16)
    assert sig.elementwise and relu.elementwise and not soft.elementwise
    assert sig.softmax is None and soft.softmax is not None

    def uses_kv(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        return score * 0.125 + kv_idx
    assert not L.trace_functors(uses_kv, None, C.OnlineIdentity(), CustomIO({}), f16).elementwise

    class TileNormalised(C.OnlineIdentity):      # no row state, but a reduction over the tile
        @staticmethod
        def online_fwd(scores, online_rowscales, b, h, q_idx):
            return scores / scores.get_reduce("abssum"), online_rowscales, C.OnlineIdentity.online_fwd(
                scores, online_rowscales, b, h, q_idx)[2]
    try:
        lf = L.trace_functors(C.make_scale_score_mod(0.125), None, TileNormalised(), CustomIO({}), f16)
    except Exception:
        lf = None
    assert lf is None or not lf.elementwise
    # tile choice: a chip-filling elementwise problem takes the pipelined kernel, a small one the generic one
    big = L.choose_prefill_tiles(128, 128, seqlen_q=4096, softmax=None, batch_heads=64, elementwise=True)
    small = L.choose_prefill_tiles(128, 128, seqlen_q=512, softmax=None, batch_heads=4, elementwise=True)
    assert big.template == "ae_prefill_pipe.hip" and small.template == "ae_prefill.hip"
    cfg = L.render_config(128, 128, f16, big, 0, False, 0, True, True, True, None, elementwise=True)
    assert "#define AE_PIPE_KIND 1" in cfg


def test_per_tile_renormalisation_is_deferred_to_the_epilogue(monkeypatch):
    """scores / r_new with o_scale = r_old / r_new (retention's running sum of |s|): the factors telescope, so
    the lowering accumulates unscaled and divides once by the final row scale - no rescale of the accumulator
    per tile.  The row state and the final row scale are untouched; graphs of another form are left alone."""
    import attn_script as C
    from core.lower import lower as L
    f16 = torch.float16
    lf = L.trace_functors(C.retention_score_mod, C.causal_mask, C.OnlineRetention(), C.retention_custom_inputs(),
                          f16, "0")
    assert lf.deferred_norm == "r" and lf.o_scale_one
    src = L.render_functors(lf)
    fwd = src[src.index("AE_DEV float ae_online_fwd"):src.index("AE_DEV void ae_epilogue")]
    assert " / " not in fwd.split("#endif")[-1] and "const float ae_o_scale = 1.0f;" in fwd
    epi = src[src.index("AE_DEV void ae_epilogue"):]
    assert "1.0f / st.r" in epi and "frs[0] = st.r;" in epi
    assert L.trace_functors(C.make_scale_score_mod(0.125), None, C.OnlineSoftmax(), CustomIO({}), f16).deferred_norm is None
    assert L.trace_functors(C.make_relu_score_mod(0.125), None, C.OnlineIdentity(), CustomIO({}), f16).deferred_norm is None

    class ScaledDifferently(C.OnlineAbsNorm):        # o_scale does not match the normalisation of the scores
        @staticmethod
        def online_fwd(scores, online_rowscales, b, h, q_idx):
            s, rs, o_scale = C.OnlineAbsNorm.online_fwd(scores, online_rowscales, b, h, q_idx)
            return s, rs, o_scale * 0.5
    assert L.trace_functors(C.make_scale_score_mod(0.125), None, ScaledDifferently(), CustomIO({}), f16).deferred_norm is None
    monkeypatch.setenv("AE_DEFER_NORM", "0")
    lf0 = L.trace_functors(C.retention_score_mod, C.causal_mask, C.OnlineRetention(), C.retention_custom_inputs(),
                           f16, "0")
    assert lf0.deferred_norm is None and not lf0.o_scale_one


def test_tuner_cache_records(tmp_path):
    """tune=True / tune_file: the json records of the reference's tuner (attn_tl.py:465-500: a list of the five
    problem keys plus ``tuned_config``), looked up at construction; nothing is measured or written without a GPU
    call."""
    import json
    from core.lower import tuner
    f = str(tmp_path / "tuned.json")
    pk = tuner.problem_keys((2, "heads", 1024, 128), 128, 128)
    assert pk == {"batch": 2, "heads": 32, "seq_len": 1024, "dim": 128, "dimv": 128}   # dynamic dims: attn_tl.py:465-472
    assert tuner.lookup(f, pk) is None
    cands = tuner.prefill_candidates(128, 128, softmax=(0.1, "m", "r"), elementwise=False)
    assert len(cands) == 4 and cands[0].template == "ae_prefill_pipe.hip"
    assert len(tuner.prefill_candidates(128, 128, None, False)) == 3
    assert [c.block_n for c in tuner.prefill_candidates(256, 512, None, False)] == [32]
    assert [(c.waves_per_eu, c.block_n) for c in tuner.prefill_candidates(192, 128, None, False)] == \
        [(2, 64), (2, 32), (1, 64), (1, 32)]
    assert [(c.template, c.block_n) for c in tuner.prefill_candidates(192, 192, None, False)] == \
        [("ae_prefill_simple.hip", 32), ("ae_prefill_simple.hip", 64)]
    tuner.store(f, pk, tuner.encode_tiles(cands[2]))
    tuner.store(f, {**pk, "batch": 4}, [128, 128, 2, 256, False])     # a record as the reference writes it
    recs = json.load(open(f))
    assert [sorted(r) for r in recs] == [sorted(list(pk) + ["tuned_config"])] * 2
    assert recs[0]["tuned_config"] == [128, 32, 2, 256, 2, "ae_prefill.hip"]
    assert tuner.decode_tiles(tuner.lookup(f, pk), cands) == cands[2]
    assert tuner.decode_tiles(tuner.lookup(f, {**pk, "batch": 4}), cands) is None   # not one of this build's tiles

    sm = C.make_scale_score_mod(0.1)
    hit = AttentionEngine(_meta(2, 32, 32, 1024, 1024, 128, 128, torch.float16), CustomIO({}), sm, C.causal_mask,
                          C.OnlineSoftmax(), tune=True, tune_file=f)
    assert hit._op.tiles == cands[2] and not hit._op._tune_pending
    assert "#define AE_BN 32" in hit.tl_code
    miss = AttentionEngine(_meta(4, 32, 32, 1024, 1024, 128, 128, torch.float16), CustomIO({}), sm, C.causal_mask,
                           C.OnlineSoftmax(), tune=True, tune_file=f)
    assert miss._op._tune_pending and miss._op.tiles == cands[0]      # measured at the first call on a GPU
    plain = AttentionEngine(_meta(2, 32, 32, 1024, 1024, 128, 128, torch.float16), CustomIO({}), sm, C.causal_mask,
                            C.OnlineSoftmax(), tune_file=f)
    assert plain._op.tiles == cands[0] and not plain._op._tune_pending
    tuner.store(f, pk, tuner.encode_tiles(cands[1]))                  # replaces the record of that problem
    assert len(json.load(open(f))) == 2 and tuner.decode_tiles(tuner.lookup(f, pk), cands) == cands[1]
    assert json.load(open(f)) == recs[1:] + [{**pk, "tuned_config": tuner.encode_tiles(cands[1])}]


def test_tuner_store_survives_a_damaged_file(tmp_path):
    """A tune_file that was cut short in the middle of a write (or written by two processes at once) still gives
    up its complete records, and the next store keeps them; the store itself replaces the file in one step and
    leaves no temporary file behind."""
    import json
    import os
    from core.lower import tuner
    f = str(tmp_path / "tuned.json")
    pk = {"batch": 2, "heads": 32, "seq_len": 1024, "dim": 128, "dimv": 128}
    for b in (1, 2, 3):
        tuner.store(f, {**pk, "batch": b}, [128, 64, 2, 256, 2, "ae_prefill.hip"])
    text = open(f).read()
    third = text.rindex("{")
    open(f, "w").write(text[:third + 40])             # the third record is torn, the closing bracket is gone
    with pytest.raises(ValueError):
        json.load(open(f))
    assert tuner.lookup(f, {**pk, "batch": 1}) == [128, 64, 2, 256, 2, "ae_prefill.hip"]
    assert tuner.lookup(f, {**pk, "batch": 3}) is None
    tuner.store(f, {**pk, "batch": 4}, [256, 64, 2, 256, 1, "ae_prefill_pipe.hip"])
    recs = json.load(open(f))                          # whole again
    assert [r["batch"] for r in recs] == [1, 2, 4]
    assert os.listdir(tmp_path) == ["tuned.json"]
    open(f, "w").write("not json at all")
    assert tuner.lookup(f, pk) is None
    tuner.store(f, pk, [1])
    assert json.load(open(f)) == [{**pk, "tuned_config": [1]}]


def test_decode_kernel_cache_is_keyed_by_the_merge_form(monkeypatch):
    """GQADecodeOp keeps one compiled kernel pair per (splits, even kv, merge form).  Whether the split kernel
    merges its waves' partial results itself (AE_MERGE_IN_WG) depends on ``static_workspace`` and on an
    environment variable, both of which may change between two calls of one engine; a kernel compiled for one
    form must never be handed to the launch of the other (the merging kernel leaves the work buffers unwritten,
    the other one stores through them).  hipRTC runs on the CPU, so the variants are really compiled here."""
    from core.lower.lower_decode import GQADecodeOp
    dt = torch.float16
    B, Hq, Hkv, Skv, D = 128, 32, 8, 777, 128          # plans 4 splits: the waves of one workgroup
    meta = (meta_tensor(B, Hq, 1, D, dtype=dt), meta_tensor(B, Hkv, Skv, D, dtype=dt), meta_tensor(B, Hkv, Skv, D, dtype=dt))
    op = GQADecodeOp(meta, CustomIO({}), C.make_scale_score_mod(D ** -0.5), None, C.OnlineSoftmax(), "-inf")
    n_split, _ = op.plan_splits(B, Hq, Hkv, Skv)
    assert n_split == op.N_WAVES
    monkeypatch.delenv("AE_DECODE_MERGE_IN_WG", raising=False)
    # the constructor compiled the merging form
    assert set(op._variants) == {(4, False, 1)}
    merged = op._variant(n_split, False, op._merge_mode(n_split))
    assert "#define AE_MERGE_IN_WG 1" in merged[3] and merged[1].merge_in_wg == 1
    # the documented toggle: the launch without allocations keeps the merge kernel
    op.static_workspace = True
    assert not op.merges_in_workgroup(n_split)
    plain = op._variant(n_split, False, op._merge_mode(n_split))
    assert plain is not merged and plain[0] is not merged[0]
    assert "#define AE_MERGE_IN_WG 0" in plain[3] and plain[1].merge_in_wg == 0
    op.static_workspace = False
    assert op._variant(n_split, False, op._merge_mode(n_split)) is merged
    # ... and the environment variable that keeps the two launches
    monkeypatch.setenv("AE_DECODE_MERGE_IN_WG", "0")
    assert op._variant(n_split, False, op._merge_mode(n_split)) is plain
    assert set(op._variants) == {(4, False, 1), (4, False, 0)}


def test_decode_splits_over_several_workgroups_merge_in_the_last_one(monkeypatch):
    """A small batch spreads one kv axis over several workgroups; the one that finishes last merges
    (AE_MERGE_LAST, merge_in_wg = 2) unless the launch must not keep buffers of its own (``static_workspace``)
    or the environment asks for the two launches.  Compiled here by hipRTC, without register spills."""
    from core.lower.lower_decode import GQADecodeOp
    dt = torch.float16
    B, Hq, Hkv, Skv, D = 1, 32, 8, 8192, 128
    meta = (meta_tensor(B, Hq, 1, D, dtype=dt), meta_tensor(B, Hkv, Skv, D, dtype=dt), meta_tensor(B, Hkv, Skv, D, dtype=dt))
    monkeypatch.delenv("AE_DECODE_MERGE_LAST", raising=False)
    op = GQADecodeOp(meta, CustomIO({}), C.make_scale_score_mod(D ** -0.5), None, C.OnlineSoftmax(), "-inf")
    n_split, _ = op.plan_splits(B, Hq, Hkv, Skv)
    assert n_split > op.N_WAVES and op._merge_mode(n_split) == 2
    assert set(op._variants) == {(n_split, True, 2)}
    last = op._variant(n_split, True, 2)
    assert "#define AE_MERGE_LAST 1" in last[3] and "#define AE_MERGE_IN_WG 0" in last[3] and last[1].merge_in_wg == 2
    op.static_workspace = True
    assert op._merge_mode(n_split) == 0
    op.static_workspace = False
    monkeypatch.setenv("AE_DECODE_MERGE_LAST", "0")
    assert op._merge_mode(n_split) == 0
    plain = op._variant(n_split, True, 0)
    assert "#define AE_MERGE_LAST 0" in plain[3] and plain[0] is not last[0]


def test_decode_build_that_spills_is_built_again_for_one_wave_a_simd():
    """Value heads of 256 do not fit the 256 registers of two waves a SIMD (85 spilled registers, 2.3x the time on
    the chip); the operator then builds the kernel for one wave a SIMD, which does not spill.  Head dims of 128
    keep two waves."""
    import warnings
    from core.lower.lower_decode import GQADecodeOp
    dt = torch.float16
    for D, want in ((256, 1), (128, 2)):
        B, Hq, Hkv, Skv = 64, 32, 8, 8192
        meta = (meta_tensor(B, Hq, 1, D, dtype=dt), meta_tensor(B, Hkv, Skv, D, dtype=dt), meta_tensor(B, Hkv, Skv, D, dtype=dt))
        with warnings.catch_warnings():
            warnings.simplefilter("error")
            op = GQADecodeOp(meta, CustomIO({}), C.make_scale_score_mod(D ** -0.5), None, C.OnlineSoftmax(), "-inf")
        (module, _, _, src), = op._variants.values()
        assert f"#define AE_WAVES_PER_EU {want}" in src
        assert module.kernel_info()["ae_decode_split_kernel"].get(".vgpr_spill_count", 0) == 0


def test_numerics_keywords_of_the_constructor(monkeypatch):
    """``exact_scale`` / ``defer_norm`` reach the generated configuration; left at None they follow the defaults
    (and the environment switches the tests use)."""
    monkeypatch.delenv("AE_PREFILL_PRESCALE", raising=False)
    monkeypatch.delenv("AE_DEFER_NORM", raising=False)
    monkeypatch.setenv("AE_PREFILL_KERNEL", "pipelined")
    f16 = torch.float16
    sm = C.make_scale_score_mod(0.1)
    meta = _meta(2, 32, 32, 1024, 1024, 128, 128, f16)
    default = AttentionEngine(meta, CustomIO({}), sm, C.causal_mask, C.OnlineSoftmax())
    exact = AttentionEngine(meta, CustomIO({}), sm, C.causal_mask, C.OnlineSoftmax(), exact_scale=True)
    folded = AttentionEngine(meta, CustomIO({}), sm, C.causal_mask, C.OnlineSoftmax(), exact_scale=False)
    assert default._op.tiles.template == "ae_prefill_pipe.hip"
    assert "AE_PRESCALE" not in default.tl_code
    assert "#define AE_PRESCALE 0" in exact.tl_code and "#define AE_PRESCALE 1" in folded.tl_code
    monkeypatch.setenv("AE_PREFILL_PRESCALE", "0")          # the keyword wins over the environment
    assert "#define AE_PRESCALE 1" in AttentionEngine(meta, CustomIO({}), sm, None, C.OnlineSoftmax(),
                                                      exact_scale=False).tl_code
    monkeypatch.delenv("AE_PREFILL_KERNEL")
    rmeta = _meta(1, 2, 2, 256, 256, 64, 64, f16)
    args = (rmeta, C.retention_custom_inputs(), C.retention_score_mod, C.causal_mask, C.OnlineRetention())
    assert AttentionEngine(*args, mask_value="0").attention.functors.deferred_norm == "r"
    assert AttentionEngine(*args, mask_value="0", defer_norm=False).attention.functors.deferred_norm is None
    monkeypatch.setenv("AE_DEFER_NORM", "0")
    assert AttentionEngine(*args, mask_value="0").attention.functors.deferred_norm is None
    assert AttentionEngine(*args, mask_value="0", defer_norm=True).attention.functors.deferred_norm == "r"


def test_tile_classes_of_a_user_block_mask():
    """PrefillBwdOp.block_mask_tile_classes (the tables the backward launches read when the forward ran on a block
    mask the user supplied) against brute force over the expanded mask, for block sizes below, equal to and above
    the tile sizes and sequence lengths that are not multiples of either."""
    from core.lower.prefill_bwd_op import PrefillBwdOp
    g = torch.Generator().manual_seed(2)
    for bm, bn, Sq, Skv in ((128, 128, 1024, 1024), (32, 64, 640, 576), (64, 128, 448, 450), (256, 32, 700, 333),
                            (48, 96, 500, 400)):
        nq, nk = -(-Sq // bm), -(-Skv // bn)
        blocks = (torch.rand(2, 3, nq, nk, generator=g) < 0.5).to(torch.int8)
        dense = blocks.bool().repeat_interleave(bm, 2).repeat_interleave(bn, 3)[:, :, :Sq, :Skv]
        for tm, tn in ((128, 64), (256, 64), (64, 128)):
            got = PrefillBwdOp.block_mask_tile_classes(blocks, bm, bn, Sq, Skv, tm, tn)
            assert got.shape == (2, 3, -(-Sq // tm), -(-Skv // tn)) and got.dtype == torch.int8
            for i in range(got.shape[2]):
                for j in range(got.shape[3]):
                    t = dense[:, :, i * tm:(i + 1) * tm, j * tn:(j + 1) * tn]
                    some, every = t.any(-1).any(-1), t.all(-1).all(-1)
                    want = some.to(torch.int8) + (some & every).to(torch.int8)
                    assert torch.equal(got[:, :, i, j], want), (bm, bn, Sq, Skv, tm, tn, i, j)
