"""Public API: ``OnlineFunc`` and ``AttentionEngine``.

Drop-in for attention_engine/attn_engine/attn_engine.py: ``OnlineFunc`` (16-105) keeps its
constructor and static-method protocol; ``AttentionEngine(qkv_meta, custom_fwd_inputs, score_mod,
mask_mod, online_func, ...)`` (108-215) keeps its signature and shape dispatch (218-332) and
returns a callable ``mod(q, k, v, *custom_inputs, block_mask=None) -> o`` (388-395).

Behind the API everything is new: the traced functions are lowered to HIP functors, spliced into
the hand-written gfx950 kernel templates under csrc/kernels, compiled with hipRTC through
libae_hip.so and launched on torch's current stream.  There is a single backend; ``backend="tl"``
and ``backend="cute"`` are both accepted and select the call convention only (for MLA the CuTe
form ``mod(q, kv_cache) -> (out, lse)``, attn_engine.py:193-214).  ``tune=True`` with a ``tune_file``
(``tune_bwd`` / ``tune_file_bwd`` for the backward) takes the tile configuration -- for decode engines the
split count -- from that file's record of the problem, or measures the candidates at the first call on a
GPU and records the winner there (core/lower/tuner.py; the reference: attn_tl.py:465-521); without it the
choice is fixed per head dimension and problem size.
"""
from __future__ import annotations

import torch

from core.transform.core import CustomIO, SymbolicArray, SymbolScalar, Var


class OnlineFunc:
    """User-defined online row-scale algorithm (see attn_script/Readme.md:45-65).

    ``online_rowscales``: running per-row state, ``{name: SymbolScalar(name, Var(init))}``;
    ``final_rowscales``: per-row results saved at the end (e.g. lse).
    Subclasses override the static methods below; they are *traced*, not executed on data.
    """

    def __init__(self, online_rowscales: dict, final_rowscales: dict, external_fwd_tensors: CustomIO):
        self.online_rowscales = online_rowscales
        self.final_rowscales = final_rowscales
        self.vars = {"scores": SymbolicArray(), "o_scale": None}
        self.external_fwd_tensors = external_fwd_tensors
        self.doosum_rowscales = SymbolicArray("doosum", Var("doosum"), shape_idx=["block_M"])

    @staticmethod
    def online_fwd(scores, online_rowscales, b, h, q_idx):
        """One kv tile: returns (scores', online_rowscales', o_scale)."""
        o_scale = SymbolScalar("o_scale", Var("o_scale"))
        return scores, online_rowscales, o_scale

    @staticmethod
    def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
        """After the last tile: returns (o', final_rowscales)."""
        return o, online_rowscales

    @staticmethod
    def forward(scores, final_rowscales, b, h, q_idx, kv_idx):
        """Recompute rule of the backward pass, p from the modified scores and the final row scales.  Traced
        for online functions that keep a final row scale of their own and override it (retention); checked
        to be the identity for online functions without row scales; for softmax attention the gradient is
        fixed by the proven forward and the rule is not traced."""
        return scores

    @staticmethod
    def backward(dp, scores, final_rowscales, b, h, q_idx, kv_idx):
        """Backward rule, dscores from dp, the recomputed p (``scores``) and the final row scales; overrides
        may take the rowsum(do * o) row scale as a fourth argument, as attn_script/retention.py:65 does
        (see ``forward``)."""
        return dp

    @staticmethod
    def combine(final_rowscales):
        """Split-KV merge: returns o_scale[num_split, row] applied to the partial outputs."""
        return SymbolScalar("o_scale", Var("o_scale"))


class AttentionEngine:
    def __init__(self, qkv_meta, custom_fwd_inputs, score_mod, mask_mod, online_func,
                 mask_value="-inf", device=None, backend="tl",
                 tune=False, tune_file="", tune_bwd=False, tune_file_bwd="",
                 infer_mask=True, infer_mask_block_M=128, infer_mask_block_N=128,
                 extern_block_mask=False, kv_shared=False, exact_scale=None, defer_norm=None, allow_spills=None):
        """The reference's constructor (attn_engine.py:109-115) plus two numerics switches of this build, both
        None by default (= the faster form) and both only meaningful for prefill engines:

        ``exact_scale=True``: the software-pipelined fp16 softmax kernel multiplies every score by the constant
        of ``score_mod`` in fp32.  By default it folds that constant (times log2 e) into its resident fp16 Q
        fragments, one rounding of the product to fp16, which moves a score by up to 2^-12 of sum|q_d k_d|*c:
        lse then stays within 1e-3 of the fp32 reference while the scaled scores stay below a few tens
        (3e-4 on N(0,1) inputs at head dim 128) and within 2^-11 * max sum|q_d||k_d| * c in general.  bf16
        engines and the other kernels never pre-scale.

        ``defer_norm=False``: online functions of the form ``scores / r_new`` with ``o_scale = r_old / r_new``
        (retention) keep that per-tile form.  By default the lowering accumulates the unnormalised scores and
        divides once in the epilogue (the factors telescope); P, the fp16 operand of the second product, then
        holds |X| instead of |X / r| <= 1, so scores of 65504 and more overflow where the script's form stays
        finite (bf16 has the range of fp32).

        ``allow_spills`` (all engines): what to do with a kernel whose compiled code moves register tuples through
        scratch memory or spills heavily -- one such build of the compiler in use returned wrong output columns,
        see ``core.runtime.hip_rt.check_spills``.  None: a RuntimeWarning names it (the builds of the family in
        which the wrong columns were seen are refused); False: it is refused (``hip_rt.SpillError``; a prefill
        engine whose own choice was the software-pipelined kernel switches to the generic kernel instead); True:
        it runs unchecked."""
        if backend not in ("tl", "cute", "hip"):
            raise ValueError(f"unknown backend {backend!r}")
        if mask_value not in ("-inf", "0"):
            raise ValueError(f"mask_value must be '-inf' or '0', got {mask_value!r}")
        self.backend = backend
        self.block_mask = None
        self.final_rowscales = {}
        if custom_fwd_inputs is None:
            custom_fwd_inputs = CustomIO()
        if online_func is None:
            # the reference's CuTe scripts pass online_func=None for identity-style attention
            online_func = _IdentityOnline()
        self._op = self._select_lower_template(
            qkv_meta, custom_fwd_inputs, score_mod, mask_mod, online_func, mask_value,
            infer_mask=infer_mask, infer_mask_block_M=infer_mask_block_M,
            infer_mask_block_N=infer_mask_block_N, extern_block_mask=extern_block_mask,
            kv_shared=kv_shared,
            tune=dict(tune=bool(tune), tune_file=tune_file, tune_bwd=bool(tune_bwd), tune_file_bwd=tune_file_bwd),
            numerics=dict(exact_scale=exact_scale, defer_norm=defer_norm), allow_spills=allow_spills)
        # generated device source, under the attribute name scripts read
        # (attn_script/reluattn.py:75-76)
        self.tl_code = self._op.source
        self.attention = self._op
        if infer_mask or extern_block_mask:
            self.block_mask = getattr(self._op, "block_mask", None)

    # same dispatch order as attn_engine.py:218-332
    def _select_lower_template(self, qkv_meta, custom_fwd_inputs, score_mod, mask_mod, online_func,
                               mask_value, infer_mask, infer_mask_block_M, infer_mask_block_N,
                               extern_block_mask, kv_shared, tune=None, numerics=None, allow_spills=None):
        dtype_map = {torch.float16: "float16", torch.bfloat16: "bfloat16"}
        q_meta, k_meta, v_meta = qkv_meta
        dtype_map[q_meta.dtype]  # KeyError for unsupported dtypes, as in the reference (225-228, 304)
        q_seqlen, kv_len = q_meta.shape[2], v_meta.shape[2]
        head, head_kv = q_meta.shape[1], v_meta.shape[1]
        # dynamic (string) extents are runtime parameters of the kernels; they only rule out the
        # shape-dependent dispatch to the decode templates
        dynamic = any(isinstance(d, str) for m in qkv_meta for d in m.shape)
        decode_tune = {k: v for k, v in (tune or {}).items() if k in ("tune", "tune_file")}

        if kv_shared:
            from core.lower.lower_decode import MLADecodeOp
            return MLADecodeOp(qkv_meta, custom_fwd_inputs, score_mod, mask_mod, online_func,
                               mask_value, cute_convention=(self.backend == "cute"), allow_spills=allow_spills,
                               **decode_tune)
        if not dynamic and q_seqlen != kv_len and head > head_kv:
            assert q_seqlen < kv_len
            assert q_seqlen == 1
            from core.lower.lower_decode import GQADecodeOp
            return GQADecodeOp(qkv_meta, custom_fwd_inputs, score_mod, mask_mod, online_func, mask_value,
                               allow_spills=allow_spills, **decode_tune)
        # MHA decode (attn_engine.py:273-290 of the reference): a few query tokens against a long KV,
        # split over the kv axis and merged with the user's combine()
        # (an online function that does not override combine() cannot merge splits: it runs unsplit)
        has_combine = online_func is not None and getattr(type(online_func), "combine", None) is not OnlineFunc.combine
        split_kv = not dynamic and q_seqlen != kv_len and head == head_kv and has_combine
        if split_kv:
            assert q_seqlen < kv_len
        from core.lower.prefill_op import PrefillOp
        return PrefillOp(qkv_meta, custom_fwd_inputs, score_mod, mask_mod, online_func, mask_value,
                         infer_mask=infer_mask, infer_mask_block_M=infer_mask_block_M,
                         infer_mask_block_N=infer_mask_block_N, extern_block_mask=extern_block_mask,
                         split_kv=split_kv, allow_spills=allow_spills, **(tune or {}), **(numerics or {}))

    def __call__(self, *args, **kargs):
        if kargs.get("block_mask") is not None:
            self.block_mask = kargs["block_mask"]
        kargs.pop("block_mask", None)
        if self.block_mask is not None:
            o = self._op(*args, self.block_mask, **kargs)
        else:
            o = self._op(*args, **kargs)
        self.final_rowscales = getattr(self._op, "final_rowscales", {})
        return o

    def forward_with_rowscales(self, *args, **kargs):
        """``mod(...)`` plus the final rowscales of that call: (o, {name: fp32 [B, Hq, Sq]})."""
        o = self(*args, **kargs)
        return o, dict(self.final_rowscales)


class _IdentityOnline(OnlineFunc):
    """No row state, no rescale: out = sum_kv score_mod(s) * v."""

    def __init__(self):
        super().__init__({}, {}, CustomIO())

    @staticmethod
    def online_fwd(scores, online_rowscales, b, h, q_idx):
        return scores, online_rowscales, SymbolScalar("o_scale", Var("1"))

    @staticmethod
    def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
        return o, {}
