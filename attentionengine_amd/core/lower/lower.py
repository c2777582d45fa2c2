"""Prefill lowering: traced user functions -> the two generated headers of the HIP template.

Stands where the reference's ``lower_tl`` fills the jinja slots of its TileLang prefill template
(attention_engine/core/lower/lower.py:617-783, with lower_score_mod 475-558, lower_online_func
318-472, lower_custom_inputs 560-614).  Output here: ``ae_config.h`` (compile-time
configuration) and ``ae_functors.h`` (ae_score_mod / ae_mask_mod / ae_online_fwd / ae_epilogue /
ae_load_custom) for csrc/kernels/ae_prefill.hip, plus the tile configuration and mask plan the
host needs at launch time.
"""
from __future__ import annotations

import math
import os
from dataclasses import dataclass, field

import torch

from ..codegen.hip_gen import Emitter, float_literal, init_literal, var_as_constant
from ..transform.core import CustomIO, SymbolicArray, SymbolScalar
from ..transform.graph import Var
from .mask import MASK_HELPERS, LoweredMask, MaskPlan, lower_mask_mod, plan_mask

DTYPE_NAMES = {torch.float16: "float16", torch.bfloat16: "bfloat16"}

# symbolic dimension name of a CustomIO tensor -> index expression inside the kernel
_DIM_INDEX = {"batch": "ctx.b", "heads": "ctx.h", "seq_len": "ctx.q_idx"}
_KV_DIM = "seq_len_kv"


@dataclass
class CustomInput:
    name: str
    shape: list          # as declared: ints or symbolic names
    per_kv: bool         # indexed by kv position -> read inside the tile loop
    torch_dtype: object  # dtype the kernel reads


@dataclass
class LoweredFunctors:
    """Everything the functor header needs, independent of tile sizes."""
    score_mod_body: str
    online_fwd_body: str
    online_fwd_return: str
    epilogue_body: str
    rowstate_fields: list
    rowstate_init: list
    final_rowscale_names: list
    o_scale_one: bool
    customs: list = field(default_factory=list)
    mask: LoweredMask = None
    # (scale, max field, sum field) when the graph is the online softmax of `scores * scale`,
    # scale > 0: the case the software-pipelined prefill kernel is written for
    softmax: tuple = None
    # out = sum_kv f(s) v: no row state, no reduction over the kv tile, no use of the kv index, o_scale = 1,
    # no final row scales (sigmoid / relu attention) - ae_online_fwd<N> may then be called on any subset
    # of a tile's scores, which is how the software-pipelined prefill kernel calls it
    elementwise: bool = False


def _custom_leaves(custom_fwd_inputs: CustomIO, in_dtype, slot_offset: int = 0):
    """Leaf expressions for the CustomIO tensors + their descriptors.

    A tensor whose shape has no kv dimension is loaded once per row into ``cust.<name>``
    (fp32, like the reference's accum_dtype fragments, lower.py:580); one with a
    ``seq_len_kv`` dimension is read per element from global memory in the input dtype
    (lower.py:590-597)."""
    leaves, descs, loads, fields, preambles = {}, [], [], [], {}
    prefetch = []      # body lines of ae_prefetch_custom (per-kv inputs, kernels that fetch a tile ahead)
    for slot, (name, sym) in enumerate(custom_fwd_inputs.input_tensors.items()):
        slot += slot_offset
        dims = list(sym.shape_idx)
        per_kv = _KV_DIM in dims
        idx_terms, stride = [], "1"
        # row-major index over the declared shape
        extents = {"batch": "p.batch", "heads": "p.heads_q", "seq_len": "p.seqlen_q",
                   _KV_DIM: "p.seqlen_kv"}
        kv_stride = None
        base_terms, q_stride = [], "0"      # the same index without its query-row term, and that term's stride
        for d in reversed(dims):
            if d in _DIM_INDEX:
                # rows past seqlen_q (a ragged last q tile) compute on the last row and are never stored
                ix = "(ctx.q_idx < p.seqlen_q ? ctx.q_idx : p.seqlen_q - 1)" if d == "seq_len" else _DIM_INDEX[d]
                idx_terms.append(f"(int64_t)({ix}) * ({stride})")
                if d == "seq_len":
                    q_stride = stride
                else:
                    base_terms.append(idx_terms[-1])
                stride = f"{stride} * (int64_t){extents[d]}"
            elif d == _KV_DIM:
                kv_stride = stride          # the kv term is added per element inside the tile loop
                stride = f"{stride} * (int64_t){extents[d]}"
            elif d == "1":
                pass
            else:
                raise NotImplementedError(
                    f"custom input {name!r}: dimension {d!r} (use 1, 'batch', 'heads', 'seq_len', 'seq_len_kv')")
        index = " + ".join(idx_terms) if idx_terms else "0"
        if per_kv:
            # one element per score (e.g. the retention decay mask, attn_script/retention.py:14-16):
            # the row's base pointer is kept per lane, elements are read in the input dtype where the
            # scores are modified; kv positions past the end of a ragged tile read the last element
            base_index = " + ".join(base_terms) if base_terms else "0"
            fields += [f"const ae_elem* {name}_row;", f"int64_t {name}_kvstride;", f"int {name}_kvlast;",
                       "#if AE_KV_PF_GROUPS > 0",
                       f"ae_elem4 {name}_pf[AE_KV_PF_GROUPS];   // the lane's elements of the tile fetched ahead",
                       "#endif",
                       "#if AE_KV_COALESCED",
                       f"const ae_elem* {name}_base;            // element (b, h, row 0, kv 0)",
                       f"int64_t {name}_qstride;                // elements between query rows",
                       f"ae_elem8 {name}_raw[AE_KV_PF_GROUPS / 2];   // the tile fetched ahead, 16 bytes of a row per lane",
                       f"bool {name}_staged;                    // raw holds the tile (else pf does)",
                       "#endif"]
            loads += [f"c.{name}_row = (const ae_elem*)p.custom[{slot}] + ({index});",
                      f"c.{name}_kvstride = {kv_stride};", f"c.{name}_kvlast = p.seqlen_kv - 1;",
                      "#if AE_KV_COALESCED",
                      f"c.{name}_base = (const ae_elem*)p.custom[{slot}] + ({base_index});",
                      f"c.{name}_qstride = {q_stride};", f"c.{name}_staged = false;",
                      "#endif"]
            leaves[id(sym)] = (f"cm_{name}", True)
            # a lane's elements come in groups of four consecutive kv positions (ae_kv_off): one 8-byte
            # load per group where the tensor allows it (unit kv stride, aligned, inside the row)
            # A kernel that defines AE_KV_PF_GROUPS (a lane's groups per tile) calls ae_prefetch_custom for
            # the NEXT tile once the functors have used the current one: the loads then have a whole tile
            # of MFMAs to arrive, instead of stalling the functor that issues them.
            group_load = [
                "    const int kv = kv_base + ae_kv_off(4 * g);",
                f"    const ae_elem* src = cust.{name}_row + (int64_t)kv * cust.{name}_kvstride;",
                f"    if (cust.{name}_kvstride == 1 && kv + 3 <= cust.{name}_kvlast && ((unsigned long)src & 7) == 0) {{",
                f"      cust.{name}_pf[g] = *(const ae_elem4*)src;",
                "    } else {",
                "#pragma unroll",
                "      for (int i = 0; i < 4; i++) {",
                f"        const int kvi = kv + i < cust.{name}_kvlast ? kv + i : cust.{name}_kvlast;",
                f"        cust.{name}_pf[g][i] = cust.{name}_row[(int64_t)kvi * cust.{name}_kvstride];",
                "      }",
                "    }"]
            # Coalesced form (kernels that define AE_KV_COALESCED and hand a wave-private LDS scratch to
            # ae_stage_custom): a lane's own elements are 8-byte pieces of 32 different rows per load
            # instruction, which the texture path serves one cache line at a time; instead instruction
            # (half h, row group rg) fetches 64 contiguous bytes of each of 16 rows (row 16*rg + lane/4,
            # 16 bytes at kv 32*h + 8*(lane%4)) and the wave redistributes the tile through LDS.
            coalesced = [
                "#if AE_KV_COALESCED",
                f"  cust.{name}_staged = cust.{name}_kvstride == 1 && kv0 + 8 * AE_KV_PF_GROUPS <= p.seqlen_kv && "
                f"(cust.{name}_qstride & 7) == 0 && (((unsigned long)cust.{name}_base) & 15) == 0;",
                f"  if (cust.{name}_staged) {{",
                "#pragma unroll",
                "    for (int i = 0; i < AE_KV_PF_GROUPS / 2; i++) {",
                "      int row = row0 + 16 * (i & 1) + (lane >> 2);",
                "      row = row < p.seqlen_q ? row : p.seqlen_q - 1;",
                f"      cust.{name}_raw[i] = *(const ae_elem8*)(cust.{name}_base + (int64_t)row * cust.{name}_qstride + "
                "kv0 + 32 * (i >> 1) + 8 * (lane & 3));",
                "    }",
                "  } else",
                "#endif",
                "  {"]
            prefetch += [*coalesced, "#pragma unroll", "  for (int g = 0; g < AE_KV_PF_GROUPS; g++) {", *group_load,
                         "  }", "  }"]
            stage = preambles.setdefault("stage", [])
            stage += [
                f"  if (cust.{name}_staged) {{",
                "#pragma unroll",
                "    for (int h = 0; h < AE_KV_PF_GROUPS / 4; h++) {",
                "      // rows of 64 bytes (32 kv positions) at a pitch of 80 (16-byte aligned for the 128-bit writes)",
                "#pragma unroll",
                "      for (int rg = 0; rg < 2; rg++)",
                "        *(__attribute__((address_space(3))) ae_elem8*)(scratch + (16 * rg + (lane >> 2)) * 80 + (lane & 3) * 16) = "
                f"cust.{name}_raw[2 * h + rg];",
                "#pragma unroll",
                "      for (int g = 0; g < 4; g++)",
                f"        cust.{name}_pf[4 * h + g] = *(const __attribute__((address_space(3))) ae_elem4*)"
                "(scratch + (lane & 31) * 80 + 16 * g + 8 * (lane >> 5));",
                "    }",
                "  }"]
            preambles[id(sym)] = [
                f"  float cm_{name}[N];",
                "#if AE_KV_PF_GROUPS > 0",
                '  static_assert(N == 4 * AE_KV_PF_GROUPS, "the kernel fetches a whole tile of a lane\'s elements ahead");',
                "#pragma unroll",
                f"  for (int e = 0; e < N; e++) cm_{name}[e] = (float)cust.{name}_pf[e >> 2][e & 3];",
                "#else",
                "#pragma unroll",
                "  for (int g = 0; g < N / 4; g++) {",
                "    const int kv = ctx.kv_base + ae_kv_off(4 * g);",
                f"    const ae_elem* src = cust.{name}_row + (int64_t)kv * cust.{name}_kvstride;",
                f"    if (cust.{name}_kvstride == 1 && kv + 3 <= cust.{name}_kvlast && ((unsigned long)src & 7) == 0) {{",
                "      const ae_elem4 w = *(const ae_elem4*)src;",
                "#pragma unroll",
                f"      for (int i = 0; i < 4; i++) cm_{name}[4 * g + i] = (float)w[i];",
                "    } else {",
                "#pragma unroll",
                "      for (int i = 0; i < 4; i++) {",
                f"        const int kvi = kv + i < cust.{name}_kvlast ? kv + i : cust.{name}_kvlast;",
                f"        cm_{name}[4 * g + i] = (float)cust.{name}_row[(int64_t)kvi * cust.{name}_kvstride];",
                "      }",
                "    }",
                "  }",
                "#endif"]
            descs.append(CustomInput(name, dims, per_kv, in_dtype))
            continue
        fields.append(f"float {name};")
        loads.append(f"c.{name} = ((const float*)p.custom[{slot}])[{index}];")
        leaves[id(sym)] = (f"cust.{name}", False)
        tdtype = torch.float32
        descs.append(CustomInput(name, dims, per_kv, tdtype))
    preambles["prefetch"] = prefetch
    preambles.setdefault("stage", [])
    return leaves, descs, loads, fields, preambles


# threshold of the lazy running maximum, in the (natural-log) units of the user's exp():
# exponentials stay below e^tau = 256, harmless for fp16/bf16 P and fp32 sums
LAZY_MAX_TAU = 8.0 * 0.6931471805599453


def is_plain_softmax(m_new, new_scores, scores_mod) -> bool:
    """True when the graph ``find_lazy_softmax`` accepted is exactly the online softmax OF scores_mod:
    ``m_new = max(m, rowmax(scores_mod))`` and ``scores' = exp(scores_mod - m_new)``.  The wider class
    (any per-row x inside the max, anything with a kv axis in front of ``- m_new``) is still
    independent of the reference point, so it may use the lazy maximum, but only this case may run
    the kernels that hard-code ``exp(c * S - m)`` or the softmax backward."""
    try:
        x = m_new.prev[1]
        return (x.code.type == "ReduceMax" and x.prev[0] is scores_mod
                and new_scores.prev[0].prev[0] is scores_mod)
    except (IndexError, AttributeError):
        return False


def find_lazy_softmax(online_func, rowscales, new_scores, new_rowscales, o_scale):
    """Return the ``m_new = max(m, x)`` symbol if the traced online function is the online softmax
    (attn_script/mha.py:47-72), whose outputs do not depend on the reference point m:

        m_new = max(m, x)                 x: one value per row
        o_scale = exp(m - m_new)
        scores' = exp(S - m_new)
        r_new = r * o_scale + rowsum(scores')
        epilogue: o / r  (or o / (r + c), c a constant of at most 1e-20)  and  lse = log(r) + m

    Every use of m_new must be one of these.  Then m_new may lag behind the true maximum
    (thresholded update, see codegen/hip_gen.py) without changing o or lse.  Anything else: None.
    """
    try:
        if len(rowscales) != 2 or set(new_rowscales) != set(rowscales):
            return None
        (mk, m_new), = [(k, v) for k, v in new_rowscales.items() if v.code.type == "Max"]
        (rk, r_new), = [(k, v) for k, v in new_rowscales.items() if k != mk]
        m, r = rowscales[mk], rowscales[rk]
        if m_new.prev[0] is not m or "block_N" in m_new.prev[1].shape_idx:
            return None

        def is_exp_minus(sym, lhs_is):
            return (sym.code.type == "Exp" and sym.prev[0].code.type == "Sub"
                    and sym.prev[0].prev[1] is m_new and lhs_is(sym.prev[0].prev[0]))
        if not (isinstance(o_scale, SymbolScalar) and is_exp_minus(o_scale, lambda x: x is m)):
            return None
        if not is_exp_minus(new_scores, lambda x: "block_N" in x.shape_idx):
            return None
        if r_new.code.type != "Add":
            return None
        a, bsum = r_new.prev
        if not (a.code.type == "Mul" and a.prev[0] is r and is_exp_minus(a.prev[1], lambda x: x is m)):
            return None
        if not (bsum.code.type == "ReduceSum" and bsum.prev[0] is new_scores):
            return None
        # every use of m_new: the two Sub nodes feeding exp (and being the new rowscale)
        for use in m_new.use_list:
            if not (use.code.type == "Sub" and use.prev[1] is m_new and
                    all(u.code.type == "Exp" for u in use.use_list) and use.use_list):
                return None
        # epilogue shape
        from ..transform.core import SymbolicArray as _SA
        for v in rowscales.values():
            v.clear_codegen()
        acc = _SA("acc_o", Var("acc_o"), shape_idx=["block_M", "dimv"])
        dummy = SymbolScalar("b", Var("b"), shape_idx=[])
        o_new, finals = online_func.online_fwd_epilogue(acc, rowscales, dummy, dummy, dummy)
        if not (o_new.code.type == "Div" and o_new.prev[0] is acc):
            return None
        den = o_new.prev[1]
        if den is not r:
            # o / (r + c) with a constant 0 <= c <= 1e-20, the guard of attn_script/sparseattn.py:68 ("to avoid division
            # by zero").  A row with a visible key has r >= 1 whatever the (lagging) reference -- its largest score
            # contributes exp(0) or more --, so r + c == r in fp32; a row without one has o = 0 and gives 0 either way.
            if den.code.type != "Add" or len(den.prev) != 2:
                return None
            rr, cc = den.prev if den.prev[0] is r else den.prev[::-1]
            if rr is not r or cc.code.type != "Const" or not 0.0 <= float(cc.code.value) <= 1e-20:
                return None
        if len(finals) != 1:
            return None
        (lse,) = finals.values()
        if lse.code.type != "Add":
            return None
        x, y = lse.prev
        ok = (x.code.type == "Log" and x.prev[0] is r and y is m) or (y.code.type == "Log" and y.prev[0] is r and x is m)
        if not ok:
            return None
        # m and r must not be used for anything else in the epilogue
        if len(m.use_list) != 1 or len(r.use_list) != 2:
            return None
        return m_new
    except (ValueError, IndexError, AttributeError):
        return None
    finally:
        for v in rowscales.values():
            v.clear_codegen()


def _pure_scale(sym, scores):
    """The constant c if ``sym`` is ``scores`` multiplied / divided by python numbers only, else None."""
    c = 1.0
    while sym is not scores:
        t = sym.code.type
        if t not in ("Mul", "Div") or len(sym.prev) != 2:
            return None
        a, b = sym.prev
        if b.code.type == "Const" and (t == "Mul" or float(b.code.value) != 0.0):
            c = c * float(b.code.value) if t == "Mul" else c / float(b.code.value)
            sym = a
        elif a.code.type == "Const" and t == "Mul":
            c *= float(a.code.value)
            sym = b
        else:
            return None
    return c


def _no_tile_reduction(node) -> bool:
    """True when no node of the graph reduces over the kv-tile axis (a reduction node, or a value without the
    ``block_N`` dimension computed from one that has it)."""
    seen, stack = set(), [node]
    while stack:
        n = stack.pop()
        if id(n) in seen or not isinstance(n, SymbolScalar):
            continue
        seen.add(id(n))
        prev = [q for q in (n.prev or []) if isinstance(q, SymbolScalar)]
        if "Reduce" in str(getattr(n.code, "type", "")):
            return False
        if "block_N" not in n.shape_idx and any("block_N" in q.shape_idx for q in prev):
            return False
        stack.extend(prev)
    return True


def _depends_on(node, target) -> bool:
    seen, stack = set(), [node]
    while stack:
        n = stack.pop()
        if n is target:
            return True
        if id(n) in seen or not isinstance(n, SymbolScalar):
            continue
        seen.add(id(n))
        stack.extend(n.prev or [])
    return False


def find_deferred_norm(rowscales, new_scores, new_rowscales, o_scale):
    """Online functions that renormalise on every tile: ``scores' = X / r_new`` and
    ``o_scale = r_old / r_new`` with r a row scale and X free of it (retention's running sum of |s|,
    attn_script/retention.py:40-60).  The factors telescope: the output equals (sum over tiles of X v) / r_final,
    so the kernels may accumulate X v unscaled - no rescale of the whole accumulator per tile - and divide
    once in the epilogue.  What changes is the range of P, the operand of the second product: |X / r| <= 1 in
    the script's form, |X| itself here, so scores of size 65504 and more overflow an fp16 P (bf16 has the
    range of fp32); ``AttentionEngine(..., defer_norm=False)`` (or AE_DEFER_NORM=0 in the environment) keeps the
    script's form.  Returns (name of r, X) or None."""
    if not (isinstance(new_scores, SymbolScalar) and isinstance(o_scale, SymbolScalar)):
        return None
    if new_scores.code.type != "Div" or o_scale.code.type != "Div":
        return None
    x, r_new = new_scores.prev
    r_old, r_new2 = o_scale.prev
    if r_new is not r_new2:
        return None
    names = [k for k, v in new_rowscales.items() if v is r_new]
    if len(names) != 1 or rowscales.get(names[0]) is not r_old:
        return None
    if _depends_on(x, r_new) or _depends_on(x, r_old):
        return None
    return names[0], x


def trace_functors(score_mod, mask_mod, online_func, custom_fwd_inputs: CustomIO, in_dtype,
                   mask_value: str = "-inf", defer_norm=None) -> LoweredFunctors:
    """Trace score_mod / online_fwd / online_fwd_epilogue on symbols and emit their bodies.  ``defer_norm``
    (None: on, unless AE_DEFER_NORM=0 is in the environment): see find_deferred_norm."""
    custom_fwd_inputs = custom_fwd_inputs if custom_fwd_inputs is not None else CustomIO()
    cust_leaves, customs, cust_loads, cust_fields, cust_preambles = _custom_leaves(custom_fwd_inputs, in_dtype)
    cust_prefetch = cust_preambles.pop("prefetch")
    cust_stage = cust_preambles.pop("stage")

    def index_leaves():
        b = SymbolScalar("b", Var("b"), shape_idx=[])
        h = SymbolScalar("h", Var("h"), shape_idx=[])
        q_idx = SymbolScalar("q_idx", Var("q_idx"), shape_idx=["block_M"])
        kv_idx = SymbolScalar("kv_idx", Var("kv_idx"), shape_idx=["block_N"])
        leaves = {id(b): ("(float)ctx.b", False), id(h): ("(float)ctx.h", False),
                  id(q_idx): ("(float)ctx.q_idx", False), id(kv_idx): ("kvf", True)}
        return b, h, q_idx, kv_idx, leaves

    # ---- score_mod + online_fwd, traced as ONE graph -------------------------------------------
    # (the reference emits two macros, lower.py:475-558 and 318-472; fusing them lets the emitter
    # fold the score scaling into the exponent of the online function)
    b, h, q_idx, kv_idx, leaves = index_leaves()
    scores = SymbolicArray("scores", Var("scores"), shape_idx=["block_M", "block_N"])
    leaves[id(scores)] = ("s", True)
    leaves.update(cust_leaves)
    scores_mod = score_mod(scores, custom_fwd_inputs, b, h, q_idx, kv_idx) if score_mod is not None else scores
    if not isinstance(scores_mod, SymbolScalar):
        raise TypeError("score_mod must return the (modified) scores symbol")
    if not isinstance(scores_mod, SymbolicArray):
        # e.g. `0.5 * scores`: keep the reduction interface of the score tile
        scores_mod.__class__ = SymbolicArray
    rowscales = online_func.online_rowscales
    fields, inits = [], []
    for k, v in rowscales.items():
        v.clear_codegen()
        leaves[id(v)] = (f"st.{k}", False)
        fields.append(k)
        inits.append(init_literal(v.code.name))
    new_scores, new_rowscales, o_scale = online_func.online_fwd(scores_mod, rowscales, b, h, q_idx)
    deferred = find_deferred_norm(rowscales, new_scores, new_rowscales, o_scale)
    if defer_norm is None:
        defer_norm = os.environ.get("AE_DEFER_NORM", "1") != "0"
    if deferred is not None and defer_norm:
        # accumulate unscaled, divide by the final row scale in the epilogue (see find_deferred_norm)
        new_scores, o_scale = deferred[1], 1.0
    else:
        deferred = None
    em = Emitter(leaves, {}, ["block_N"], n="N", prefix="of")
    lazy = find_lazy_softmax(online_func, rowscales, new_scores, new_rowscales, o_scale)
    softmax = None
    if lazy is not None:
        em.lazy_max[id(lazy)] = LAZY_MAX_TAU
        scale = _pure_scale(scores_mod, scores) if is_plain_softmax(lazy, new_scores, scores_mod) else None
        # the specialised kernels start every row from m = -inf (lower.py:23-29: -1e38) and r = 0
        init = {k: float(init_literal(v.code.name).rstrip("f")) for k, v in rowscales.items()}
        inits_ok = all((v <= -1e30) if new_rowscales[k] is lazy else (v == 0.0) for k, v in init.items())
        if scale is not None and inits_ok and scale > 0.0 and math.isfinite(scale):
            (mk,) = [k for k, v in new_rowscales.items() if v is lazy]
            (rk,) = [k for k in new_rowscales if k != mk]
            softmax = (scale, mk, rk)
    new_vals = {k: em.value(v) for k, v in new_rowscales.items()}
    sval = em.value(new_scores)
    o_scale_const = var_as_constant(o_scale) if isinstance(o_scale, SymbolScalar) else float(o_scale)
    o_scale_one = o_scale_const is not None and float(o_scale_const) == 1.0
    oval = em.value(o_scale) if isinstance(o_scale, SymbolScalar) else (repr(float(o_scale)) + "f", False)
    if oval[1]:
        raise NotImplementedError("o_scale must be one value per row")
    body = []
    if id(kv_idx) in em.done:
        body += ["  float kvf[N];", "#pragma unroll",
                 "  for (int e = 0; e < N; e++) kvf[e] = (float)(ctx.kv_base + ae_kv_off(e));"]
    for sid, lines in cust_preambles.items():
        if sid in em.done:
            body += lines
    body.append(em.code())
    if sval[0] != "s":
        src = f"{sval[0]}[e]" if sval[1] else sval[0]
        body += ["#pragma unroll", f"  for (int e = 0; e < N; e++) s[e] = {src};"]
    body.append(f"  const float ae_o_scale = {oval[0]};")
    for k, (expr, is_arr) in new_vals.items():
        if k not in rowscales:
            raise NotImplementedError(f"online_fwd returned an undeclared rowscale {k!r}")
        if is_arr:
            raise NotImplementedError(f"rowscale {k!r} must be one value per row")
        if expr != f"st.{k}":
            body.append(f"  st.{k} = {expr};")
    online_fwd_body = "\n".join(body)
    elementwise = (not rowscales and not new_rowscales and o_scale_one and id(kv_idx) not in em.done
                   and not any(sid in em.done for sid in cust_preambles) and _no_tile_reduction(new_scores))
    score_mod_body = "  // score_mod is fused into ae_online_fwd"

    # ---- epilogue -------------------------------------------------------------------------
    b, h, q_idx, _, leaves = index_leaves()
    acc = SymbolicArray("acc_o", Var("acc_o"), shape_idx=["block_M", "dimv"])
    leaves[id(acc)] = ("o", True)
    leaves.update(cust_leaves)
    for k, v in rowscales.items():
        v.clear_codegen()
        leaves[id(v)] = (f"st.{k}", False)
    o_new, final_rowscales = online_func.online_fwd_epilogue(acc, rowscales, b, h, q_idx)
    em = Emitter(leaves, {}, ["dimv"], n="N", prefix="ep")
    oval = em.value(o_new)
    fvals = [(k, em.value(v)) for k, v in final_rowscales.items()]
    if any(sid in em.done for sid in cust_preambles):
        raise NotImplementedError("a custom input with a seq_len_kv dimension cannot be used in the epilogue")
    body = []
    if deferred is not None:
        body += [f"  // the accumulator holds the unscaled sum: the per-tile normalisation by st.{deferred[0]} was deferred",
                 f"  {{ const float ae_inv = 1.0f / st.{deferred[0]};", "#pragma unroll",
                 "    for (int e = 0; e < N; e++) o[e] *= ae_inv; }"]
    body.append(em.code())
    if oval[0] != "o":
        src = f"{oval[0]}[e]" if oval[1] else oval[0]
        body += ["#pragma unroll", f"  for (int e = 0; e < N; e++) o[e] = {src};"]
    for i, (k, (expr, is_arr)) in enumerate(fvals):
        if is_arr:
            raise NotImplementedError(f"final rowscale {k!r} must be one value per row")
        body.append(f"  frs[{i}] = {expr};")
    epilogue_body = "\n".join(body)

    lowered_mask = lower_mask_mod(mask_mod) if mask_mod is not None else None
    lf = LoweredFunctors(score_mod_body, online_fwd_body, "ae_o_scale", epilogue_body, fields, inits,
                         [k for k, _ in fvals], o_scale_one, customs, lowered_mask)
    lf.custom_fields = cust_fields
    lf.custom_loads = cust_loads
    lf.custom_prefetch = cust_prefetch
    lf.custom_stage = cust_stage
    lf.softmax = softmax
    lf.elementwise = bool(elementwise and not fvals)
    lf.deferred_norm = deferred[0] if deferred is not None else None
    return lf


def render_functors(lf: LoweredFunctors) -> str:
    """Text of ae_functors.h."""
    nrs = max(1, len(lf.final_rowscale_names))
    fields = "\n".join(f"  float {f};" for f in lf.rowstate_fields) or "  int ae_unused;"
    inits = "\n".join(f"  st.{f} = {v};" for f, v in zip(lf.rowstate_fields, lf.rowstate_init)) or "  st.ae_unused = 0;"
    cfields = "\n".join("  " + f for f in lf.custom_fields) or "  int ae_unused;"
    cloads = "\n".join("  " + ld for ld in lf.custom_loads) or "  c.ae_unused = 0;"
    mask_body = lf.mask.body if lf.mask is not None else "  return true;"
    prefetch = ""
    if getattr(lf, "custom_prefetch", None):
        body = "\n".join(lf.custom_prefetch)
        stage_body = "\n".join(getattr(lf, "custom_stage", []))
        prefetch = f"""#if AE_KV_PF_GROUPS > 0
// custom inputs with a kv dimension: the lane's elements of the tile whose first kv position (for this lane)
// is kv_base, fetched into cust for the functors' next call
#define AE_HAS_KV_PREFETCH 1
// kv_base: the lane's first kv position of the tile (its own elements); row0 / kv0: first query row of the wave's
// 32-row block and first kv position of the tile (the coalesced form)
AE_DEV void ae_prefetch_custom(ae_custom& cust, int kv_base, int row0, int kv0, const ae_attn_params& p) {{
  const int lane = threadIdx.x & 63; (void)lane; (void)row0; (void)kv0;
{body}
}}
#if AE_KV_COALESCED
// the tile fetched ahead goes from the coalesced layout to the lanes that own its elements, through 2560 bytes of
// LDS that belong to this wave alone (a wave's LDS operations complete in order: no wait between its writes and reads)
AE_DEV void ae_stage_custom(ae_custom& cust, __attribute__((address_space(3))) unsigned char* scratch) {{
  const int lane = threadIdx.x & 63;
{stage_body}
}}
#endif
#endif
"""
    return f"""// generated by core/lower/lower.py -- do not edit
{MASK_HELPERS}
#ifndef AE_KV_PF_GROUPS
#define AE_KV_PF_GROUPS 0      // kernels that fetch per-score custom inputs a tile ahead define it before this header
#endif
#ifndef AE_KV_COALESCED
#define AE_KV_COALESCED 0      // ... and 1 if they also hand ae_stage_custom a wave-private LDS scratch
#endif
struct ae_custom {{
{cfields}
}};
AE_DEV void ae_load_custom(ae_custom& c, const ae_attn_params& p, const ae_ctx& ctx) {{
{cloads}
}}
{prefetch}struct ae_rowstate {{
{fields}
}};
AE_DEV void ae_rowstate_init(ae_rowstate& st) {{
{inits}
}}
AE_DEV bool ae_mask_mod(int b, int h, int q_idx, int kv_idx) {{
{mask_body}
}}
template <int N>
AE_DEV void ae_score_mod(float (&s)[N], const ae_ctx& ctx, const ae_custom& cust) {{
{lf.score_mod_body}
}}
template <int N>
AE_DEV float ae_online_fwd(float (&s)[N], ae_rowstate& st, const ae_ctx& ctx, const ae_custom& cust) {{
{lf.online_fwd_body}
  return {lf.online_fwd_return};
}}
template <int N>
AE_DEV void ae_epilogue(float (&o)[N], ae_rowstate& st, float (&frs)[{nrs}], const ae_ctx& ctx,
                        const ae_custom& cust) {{
{lf.epilogue_body}
}}
"""


@dataclass
class PrefillTiles:
    """Tile configuration of a prefill template: ``choose_prefill_tiles`` fixes it per head dim and problem size
    from measurements; engines built with ``tune=True`` measure the candidates of core/lower/tuner.py instead."""
    template: str = "ae_prefill.hip"   # direct-to-LDS kernel
    n_waves: int = 4
    block_n: int = 64
    waves_per_eu: int = 2
    k_pad: int = 0
    v_pad: int = 0
    rows_per_wave: int = 32
    kv_stages: int = 2                 # K / V tile stages in LDS (AE_KV_STAGES of the pipelined kernel: 2 or 3)

    @property
    def block_m(self):
        return self.rows_per_wave * self.n_waves

    def lds_bytes(self, d: int, dv: int) -> int:
        stages = self.kv_stages * self.block_n * ((2 * d + self.k_pad) + (2 * dv + self.v_pad))
        if self.template == "ae_prefill_pipe.hip":
            # behind the tile stages every wave has room for its 64 Q rows (later its 64 O rows), which travel
            # through LDS as whole rows (AE_QO_BYTES of the kernel)
            stages += self.n_waves * 64 * 2 * max(d, dv)
        return stages


# Compute units of an MI355X: the pipelined kernel's 256-row tiles are only chosen when there are
# enough of them to occupy the chip.
_MI355X_CUS = 256


# Head dims the direct-to-LDS kernel (ae_prefill.hip) is written for: its K rows are swizzled for lengths of
# 2^n, 4*odd or 8*odd 16-byte chunks, its V rows for powers of two.
DIRECT_D = (64, 96, 128, 160, 192, 256)
DIRECT_DV = (64, 128, 256, 512)


def direct_tile_ok(d: int, dv: int, block_n: int, n_waves: int = 4) -> bool:
    """A K / V tile of block_n rows is fetched as whole 16-byte chunks, the same number per lane, at most eight
    a wave and tile (one burst of direct loads)."""
    nt = 64 * n_waves
    return all((block_n * x // 8) % nt == 0 and (block_n * x // 8) // nt <= 8 for x in (d, dv))


PIPE_KV_STAGES = 2      # default number of K / V stages of the pipelined kernel (AE_PIPE_STAGES=2|3 overrides)


def pipelined_tiles(d: int, dv: int) -> PrefillTiles:
    """The software-pipelined kernel's tile configuration: 256-row q tiles, one wave per SIMD, and as many K / V
    stages as asked for while they fit the 160 KiB of LDS beside the waves' Q / O rows."""
    stages = int(os.environ.get("AE_PIPE_STAGES", "") or PIPE_KV_STAGES)
    t = PrefillTiles(template="ae_prefill_pipe.hip", waves_per_eu=1, rows_per_wave=64, kv_stages=stages)
    if stages != 2 and t.lds_bytes(d, dv) > 160 * 1024:
        t.kv_stages = 2
    return t


def choose_prefill_tiles(d: int, dv: int, seqlen_q: int = 0, softmax=None, batch_heads: int = 0,
                         elementwise: bool = False, seqlen_kv: int = 0) -> PrefillTiles:
    """The direct-to-LDS kernels handle head dims 64 and 128 (and, the generic one, 96, 160, 192, 256 and value
    head dims up to 512, with one wave per SIMD where the accumulators need it): the
    software-pipelined one (64 rows per wave, 256-row q tiles, one wave per SIMD) when the graph is
    the online softmax of scaled scores, or elementwise (out = sum f(s) v: the kernel then calls the
    generated functor), and the problem has enough q tiles to occupy the chip
    (measured on B2 H32 S4096 D128 fp16: 1.0 against 0.86 PFLOP/s non-causal) and its rows are long enough
    for the pipeline to pay (short sequences are bound by the Q / O traffic and the start-up of a workgroup,
    which two workgroups per CU hide better: 16k tokens fp16 H32, S256 D128 0.136 against 0.162 ms, S512
    D64 causal 0.085 against 0.111 ms; from S1024 D128 / S2048 D64 on the pipelined kernel wins), otherwise
    the generic one (32 rows per wave, two waves per SIMD, runs any functor).  Other head dims use the
    register-staged kernel with padded LDS rows (ae_prefill_simple.hip), with one wave per SIMD and a
    shorter kv tile once the accumulators outgrow 256 registers.  AE_PREFILL_KERNEL=generic|pipelined
    overrides the choice between the first two (tests)."""
    if d in DIRECT_D and dv in DIRECT_DV and (d > 128 or dv > 128):
        if d <= 192 and dv <= 128:
            # head dims 160 / 192 with up to 128 value columns (192 / 128: multi-head latent attention before its
            # absorption): the wave still fits 256 registers, two waves per SIMD; 32-key tiles where two workgroups
            # with 64-key tiles would not fit the LDS of a compute unit
            return PrefillTiles(block_n=64 if direct_tile_ok(d, dv, 64) and d <= 160 else 32)
        # wide heads in the direct-to-LDS kernel: the accumulators of 32 rows (up to 256 registers for 512
        # value columns) and the Q fragments take one wave per SIMD; 64-key tiles while a wave's share of
        # a tile fits one burst of eight loads, else 32
        return PrefillTiles(waves_per_eu=1, block_n=64 if dv <= 256 and direct_tile_ok(d, dv, 64) else 32)
    if d in DIRECT_D and dv in DIRECT_DV:
        force = os.environ.get("AE_PREFILL_KERNEL", "")
        n_tiles = batch_heads * ((seqlen_q + 255) // 256)
        # (elementwise graphs at head dim 64 have too little matrix work per score for the pipelined kernel's
        # one wave per SIMD to pay: relu attention B64 H6 S2048 D64 0.48 ms against 0.45 ms in the generic one)
        fits = softmax is not None or (elementwise and max(d, dv) > 64)
        if seqlen_kv and seqlen_kv * max(d, dv) < 1024 * 128:
            fits = False
        if d in (64, 128) and (softmax is not None or elementwise) and force != "generic" and (
                force == "pipelined" or (fits and n_tiles >= (3 * _MI355X_CUS) // 4)):
            return pipelined_tiles(d, dv)
        return PrefillTiles()
    t = PrefillTiles(template="ae_prefill_simple.hip", k_pad=16)
    if max(d, dv) > 128:
        t.block_n, t.waves_per_eu = 32, 1
    # the workgroup copies K and V tiles as 16-byte chunks, a whole number per thread: take the
    # preferred kv tile if it divides, else the other one, else two waves instead of four
    for n_waves, block_n in ((4, t.block_n), (4, 96 - t.block_n), (2, t.block_n), (2, 96 - t.block_n)):
        nt = 64 * n_waves
        if (block_n * d // 8) % nt == 0 and (block_n * dv // 8) % nt == 0:
            t.n_waves, t.block_n = n_waves, block_n
            break
    else:
        raise NotImplementedError(f"no tile shape for head dims D={d}, DV={dv}")
    # V rows must land on distinct LDS bank groups for the transpose reads: pitch = 64 mod 256
    t.v_pad = (64 - (2 * dv) % 256) % 256
    if t.v_pad == 0:
        t.v_pad = 256
    return t


def render_config(d: int, dv: int, dtype, tiles: PrefillTiles, mask_mode: int, has_mask_mod: bool,
                  n_rowscales: int, o_scale_one: bool, even_q: bool, even_kv: bool, softmax=None,
                  elementwise: bool = False, exact_scale=None) -> str:
    """Text of ae_config.h.  ``softmax`` / ``elementwise`` say what the software-pipelined kernel does with a
    score (AE_PIPE_KIND 0: its built-in online softmax; 1: the generated functor); other kernels ignore them.
    ``exact_scale`` (None: the kernel's default, unless AE_PREFILL_PRESCALE is in the environment): True builds the
    pipelined fp16 softmax kernel WITHOUT the score scale folded into its Q fragments."""
    extra = []
    if softmax is None and elementwise:
        extra = ["#define AE_PIPE_KIND 1"]
    if softmax is not None:
        extra = [f"#define AE_SM_SCALE {float_literal(softmax[0])}", f"#define AE_SM_M {softmax[1]}",
                 f"#define AE_SM_R {softmax[2]}"]
        # The pipelined kernel folds the score scale into its fp16 Q fragments (one rounding of q*c*log2e
        # to fp16: a score moves by about 2^-12 of its size, i.e. lse by < 1e-3 while |score*c| stays below
        # ~20).  exact_scale=True (AE_PREFILL_PRESCALE=0) keeps Q as it is and multiplies every score in fp32 instead.
        if exact_scale is not None:
            extra.append(f"#define AE_PRESCALE {0 if exact_scale else 1}")
        elif os.environ.get("AE_PREFILL_PRESCALE", "") in ("0", "1"):
            extra.append(f"#define AE_PRESCALE {os.environ['AE_PREFILL_PRESCALE']}")
    return "\n".join([
        "// generated by core/lower/lower.py -- do not edit",
        f"#define AE_D {d}",
        f"#define AE_DV {dv}",
        f"#define AE_BN {tiles.block_n}",
        f"#define AE_NWAVES {tiles.n_waves}",
        f"#define AE_DTYPE_BF16 {1 if dtype == torch.bfloat16 else 0}",
        f"#define AE_MASK_MODE {mask_mode}",
        f"#define AE_HAS_MASK_MOD {1 if has_mask_mod else 0}",
        f"#define AE_N_ROWSCALES {n_rowscales}",
        f"#define AE_O_SCALE_ONE {1 if o_scale_one else 0}",
        f"#define AE_EVEN_Q {1 if even_q else 0}",
        f"#define AE_EVEN_KV {1 if even_kv else 0}",
        f"#define AE_WAVES_PER_EU {tiles.waves_per_eu}",
        f"#define AE_K_PAD {tiles.k_pad}",
        f"#define AE_V_PAD {tiles.v_pad}",
        *([f"#define AE_KV_STAGES {tiles.kv_stages}"] if tiles.template == "ae_prefill_pipe.hip" else []),
        # (measurement switch of the pipelined kernel: the order of a causal launch's workgroups)
        *([f"#define AE_CAUSAL_ORDER {os.environ['AE_CAUSAL_ORDER']}"]
          if tiles.template == "ae_prefill_pipe.hip" and os.environ.get("AE_CAUSAL_ORDER", "") in ("0", "1") else []),
        *extra,
        "",
    ])
