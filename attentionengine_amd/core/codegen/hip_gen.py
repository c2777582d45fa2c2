"""Traced expression graph -> HIP device statements.

This is the HIP counterpart of the reference's ``generate_tl_from_dag`` / ``to_tl_op``
(attention_engine/core/codegen/tl_gen.py:306-370, 7-132).  Operation semantics follow that
file: Exp is ``exp2(x * log2 e)`` (89-92), Log is ``log2(x) * ln 2`` (105-108), Tanh is a fast
approximation (113-117), row reductions reduce the kv axis of the score tile (9-21), operands
broadcast by shape name (44-62).

Register model.  In the kernels every lane owns ONE query row, so a value is either
  * "scalar": one float per lane  (constants, b/h/q_idx, online rowscales, row reductions), or
  * "array" : ``float x[N]`` over the lane's slice of the kv axis (score tile, kv_idx) or of
              the dv axis (the output accumulator in the epilogue).
A value is an array iff its ``shape_idx`` names one of the array axes given to the emitter.
All loops are fully unrolled, so the arrays live in VGPRs.
"""
from __future__ import annotations

import math

from ..transform.core import SymbolScalar
from ..transform.graph import COL_REDUCTIONS, ELEMENTWISE_BINARY, ELEMENTWISE_UNARY, ROW_REDUCTIONS

_INIT_WORDS = {"-inf": "-1e38f", "inf": "1e38f", "+inf": "1e38f"}


def float_literal(v) -> str:
    """C++ float literal of a python number (infinities become the finite sentinel the
    reference uses, core/lower/lower.py:23-29)."""
    v = float(v)
    if math.isinf(v):
        return "1e38f" if v > 0 else "-1e38f"
    if math.isnan(v):
        raise ValueError("NaN constant in traced graph")
    r = repr(v)
    if "e" not in r and "." not in r:
        r += ".0"
    return r + "f"


def init_literal(name: str) -> str:
    """Initial value of an online rowscale declared as ``Var("<name>")``."""
    name = name.strip()
    if name in _INIT_WORDS:
        return _INIT_WORDS[name]
    try:
        return float_literal(float(name))
    except ValueError:
        raise NotImplementedError(f"unsupported rowscale initial value {name!r}") from None


def var_as_constant(sym: SymbolScalar):
    """A leaf ``Var`` that denotes a number: ``Var("1")``, ``Var("0.0")``, ``Var("-inf")`` or the
    base class's ``Var("o_scale")`` placeholder, whose buffer the reference pre-fills with 1.0
    (attn_tl.py:108).  Returns the python float or None."""
    if sym.code.type != "Var" or sym.prev:
        return None
    name = sym.code.name.strip()
    if name == "o_scale":
        return 1.0
    if name in ("-inf",):
        return -math.inf
    if name in ("inf", "+inf"):
        return math.inf
    try:
        return float(name)
    except ValueError:
        return None


class Emitter:
    """Emits one functor body.

    ``leaves`` maps ``id(symbol)`` -> (expression, is_array); ``named_leaves`` maps a ``Var`` name
    to the same pair for symbols the user created by name.  ``array_axes`` are the shape names
    that make a value an array; ``n`` is the C++ expression of the array length.
    """

    def __init__(self, leaves: dict, named_leaves: dict, array_axes, n: str = "N", prefix: str = "t",
                 split_axis: bool = False):
        # split_axis: the array axis is the split axis of OnlineFunc.combine, reduced by ColReduce*
        self.split_axis = split_axis
        self.leaves = leaves
        self.named_leaves = named_leaves
        self.array_axes = set(str(a) for a in array_axes)
        self.n = n
        self.prefix = prefix
        self.lines = []
        self.done = {}   # id(symbol) -> (expr, is_array)
        self.counter = 0
        self._keep = []  # keep traced symbols alive so ids stay unique

    # ---- helpers ----------------------------------------------------------------------
    def _tmp(self):
        self.counter += 1
        return f"{self.prefix}{self.counter}"

    def _is_array(self, sym: SymbolScalar) -> bool:
        return any(s in self.array_axes for s in sym.shape_idx)

    def _loop(self, body: str):
        self.lines.append("#pragma unroll")
        self.lines.append(f"for (int e = 0; e < {self.n}; e++) {body}")

    @staticmethod
    def _at(val):
        expr, is_arr = val
        return f"{expr}[e]" if is_arr else expr

    # ---- graph walk ---------------------------------------------------------------------
    def value(self, sym: SymbolScalar):
        """(expression, is_array) of ``sym``, emitting whatever it depends on first."""
        key = id(sym)
        if key in self.done:
            return self.done[key]
        self._keep.append(sym)
        if key in self.leaves:
            val = self.leaves[key]
        elif sym.code.type == "Const":
            val = (float_literal(sym.code.value), False)
        elif sym.code.type == "Var" and not sym.prev:
            c = var_as_constant(sym)
            if c is not None:
                val = (float_literal(c), False)
            elif sym.code.name in self.named_leaves:
                val = self.named_leaves[sym.code.name]
            else:
                raise NotImplementedError(f"unknown input {sym.code.name!r} in traced function")
        else:
            val = self._emit_op(sym)
        self.done[key] = val
        return val

    def _emit_op(self, sym: SymbolScalar):
        t = sym.code.type
        if t == "Exp":
            fused = self._emit_exp_of_difference(sym)
            if fused is not None:
                return fused
        ins = [self.value(p) for p in sym.prev]
        out = self._tmp()
        if t in ROW_REDUCTIONS:
            if self.split_axis:
                raise NotImplementedError(f"{t} inside OnlineFunc.combine (use the column reductions)")
            src, is_arr = ins[0]
            if not is_arr:
                raise NotImplementedError(f"{t} of a value that has no kv axis")
            fn = {"ReduceSum": "ae_row_sum", "ReduceMax": "ae_row_max", "ReduceAbsSum": "ae_row_abssum"}[t]
            self.lines.append(f"const float {out} = {fn}<{self.n}>({src});")
            return (out, False)
        if t in COL_REDUCTIONS:
            if not self.split_axis:
                raise NotImplementedError(f"{t} is only meaningful inside OnlineFunc.combine")
            src, is_arr = ins[0]
            if not is_arr:
                raise NotImplementedError(f"{t} of a value that has no split axis")
            fn = {"ColReduceSum": "ae_arr_sum", "ColReduceMax": "ae_arr_max",
                  "ColReduceAbsSum": "ae_arr_abssum"}[t]
            self.lines.append(f"const float {out} = {fn}<{self.n}>({src});")
            return (out, False)
        if t == "MaxBwd":
            raise NotImplementedError("MaxBwd belongs to the backward pass")
        if t not in ELEMENTWISE_UNARY and t not in ELEMENTWISE_BINARY:
            raise NotImplementedError(str(t))

        is_arr = any(a for _, a in ins)
        expr = self._elementwise(t, ins)
        if is_arr:
            self.lines.append(f"float {out}[{self.n}];")
            self._loop(f"{out}[e] = {expr};")
        else:
            self.lines.append(f"const float {out} = {expr};")
        return (out, is_arr)

    def _emit_exp_of_difference(self, sym: SymbolScalar):
        """exp(x - y) with an array x and a per-row y becomes one fma + exp2 per element:
        exp2(x*log2e + (-y*log2e)), the second term hoisted out of the loop."""
        src = sym.prev[0]
        if src.code.type != "Sub" or len(src.prev) != 2 or id(src) in self.done:
            return None
        if not self._is_array(src.prev[0]) or self._is_array(src.prev[1]):
            return None
        x = self.value(src.prev[0])
        y = self.value(src.prev[1])
        if not x[1] or y[1]:
            return None
        hoist, out = self._tmp(), self._tmp()
        self.lines.append(f"const float {hoist} = -({y[0]}) * AE_LOG2E;")
        self.lines.append(f"float {out}[{self.n}];")
        self._loop(f"{out}[e] = ae_exp2(__builtin_fmaf({x[0]}[e], AE_LOG2E, {hoist}));")
        return (out, True)

    def _elementwise(self, t: str, ins):
        a = self._at(ins[0])
        b = self._at(ins[1]) if len(ins) > 1 else None
        if t == "Add":
            return f"({a} + {b})"
        if t == "Sub":
            return f"({a} - {b})"
        if t == "Mul":
            return f"({a} * {b})"
        if t == "Div":
            return f"({a} / {b})"
        if t == "Max":
            return f"ae_max({a}, {b})"
        if t == "Neg":
            return f"(-{a})"
        if t == "Abs":
            return f"ae_abs({a})"
        if t == "Tanh":
            return f"ae_tanh({a})"
        if t == "Exp2":
            return f"ae_exp2({a})"
        if t == "Log":
            return f"ae_log({a})"
        if t == "Log2":
            return f"ae_log2({a})"
        if t == "Exp":
            return f"ae_exp({a})"
        raise NotImplementedError(t)

    def code(self, indent: str = "  ") -> str:
        return "\n".join(indent + ln for ln in self.lines)
