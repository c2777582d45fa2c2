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

Two rewrites keep the per-element instruction count of the common graphs at its minimum:
  * affine folding: ``x * c``, ``x + y``, ``x - y``, ``-x`` with a constant c and a per-row y are
    carried symbolically as ``base[e] * mul + add`` and only materialised where a non-affine
    consumer needs them.  ``exp`` consumes the affine form as one fma + exp2 per element (the
    per-row part ``add * log2e`` is hoisted) and ``ReduceMax`` as ``rowmax(base) * mul + add`` for
    mul > 0, so ``softmax(scale * s)`` costs no multiply by the scale at all;
  * lazy running maximum (``lazy_max``): where the lowering has proved that the graph is the online
    softmax (results invariant under the choice of the reference point m), the update
    ``m_new = max(m, x)`` becomes ``m_new = (x > m + tau) ? x : m``.  The exponentials then stay
    below e^tau, the running sum and the output are rescaled only when a row's maximum grows by
    more than tau, and the kernels skip the rescale of the accumulator when o_scale == 1.
"""
from __future__ import annotations

import math

LOG2E = 1.4426950408889634

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
        self.affine = {}  # id(symbol) -> (base array expr, mul: float, add: scalar expr or None)
        self.lazy_max = {}  # id(Max symbol) -> tau: emit the thresholded update
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
    def _value_plain(self, sym: SymbolScalar):
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

    # ---- affine forms -------------------------------------------------------------------
    def _as_affine(self, sym: SymbolScalar):
        """(base, mul, add) if ``sym`` is an array that can be carried as base[e]*mul + add."""
        key = id(sym)
        if key in self.affine:
            return self.affine[key]
        if key in self.done:
            expr, is_arr = self.done[key]
            return (expr, 1.0, None) if is_arr else None
        if not self._is_array(sym):
            return None
        t = sym.code.type
        if key in self.leaves or t in ("Var", "Const") or not sym.prev:
            expr, is_arr = self.value(sym)
            return (expr, 1.0, None) if is_arr else None
        aff = None
        if t in ("Mul", "Div") and len(sym.prev) == 2:
            a, b = sym.prev
            ca = a.code.value if a.code.type == "Const" else None
            cb = b.code.value if b.code.type == "Const" else None
            if cb is not None and (t == "Mul" or float(cb) != 0.0):
                inner = self._as_affine(a)
                if inner is not None:
                    f = float(cb) if t == "Mul" else 1.0 / float(cb)
                    aff = self._scale(inner, f)
            elif ca is not None and t == "Mul":
                inner = self._as_affine(b)
                if inner is not None:
                    aff = self._scale(inner, float(ca))
        elif t in ("Add", "Sub") and len(sym.prev) == 2:
            a, b = sym.prev
            if self._is_array(a) and not self._is_array(b):
                inner = self._as_affine(a)
                if inner is not None:
                    y = self.value(b)[0]
                    aff = (inner[0], inner[1], self._sum(inner[2], y, "+" if t == "Add" else "-"))
            elif t == "Add" and self._is_array(b) and not self._is_array(a):
                inner = self._as_affine(b)
                if inner is not None:
                    aff = (inner[0], inner[1], self._sum(inner[2], self.value(a)[0], "+"))
            elif t == "Sub" and self._is_array(b) and not self._is_array(a):
                inner = self._as_affine(b)
                if inner is not None:
                    neg = self._scale(inner, -1.0)
                    aff = (neg[0], neg[1], self._sum(neg[2], self.value(a)[0], "+"))
        elif t == "Neg":
            inner = self._as_affine(sym.prev[0])
            if inner is not None:
                aff = self._scale(inner, -1.0)
        if aff is not None:
            self.affine[key] = aff
            self._keep.append(sym)
        return aff

    def _scale(self, aff, f: float):
        base, mul, add = aff
        if add is not None:
            t = self._tmp()
            self.lines.append(f"const float {t} = ({add}) * {float_literal(f)};")
            add = t
        return (base, mul * f, add)

    def _sum(self, add, y: str, op: str):
        t = self._tmp()
        if add is None:
            self.lines.append(f"const float {t} = {'' if op == '+' else '-'}({y});")
        else:
            self.lines.append(f"const float {t} = ({add}) {op} ({y});")
        return t

    def _materialise(self, sym: SymbolScalar):
        """Array temp holding the value of an affine symbol."""
        base, mul, add = self.affine[id(sym)]
        out = self._tmp()
        self.lines.append(f"float {out}[{self.n}];")
        if add is None:
            self._loop(f"{out}[e] = {base}[e] * {float_literal(mul)};")
        else:
            self._loop(f"{out}[e] = __builtin_fmaf({base}[e], {float_literal(mul)}, {add});")
        return (out, True)

    # ---- a * tanh(x) + b ----------------------------------------------------------------
    def _affine_of_tanh(self, sym: SymbolScalar):
        """(tanh symbol, a, b) if ``sym`` is a*tanh(x) + b built from Mul/Div/Add/Sub/Neg with literal
        constants, x an array; None otherwise."""
        a, b = 1.0, 0.0
        cur = sym
        while True:
            t = cur.code.type
            if t == "Tanh":
                return (cur, a, b) if self._is_array(cur.prev[0]) and cur is not sym else None
            if id(cur) in self.done or id(cur) in self.leaves or not cur.prev:
                return None
            if t == "Neg":
                a, cur = -a, cur.prev[0]
                continue
            if t not in ("Mul", "Div", "Add", "Sub") or len(cur.prev) != 2:
                return None
            x, y = cur.prev
            cx = float(x.code.value) if x.code.type == "Const" else None
            cy = float(y.code.value) if y.code.type == "Const" else None
            if cy is not None and cx is None:
                if t == "Mul":
                    a, b = a, b          # out = a*(inner*cy)+b
                    a *= cy
                elif t == "Div":
                    if cy == 0.0:
                        return None
                    a /= cy
                elif t == "Add":
                    b += a * cy
                else:
                    b -= a * cy
                cur = x
            elif cx is not None and cy is None:
                if t == "Mul":
                    a *= cx
                elif t == "Add":
                    b += a * cx
                elif t == "Sub":     # cx - inner
                    b += a * cx
                    a = -a
                else:
                    return None
                cur = y
            else:
                return None

    def _emit_affine_of_tanh(self, sym, tanh_sym, a: float, b: float):
        """a*tanh(x)+b = (a+b) - 2a / (exp(2x) + 1): one exponential and one reciprocal per element,
        with x's own affine form folded into the exponent.  a = b = 1/2 is the logistic function
        1 / (1 + exp(-2x)) (attn_script/sigmoidattn.py:14-18 writes sigmoid this way)."""
        arg = tanh_sym.prev[0]
        aff = self._as_affine(arg)
        if aff is None:
            base, mul, add = self.value(arg)[0], 1.0, None
        else:
            base, mul, add = aff
        logistic = abs(a - 0.5) < 1e-12 and abs(b - 0.5) < 1e-12
        k = (-2.0 if logistic else 2.0) * mul * LOG2E
        if add is None:
            ex = f"ae_exp2({base}[e] * {float_literal(k)})"
        else:
            hoist = self._tmp()
            self.lines.append(f"const float {hoist} = ({add}) * {float_literal((-2.0 if logistic else 2.0) * LOG2E)};")
            ex = f"ae_exp2(__builtin_fmaf({base}[e], {float_literal(k)}, {hoist}))"
        out = self._tmp()
        self.lines.append(f"float {out}[{self.n}];")
        if logistic:
            self._loop(f"{out}[e] = ae_rcp(1.0f + {ex});")
        else:
            self._loop(f"{out}[e] = __builtin_fmaf(ae_rcp({ex} + 1.0f), {float_literal(-2.0 * a)}, {float_literal(a + b)});")
        return (out, True)

    def value(self, sym: SymbolScalar):  # noqa: F811  (affine-aware front end of the graph walk)
        key = id(sym)
        if key in self.done:
            return self.done[key]
        if self._is_array(sym) and sym.code.type in ("Mul", "Div", "Add", "Sub", "Neg") and sym.prev:
            ft = self._affine_of_tanh(sym)
            if ft is not None:
                val = self._emit_affine_of_tanh(sym, *ft)
                self.done[key] = val
                self._keep.append(sym)
                return val
        if self._is_array(sym) and sym.code.type in ("Mul", "Div", "Add", "Sub", "Neg") and sym.prev:
            aff = self._as_affine(sym)
            if aff is not None and key in self.affine:
                if aff[1] == 1.0 and aff[2] is None:
                    val = (aff[0], True)
                else:
                    val = self._materialise(sym)
                self.done[key] = val
                return val
        return self._value_plain(sym)

    def _emit_op(self, sym: SymbolScalar):
        t = sym.code.type
        if t in ("Exp", "Exp2") and self._is_array(sym.prev[0]):
            aff = self._as_affine(sym.prev[0])
            if aff is not None and not (aff[1] == 1.0 and aff[2] is None):
                base, mul, add = aff
                k = mul * (LOG2E if t == "Exp" else 1.0)
                out = self._tmp()
                if add is None:
                    body = f"ae_exp2({base}[e] * {float_literal(k)})"
                else:
                    hoist = self._tmp()
                    scale = " * AE_LOG2E" if t == "Exp" else ""
                    self.lines.append(f"const float {hoist} = ({add}){scale};")
                    body = f"ae_exp2(__builtin_fmaf({base}[e], {float_literal(k)}, {hoist}))"
                self.lines.append(f"float {out}[{self.n}];")
                self._loop(f"{out}[e] = {body};")
                return (out, True)
        if t == "ReduceMax" and not self.split_axis and self._is_array(sym.prev[0]):
            aff = self._as_affine(sym.prev[0])
            if aff is not None and aff[1] > 0.0 and not (aff[1] == 1.0 and aff[2] is None):
                base, mul, add = aff
                out = self._tmp()
                tail = f" + ({add})" if add is not None else ""
                self.lines.append(f"const float {out} = ae_row_max<{self.n}>({base}) * {float_literal(mul)}{tail};")
                return (out, False)
        if t == "Max" and id(sym) in self.lazy_max:
            m_val = self.value(sym.prev[0])[0]
            x_val = self.value(sym.prev[1])[0]
            out = self._tmp()
            tau = float_literal(self.lazy_max[id(sym)])
            self.lines.append(f"const float {out} = (({x_val}) - ({m_val}) > {tau}) ? ({x_val}) : ({m_val});")
            return (out, False)
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
            # gradient g of max(x, y) with respect to x: passes where x won (zero at a tie)
            is_arr = any(a for _, a in ins)
            expr = f"({self._at(ins[1])} > {self._at(ins[2])} ? {self._at(ins[0])} : 0.0f)"
            if is_arr:
                self.lines.append(f"float {out}[{self.n}];")
                self._loop(f"{out}[e] = {expr};")
            else:
                self.lines.append(f"const float {out} = {expr};")
            return (out, is_arr)
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
