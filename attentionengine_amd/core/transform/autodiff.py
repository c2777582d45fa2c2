"""Symbolic derivative of a traced elementwise graph with respect to one of its leaves.

Role of ``SymbolScalar.backward`` / ``_backward`` in attention_engine/core/transform/core.py:119-199,
which the reference uses to turn ``score_mod`` into ``score_mod_backward`` (core/lower/lower.py:
lower_score_mod).  Reverse mode over the node types the tracer has; the result is again a traced
expression, so the same emitter prints it.  ``max(a, b)`` passes the gradient to ``a`` where ``a > b``
(``MaxBwd``; zero at a tie, the convention of relu).
"""
from __future__ import annotations

from .core import SymbolScalar, SymbolicConst


def _topo(root):
    order, seen = [], set()

    def visit(s):
        if id(s) in seen:
            return
        seen.add(id(s))
        for x in s.prev:
            visit(x)
        order.append(s)
    visit(root)
    return order


def _reverse(out: SymbolScalar, seed: SymbolScalar, wrt):
    """Reverse sweep from ``out`` seeded with ``seed``: {id(symbol): gradient expression} for the symbols on
    a path from ``out`` to one of ``wrt`` (to any leaf when ``wrt`` is None)."""
    order = _topo(out)
    if wrt is None:
        depends = {id(s) for s in order}
    else:
        depends = {id(w) for w in wrt}
        for s in order:
            if any(id(x) in depends for x in s.prev):
                depends.add(id(s))
    if id(out) not in depends:
        return {}, order
    grads = {id(out): seed}

    def add(sym, g):
        if id(sym) not in depends:
            return
        grads[id(sym)] = g if id(sym) not in grads else grads[id(sym)] + g

    for s in reversed(order):
        g = grads.get(id(s))
        if g is None or not s.prev or id(s) not in depends:
            continue
        t = s.code.type
        a = s.prev[0]
        b = s.prev[1] if len(s.prev) > 1 else None
        if t == "Add":
            add(a, g)
            add(b, g)
        elif t == "Sub":
            add(a, g)
            add(b, -g)
        elif t == "Mul":
            add(a, g * b)
            add(b, g * a)
        elif t == "Div":
            add(a, g / b)
            add(b, -(g * s) / b)
        elif t == "Neg":
            add(a, -g)
        elif t == "Abs":
            add(a, g.maxbwd(a, SymbolicConst(0.0)) - g.maxbwd(-a, SymbolicConst(0.0)))
        elif t == "Tanh":
            add(a, g - g * s * s)
        elif t == "Exp":
            add(a, g * s)
        elif t == "Exp2":
            add(a, g * s * 0.6931471805599453)
        elif t == "Log":
            add(a, g / a)
        elif t == "Log2":
            add(a, g / (a * 0.6931471805599453))
        elif t == "Max":
            add(a, g.maxbwd(a, b))
            add(b, g.maxbwd(b, a))
        else:
            raise NotImplementedError(f"derivative of {t}")
    return grads, order


def derivative(out: SymbolScalar, wrt: SymbolScalar) -> SymbolScalar:
    """d out / d wrt as a traced expression (a constant 0 if ``out`` does not depend on ``wrt``)."""
    grads, _ = _reverse(out, SymbolicConst(1.0), [wrt])
    return grads.get(id(wrt), SymbolicConst(0.0))


def backward(out: SymbolScalar, grad=None) -> None:
    """``out.backward(grad)`` of the reference (core/transform/core.py:119-199): leave on every symbol the
    output was computed from its gradient expression in ``.grad`` (``grad`` times d out / d symbol; ``grad``
    defaults to 1).  Symbols that ``out`` reaches on several paths get the sum."""
    seed = SymbolicConst(1.0) if grad is None else grad
    grads, order = _reverse(out, seed, None)
    for sym in order:
        if id(sym) in grads:
            sym.grad = grads[id(sym)]
