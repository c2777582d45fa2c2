"""Expression-node vocabulary of the symbolic frontend.

Same public names and ``type`` strings as the reference's
attention_engine/core/transform/graph.py:2-243 (Var, Const, Add, Mul, Neg, Sub, Div, Exp, Exp2,
Log, Log2, Tanh, Abs, Max, MaxBwd, ReduceSum, ReduceMax, ReduceAbsSum, ColReduceMax,
ColReduceSum, ColReduceAbsSum).  The HIP functor emitter and the CPU interpreter dispatch on
``Node.type``.  The reference's per-node ``_backward`` rules (graph.py:2-243, driven by
SymbolScalar.backward, core.py:119-199) are replaced by one function,
core.transform.autodiff.derivative, which returns the derivative as a traced expression.
"""


class Node:
    """An operation applied to ``inputs`` (other nodes)."""

    def __init__(self, type: str, inputs=()):
        self.type = type
        self.inputs = list(inputs)
        self.grad = None

    def backward(self, grad=None):
        raise NotImplementedError("use core.transform.autodiff.derivative(out, wrt): the derivative as a traced expression")

    def __str__(self):
        return f"{self.type}(" + "".join(f"{n}, " for n in self.inputs) + ")"

    __repr__ = __str__


class Var(Node):
    """A named leaf.  The name doubles as the initial value of an online rowscale
    ("-inf", "0.0", "1", ...), see attn_script/mha.py:33-36."""

    def __init__(self, name: str):
        super().__init__("Var")
        self.name = name

    def __str__(self):
        return f'Var("{self.name}")'


class Const(Node):
    """A python number captured while tracing."""

    def __init__(self, value: float):
        super().__init__("Const")
        self.value = value

    def __str__(self):
        return f"Const({self.value})"


def _make_op(name: str, arity: int):
    def __init__(self, *operands):
        if len(operands) != arity:
            raise TypeError(f"{name} takes {arity} operand(s), got {len(operands)}")
        Node.__init__(self, name, operands)

    return type(name, (Node,), {"__init__": __init__, "__doc__": f"{name} node ({arity} operand(s))."})


# binary elementwise
Add = _make_op("Add", 2)
Sub = _make_op("Sub", 2)
Mul = _make_op("Mul", 2)
Div = _make_op("Div", 2)
Max = _make_op("Max", 2)
# unary elementwise
Neg = _make_op("Neg", 1)
Exp = _make_op("Exp", 1)
Exp2 = _make_op("Exp2", 1)
Log = _make_op("Log", 1)
Log2 = _make_op("Log2", 1)
Tanh = _make_op("Tanh", 1)
Abs = _make_op("Abs", 1)
# backward-only select: grad where left > right else 0 (core/codegen/tl_gen.py:122-125)
MaxBwd = _make_op("MaxBwd", 3)
# reductions over the kv axis of a [block_M, block_N] tile
ReduceSum = _make_op("ReduceSum", 1)
ReduceMax = _make_op("ReduceMax", 1)
ReduceAbsSum = _make_op("ReduceAbsSum", 1)
# reductions over the split axis of a [num_split, block_M] array (split-KV combine)
ColReduceMax = _make_op("ColReduceMax", 1)
ColReduceSum = _make_op("ColReduceSum", 1)
ColReduceAbsSum = _make_op("ColReduceAbsSum", 1)

ELEMENTWISE_UNARY = ("Neg", "Exp", "Exp2", "Log", "Log2", "Tanh", "Abs")
ELEMENTWISE_BINARY = ("Add", "Sub", "Mul", "Div", "Max")
ROW_REDUCTIONS = ("ReduceSum", "ReduceMax", "ReduceAbsSum")
COL_REDUCTIONS = ("ColReduceSum", "ColReduceMax", "ColReduceAbsSum")

__all__ = [
    "Node", "Var", "Const", "Add", "Sub", "Mul", "Div", "Max", "Neg", "Exp", "Exp2", "Log",
    "Log2", "Tanh", "Abs", "MaxBwd", "ReduceSum", "ReduceMax", "ReduceAbsSum", "ColReduceMax",
    "ColReduceSum", "ColReduceAbsSum",
]
