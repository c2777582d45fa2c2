"""Symbolic tracer and mask utilities of the frontend.

API-compatible with attention_engine/core/transform/core.py:
  SymbolScalar (36-250), SymbolicArray.get_reduce (253-278), SymbolicColReduceArray (280-304),
  SymbolicTensor (306-316), SymbolicConst (319-328), CustomIO (331-349), create_mask (352-398),
  _convert_mask_to_block_mask (410-453), is_causal_mask (455-470), is_less_causal_mask
  (472-488), create_block_mask (492-506), create_block_idx (508-512).

User callables (score_mod, OnlineFunc.online_fwd, ...) are traced by calling them on these
objects; every operation appends a node and returns a new symbol whose ``prev`` are its
operands.  The symbolic differentiation (119-199) lives in autodiff.py (``derivative``).
"""
from __future__ import annotations

from typing import Literal, Optional, Type

import torch

from .graph import *  # noqa: F401,F403  (the reference re-exports the node types from here)
from .graph import (Abs, Add, ColReduceAbsSum, ColReduceMax, ColReduceSum, Const, Div, Exp,
                    Exp2, Log, Log2, Max, MaxBwd, Mul, Neg, Node, ReduceAbsSum, ReduceMax,
                    ReduceSum, Sub, Tanh, Var)


_DIM_ORDER = {"num_split": 0, "block_M": 1, "seq_len": 1, "block_N": 2, "seq_len_kv": 2, "dimv": 2}


def _broadcast_shape(shapes):
    """Ordered union of dimension names; "1" entries are dropped when another dimension exists.
    Known names are ordered (split, row, column); unknown names keep their order of appearance."""
    dims = []
    for sh in shapes:
        for d in sh:
            if d != "1" and d not in dims:
                dims.append(d)
    if not dims:
        return ["1"] if any("1" in sh for sh in shapes) else []
    if all(d in _DIM_ORDER for d in dims):
        dims.sort(key=lambda d: _DIM_ORDER[d])
    return dims


class SymbolScalar:
    """A traced value: scalar per row (``shape_idx=["block_M"]``), a score tile
    (``["block_M","block_N"]``), a constant (``[]``) or a custom input tensor."""

    def __init__(self, varname: str, value: Node, prev=None, shape_idx=("block_M",),
                 require_grad: bool = True, dtype: str = "float"):
        self.varname = varname
        self.code = value
        self.prev = list(prev) if prev is not None else []
        self.shape_idx = [str(i) for i in shape_idx]
        self.require_grad = require_grad
        self.dtype = dtype
        # bookkeeping the reference's code generator relies on (use counts, reuse hints)
        self.count = 0
        self.use_list = []
        self.allow_reuse = True
        self.lowered = False
        self.visit_count = 0
        self.grad = None

    # -- introspection -----------------------------------------------------------------
    def __repr__(self):
        return (f"SymbolScalar({self.varname}, {self.code}, {self.prev}, {self.shape_idx}, "
                f"{self.require_grad}, {self.dtype})")

    @property
    def name(self):
        return self.varname

    @property
    def shape(self):
        import sympy
        return [sympy.simplify(s) for s in self.shape_idx]

    def set_allow_reuse(self, allow_reuse: bool):
        self.allow_reuse = allow_reuse

    def clear_usecount(self):
        self.count = 0
        self.use_list.clear()

    def clear_visit(self):
        self.visit_count = 0
        self.lowered = False

    def clear_codegen(self):
        self.clear_usecount()
        self.clear_visit()

    # -- tracing -------------------------------------------------------------------------
    def op(self, code: Type[Node], others=None, shape_idx=None, varname_suffix: str = None):
        """Apply node type ``code`` to ``self`` and ``others``; python numbers become
        constants.  Result name: ``<varname>[_<suffix>]_<use count of self>``."""
        operands = []
        for other in (others or []):
            if isinstance(other, (int, float)) and not isinstance(other, bool):
                other = SymbolicConst(other)
            elif not isinstance(other, SymbolScalar):
                raise TypeError(f"cannot trace operand of type {type(other).__name__}")
            operands.append(other)
        if shape_idx is None:
            # elementwise result broadcasts by dimension NAME (core/codegen/tl_gen.py:44-62):
            # ordered union of the operands' dimensions, e.g. [block_M] op [block_N] -> tile
            shape_idx = _broadcast_shape([self.shape_idx] + [o.shape_idx for o in operands])
        stem = self.varname if varname_suffix is None else f"{self.varname}_{varname_suffix}"
        node = code(*[x.code for x in [self] + operands])
        out = self.__class__.__new__(self.__class__)
        SymbolScalar.__init__(out, f"{stem}_{self.count}", node, [self] + operands, shape_idx)
        for x in [self] + operands:
            x.use_list.append(out)
            x.count += 1
        return out

    def backward(self, grad=None):
        """Symbolic reverse-mode differentiation (core/transform/core.py:119-199 of the reference): after the
        call every symbol this one was computed from carries its gradient expression in ``.grad``."""
        from .autodiff import backward as _backward
        _backward(self, grad)

    def __add__(self, other):
        return self.op(Add, [other])

    def __sub__(self, other):
        return self.op(Sub, [other])

    def __mul__(self, other):
        return self.op(Mul, [other])

    def __truediv__(self, other):
        return self.op(Div, [other])

    def __neg__(self):
        return self.op(Neg)

    # python number on the left (the reference only supports `x + 1`, not `1 + x`)
    def __radd__(self, other):
        return SymbolicConst(other).op(Add, [self])

    def __rsub__(self, other):
        return SymbolicConst(other).op(Sub, [self])

    def __rmul__(self, other):
        return SymbolicConst(other).op(Mul, [self])

    def __rtruediv__(self, other):
        return SymbolicConst(other).op(Div, [self])

    def abs(self):
        return self.op(Abs)

    def tanh(self):
        return self.op(Tanh)

    def exp(self):
        return self.op(Exp)

    def exp2(self):
        return self.op(Exp2)

    def log(self):
        return self.op(Log)

    def log2(self):
        return self.op(Log2)

    def max(self, other):
        return self.op(Max, [other])

    def maxbwd(self, other1, other2):
        return self.op(MaxBwd, [other1, other2])


_ROW_REDUCE = {"sum": ReduceSum, "max": ReduceMax, "abssum": ReduceAbsSum}
_COL_REDUCE = {"sum": ColReduceSum, "max": ColReduceMax, "abssum": ColReduceAbsSum}


class SymbolicArray(SymbolScalar):
    """Score tile ``[block_M, block_N]`` handed to ``OnlineFunc.online_fwd``."""

    def __init__(self, varname: str = "", code: Node = None, prev=None,
                 shape_idx=("block_M", "block_N")):
        super().__init__(varname, code if code is not None else Var(" "), prev, shape_idx)

    def get_reduce(self, op: Literal["sum", "max", "abssum"]):
        """Reduce over the kv axis (last dimension)."""
        if op not in _ROW_REDUCE:
            raise NotImplementedError(op)
        return self.op(_ROW_REDUCE[op], shape_idx=self.shape_idx[:-1], varname_suffix=op)


class SymbolicColReduceArray(SymbolScalar):
    """Per-split rowscale array ``[num_split, block_M]`` handed to ``OnlineFunc.combine``."""

    def __init__(self, varname: str = "", code: Node = None, prev=None,
                 shape_idx=("block_M", "block_N")):
        super().__init__(varname, code if code is not None else Var(" "), prev, shape_idx)

    def get_reduce(self, op: Literal["sum", "max", "abssum"]):
        """Reduce over the split axis (second to last dimension)."""
        if op not in _COL_REDUCE:
            raise NotImplementedError(op)
        shape_idx = self.shape_idx[:-2] + [self.shape_idx[-1]]
        return self.op(_COL_REDUCE[op], shape_idx=shape_idx, varname_suffix=op)


class SymbolicTensor(SymbolScalar):
    """A CustomIO input tensor; ``shape`` entries are ints or the symbolic names
    "batch", "heads", "seq_len", "seq_len_kv"."""

    def __init__(self, varname: str, shape: tuple):
        super().__init__(varname, Var(varname), shape_idx=[str(i) for i in shape])


class SymbolicConst(SymbolScalar):
    """A python number lifted into the graph (shape ``[]``)."""

    def __init__(self, value):
        super().__init__(f"float({value})", Const(value), prev=[], shape_idx=[], require_grad=False)


class CustomIO:
    """Named extra input tensors of a score_mod / OnlineFunc:
    ``CustomIO({"softmax_bias": (1,)})`` (attn_script/sigmoidattn.py:51-53)."""

    def __init__(self, input_tensors: Optional[dict] = None):
        self.input_tensors = {}
        for name, shape in (input_tensors or {}).items():
            self.input_tensors[name] = SymbolicTensor(name, shape)

    def __call__(self, tensor_name: str, tensor_shape: tuple):
        if tensor_name in self.input_tensors:
            raise ValueError(f"Tensor {tensor_name} already exists")
        self.input_tensors[tensor_name] = SymbolicTensor(tensor_name, tensor_shape)

        def decorator(func):
            return func
        return decorator


# ------------------------------------------------------------------------------------------
# mask utilities
# ------------------------------------------------------------------------------------------
def create_mask(mod_fn, B: Optional[int], H: Optional[int], Q_LEN: int, KV_LEN: int,
                device: str = "cuda") -> torch.Tensor:
    """Materialise ``mod_fn(b, h, q_idx, kv_idx)`` on the full index grid -> bool [B,H,Q,KV]."""
    B = 1 if B is None else B
    H = 1 if H is None else H
    b = torch.arange(B, device=device).view(B, 1, 1, 1)
    h = torch.arange(H, device=device).view(1, H, 1, 1)
    q = torch.arange(Q_LEN, device=device).view(1, 1, Q_LEN, 1)
    kv = torch.arange(KV_LEN, device=device).view(1, 1, 1, KV_LEN)
    mask = mod_fn(b, h, q, kv)
    if not isinstance(mask, torch.Tensor):
        mask = torch.tensor(bool(mask), device=device)
    return mask.to(torch.bool).expand(B, H, Q_LEN, KV_LEN)


_DEFAULT_SPARSE_BLOCK_SIZE = 128
BLOCK_SIZE = 128


def _round_up(x: int, multiple: int) -> int:
    return (x + multiple - 1) // multiple * multiple


def _convert_mask_to_block_mask(mask: torch.Tensor, Q_BLOCK_SIZE=_DEFAULT_SPARSE_BLOCK_SIZE,
                                KV_BLOCK_SIZE=_DEFAULT_SPARSE_BLOCK_SIZE,
                                separate_full_blocks: bool = False):
    """bool [.., Q, KV] -> int8 [B, H, ceil(Q/bm), ceil(KV/bn)]; an entry is 1 when ANY element of
    the block is visible.  With ``separate_full_blocks`` returns (partial, full)."""
    assert mask.dtype == torch.bool
    while mask.dim() < 4:
        mask = mask.unsqueeze(0)
    B, H, Q, KV = mask.shape
    Qp, KVp = _round_up(Q, Q_BLOCK_SIZE), _round_up(KV, KV_BLOCK_SIZE)
    if (Qp, KVp) != (Q, KV):
        mask = torch.nn.functional.pad(mask, (0, KVp - KV, 0, Qp - Q))
    blocks = mask.reshape(B, H, Qp // Q_BLOCK_SIZE, Q_BLOCK_SIZE, KVp // KV_BLOCK_SIZE, KV_BLOCK_SIZE)
    visible = blocks.sum(dim=(3, 5), dtype=torch.int64)
    if separate_full_blocks:
        full = visible == Q_BLOCK_SIZE * KV_BLOCK_SIZE
        partial = (visible > 0) & ~full
        return partial.to(torch.int8), full.to(torch.int8)
    return (visible > 0).to(torch.int8), None


def _block_grid(mask_tensor):
    _, _, M, N = mask_tensor.shape
    qi = torch.arange(M, device=mask_tensor.device).view(M, 1)
    ki = torch.arange(N, device=mask_tensor.device).view(1, N)
    return qi, ki


def is_causal_mask(mask_tensor, block_M, block_N):
    """True iff the block mask [B,H,M,N] is exactly the block pattern of q_idx >= kv_idx:
    block (i, j) set iff (i+1)*block_M > j*block_N."""
    qi, ki = _block_grid(mask_tensor)
    expect = (qi + 1) * block_M > ki * block_N
    return torch.all(mask_tensor.bool() == expect)


def is_less_causal_mask(mask_tensor, block_M, block_N):
    """True iff no block strictly above the causal diagonal is set, i.e. every block with
    (i+1)*block_M - 1 < j*block_N is zero (so the kv loop may stop at the diagonal)."""
    qi, ki = _block_grid(mask_tensor)
    above = (qi + 1) * block_M - 1 < ki * block_N
    return torch.all(mask_tensor[..., above] == 0)


def create_block_mask(mask_mod, B, H, QLen, KVLen, device, Q_BLOCK_SIZE=None, KV_BLOCK_SIZE=None):
    """int8 [B,H,ceil(Q/bm),ceil(KV/bn)] "any visible" block mask of ``mask_mod``."""
    Q_BLOCK_SIZE = BLOCK_SIZE if Q_BLOCK_SIZE is None else Q_BLOCK_SIZE
    KV_BLOCK_SIZE = BLOCK_SIZE if KV_BLOCK_SIZE is None else KV_BLOCK_SIZE
    mask = create_mask(mask_mod, B, H, QLen, KVLen, device)
    partial, _ = _convert_mask_to_block_mask(mask, Q_BLOCK_SIZE, KV_BLOCK_SIZE, False)
    return partial


def create_block_idx(mask_mod, B, H, QLen, KVLen, device, Q_BLOCK_SIZE=None, KV_BLOCK_SIZE=None):
    """Indices [n, 4] of the non-empty blocks of ``mask_mod``."""
    block_mask = create_block_mask(mask_mod, B, H, QLen, KVLen, device, Q_BLOCK_SIZE, KV_BLOCK_SIZE)
    return torch.nonzero(block_mask, as_tuple=False)
