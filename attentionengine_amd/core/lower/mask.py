"""mask_mod lowering and mask inference.

The reference traces ``mask_mod(b, h, q_idx, kv_idx)`` with ``torch.fx`` and prints one python
statement per node (attention_engine/core/codegen/common.py:124-152, vocabulary: python
``operator.*`` functions and ``torch.logical_and``), then materialises the block mask to choose
between the dense-causal and the block-sparse template (core/lower/lower.py:721-756).

Here the same fx graph becomes one C++ statement per node inside ``ae_mask_mod``; arithmetic is
done on ``int`` exactly as python does it (floor division and modulo keep python's sign rules),
so the device mask equals the host mask bit for bit.  Mask inference classifies every
(q-tile, kv-tile) pair as empty / partial / full so the kernel can skip empty tiles and skip the
elementwise test on full ones.
"""
from __future__ import annotations

import operator

import torch
import torch.fx as fx


# fx target -> C++ expression template.  Comparison results are bool, arithmetic is int.
_BINARY = {
    operator.ge: "({0} >= {1})", operator.gt: "({0} > {1})", operator.le: "({0} <= {1})",
    operator.lt: "({0} < {1})", operator.eq: "({0} == {1})", operator.ne: "({0} != {1})",
    operator.add: "({0} + {1})", operator.sub: "({0} - {1})", operator.mul: "({0} * {1})",
    operator.floordiv: "ae_floordiv({0}, {1})", operator.mod: "ae_pymod({0}, {1})",
    operator.and_: "({0} & {1})", operator.or_: "({0} | {1})", operator.xor: "({0} ^ {1})",
    torch.logical_and: "((bool)({0}) & (bool)({1}))", torch.logical_or: "((bool)({0}) | (bool)({1}))",
    torch.logical_xor: "((bool)({0}) ^ (bool)({1}))",
}
_UNARY = {
    operator.neg: "(-{0})", operator.not_: "(!{0})", operator.invert: "ae_invert({0})",
    operator.abs: "ae_iabs({0})", abs: "ae_iabs({0})", torch.logical_not: "(!(bool)({0}))",
    torch.abs: "ae_iabs({0})",
}

MASK_HELPERS = """
AE_DEV int ae_floordiv(int a, int b) { int q = a / b; return ((a % b != 0) && ((a < 0) != (b < 0))) ? q - 1 : q; }
AE_DEV int ae_pymod(int a, int b) { int r = a % b; return (r != 0 && ((r < 0) != (b < 0))) ? r + b : r; }
AE_DEV int ae_iabs(int a) { return a < 0 ? -a : a; }
AE_DEV bool ae_invert(bool a) { return !a; }
AE_DEV int ae_invert(int a) { return ~a; }
"""


def _arg(a):
    if isinstance(a, fx.Node):
        return "n_" + a.name   # prefixed: fx names such as "xor" / "and" are C++ tokens
    if isinstance(a, bool):
        return "true" if a else "false"
    if isinstance(a, int):
        return str(a)
    raise NotImplementedError(f"mask_mod: unsupported constant operand {a!r} (integers only)")


class LoweredMask:
    """Result of tracing a mask_mod."""

    def __init__(self, body: str, uses_b: bool, uses_h: bool, python_lines):
        self.body = body              # statements of ae_mask_mod, ending in a return
        self.uses_b = uses_b
        self.uses_h = uses_h
        self.python_lines = python_lines  # the traced graph, one line per node (debug aid)


def lower_mask_mod(mask_mod) -> LoweredMask:
    """fx-trace ``mask_mod`` and translate it to the body of
    ``bool ae_mask_mod(int b, int h, int q_idx, int kv_idx)``."""
    graph = fx.symbolic_trace(mask_mod).graph
    nodes = list(graph.nodes)
    placeholders = [n for n in nodes if n.op == "placeholder"]
    if len(placeholders) != 4:
        raise NotImplementedError("mask_mod must take exactly (b, h, q_idx, kv_idx)")
    canonical = ["b", "h", "q_idx", "kv_idx"]
    lines = [f"const int n_{ph.name} = {c}; (void)n_{ph.name};" for ph, c in zip(placeholders, canonical)]
    py = []
    ret = None
    for n in nodes:
        if n.op == "placeholder":
            continue
        if n.op == "output":
            ret = n.args[0]
            continue
        if n.op != "call_function":
            raise NotImplementedError(f"mask_mod: unsupported graph node {n.op} ({n.target})")
        if n.target in _BINARY and len(n.args) == 2:
            expr = _BINARY[n.target].format(_arg(n.args[0]), _arg(n.args[1]))
        elif n.target in _UNARY and len(n.args) == 1:
            expr = _UNARY[n.target].format(_arg(n.args[0]))
        else:
            raise NotImplementedError(f"mask_mod: unsupported operation {n.target}")
        lines.append(f"const auto n_{n.name} = {expr};")
        py.append(f"{n.name} = {getattr(n.target, '__name__', n.target)}({', '.join(_arg(a) for a in n.args)})")
    if ret is None:
        raise NotImplementedError("mask_mod returned nothing")
    lines.append(f"return (bool)({_arg(ret)});")
    used = {a.name for n in nodes for a in n.all_input_nodes}
    return LoweredMask("\n".join("  " + ln for ln in lines), placeholders[0].name in used,
                       placeholders[1].name in used, py)


class MaskPlan:
    """What the prefill kernel needs to know about a mask.

    mode 0: no mask; mode 1: exactly ``q_idx >= kv_idx`` (analytic tile skip + diagonal test);
    mode 2: tile-class table int8 [b|1, h|1, n_q_tiles, n_kv_tiles] with 0 = skip, 1 = visit and
    apply the elementwise mask, 2 = visit, fully visible.
    """

    def __init__(self, mode: int, table=None, block_m: int = 0, block_n: int = 0, elementwise: bool = False):
        self.mode = mode
        self.table = table
        self.block_m = block_m
        self.block_n = block_n
        self.elementwise = elementwise
        # late q tiles visit clearly more kv tiles than early ones (causal variants, long sliding windows): the
        # kernels then start the long q tiles first
        self.heavy_last = False
        if table is not None and table.shape[2] >= 4:
            work = (table > 0).sum(dim=-1).to(torch.float32).mean(dim=(0, 1))
            third = table.shape[2] // 3
            self.heavy_last = bool(work[-third:].mean() >= 1.25 * work[:third].mean())


def plan_mask(mask_mod, lowered: LoweredMask, B: int, H: int, Sq: int, Skv: int, tile_m: int,
              tile_n: int, elementwise: bool = True, chunk_rows: int = 4096) -> MaskPlan:
    """Classify the mask on the host.  The mask is evaluated with batch/head extent 1 when the
    traced graph does not read b / h, and in row chunks so the full [Sq, Skv] grid is never
    resident at once."""
    if mask_mod is None:
        return MaskPlan(0)
    mb = B if lowered.uses_b else 1
    mh = H if lowered.uses_h else 1
    n_qt = (Sq + tile_m - 1) // tile_m
    n_kt = (Skv + tile_n - 1) // tile_n
    table = torch.zeros(mb, mh, n_qt, n_kt, dtype=torch.int8)
    exactly_causal = True
    chunk_rows = max(tile_m, (chunk_rows // tile_m) * tile_m)
    kv = torch.arange(Skv).view(1, 1, 1, Skv)
    bb = torch.arange(mb).view(mb, 1, 1, 1)
    hh = torch.arange(mh).view(1, mh, 1, 1)
    for r0 in range(0, Sq, chunk_rows):
        r1 = min(Sq, r0 + chunk_rows)
        q = torch.arange(r0, r1).view(1, 1, r1 - r0, 1)
        m = mask_mod(bb, hh, q, kv)
        if not isinstance(m, torch.Tensor):
            m = torch.tensor(bool(m))
        m = m.to(torch.bool).expand(mb, mh, r1 - r0, Skv)
        if exactly_causal:
            exactly_causal = bool(torch.equal(m, (q >= kv).expand_as(m)))
        # a block cut by the sequence end is "full" when every in-range element is visible
        vis = _count_blocks(m, tile_m, tile_n)
        tot = _count_blocks(torch.ones(1, 1, r1 - r0, Skv, dtype=torch.bool), tile_m, tile_n)
        full = ((vis == tot) & (vis > 0)).to(torch.int8)
        partial = ((vis > 0) & (vis < tot)).to(torch.int8)
        cls = partial + 2 * full
        t0 = r0 // tile_m
        table[:, :, t0:t0 + cls.shape[2], :] = cls
    if exactly_causal and Sq == Skv and elementwise:
        return MaskPlan(1, None, tile_m, tile_n, True)
    if not elementwise:
        # mask_value != "-inf": the forward only skips tiles (attn_tl.py:124-137 guards the
        # elementwise test with is_inf_mask); visited tiles are treated as fully visible.
        table = torch.where(table > 0, torch.full_like(table, 2), table)
    return MaskPlan(2, table.contiguous(), tile_m, tile_n, elementwise)


def _count_blocks(mask: torch.Tensor, bm: int, bn: int) -> torch.Tensor:
    """Number of True elements per (bm x bn) block of a bool [B,H,Q,KV] tensor (zero padded)."""
    B, H, Q, KV = mask.shape
    Qp, KVp = (Q + bm - 1) // bm * bm, (KV + bn - 1) // bn * bn
    if (Qp, KVp) != (Q, KV):
        mask = torch.nn.functional.pad(mask, (0, KVp - KV, 0, Qp - Q))
    return mask.reshape(B, H, Qp // bm, bm, KVp // bn, bn).sum(dim=(3, 5), dtype=torch.int64)
