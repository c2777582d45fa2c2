"""Interpreter for traced score_mod / mask_mod / OnlineFunc graphs.  Test infrastructure only.

Runs the generic online algorithm of the reference (attn_script/Readme.md:45-65; operation order
of core/template/tl_template/attn/attn_tl.py:105-172) on the host, one kv tile at a time, by
*evaluating the traced expression graph* with torch -- so it checks the tracer and the functor
semantics independently of any GPU code:

    for each kv tile:  s = mask ? QK^T : -inf;  s = score_mod(s);
                       s, rowscales, o_scale = online_fwd(s, rowscales);
                       acc = acc * o_scale + cast(s) @ V
    o, final_rowscales = online_fwd_epilogue(acc, rowscales)

Operation semantics follow core/codegen/tl_gen.py:7-132 with exact transcendentals (exp, log,
tanh); "-inf" initial values use the finite sentinel of core/lower/lower.py:23-29.
"""
from __future__ import annotations

import math

import torch

_NEG = -1e38


def _init_value(name):
    name = name.strip()
    if name == "-inf":
        return _NEG
    if name in ("inf", "+inf"):
        return -_NEG
    return float(name)


def evaluate(sym, env, memo=None):
    """Value of traced symbol ``sym``; ``env`` maps id(leaf symbol) -> tensor/float."""
    memo = {} if memo is None else memo
    key = id(sym)
    if key in memo:
        return memo[key]
    t = sym.code.type
    if key in env:
        val = env[key]
    elif t == "Const":
        val = float(sym.code.value)
    elif t == "Var" and not sym.prev:
        name = sym.code.name.strip()
        if name == "o_scale":
            val = 1.0   # the o_scale buffer is pre-filled with 1.0 (attn_tl.py:108)
        else:
            try:
                val = _init_value(name)
            except ValueError:
                raise KeyError(f"no value for input {name!r}") from None
    else:
        a = [evaluate(p, env, memo) for p in sym.prev]
        a = [x if isinstance(x, torch.Tensor) else torch.tensor(x, dtype=torch.float64) for x in a]
        if t == "Add":
            val = a[0] + a[1]
        elif t == "Sub":
            val = a[0] - a[1]
        elif t == "Mul":
            val = a[0] * a[1]
        elif t == "Div":
            val = a[0] / a[1]
        elif t == "Max":
            val = torch.maximum(a[0], a[1])
        elif t == "Neg":
            val = -a[0]
        elif t == "Abs":
            val = a[0].abs()
        elif t == "Tanh":
            val = torch.tanh(a[0])
        elif t == "Exp":
            val = torch.exp(a[0])
        elif t == "Exp2":
            val = torch.exp2(a[0])
        elif t == "Log":
            val = torch.log(a[0])
        elif t == "Log2":
            val = torch.log2(a[0])
        elif t == "MaxBwd":
            # gradient a[0] of max(x, y) with respect to x: passes where x won (zero at a tie)
            val = torch.where(a[1] > a[2], a[0], torch.zeros_like(a[0]))
        elif t == "ReduceSum":
            val = a[0].sum(dim=-1, keepdim=True)
        elif t == "ReduceMax":
            val = a[0].max(dim=-1, keepdim=True).values
        elif t == "ReduceAbsSum":
            val = a[0].abs().sum(dim=-1, keepdim=True)
        elif t == "ColReduceSum":
            val = a[0].sum(dim=0, keepdim=True)
        elif t == "ColReduceMax":
            val = a[0].max(dim=0, keepdim=True).values
        elif t == "ColReduceAbsSum":
            val = a[0].abs().sum(dim=0, keepdim=True)
        else:
            raise NotImplementedError(t)
    memo[key] = val
    return val


def _as_tensor(x, like):
    if isinstance(x, torch.Tensor):
        return x
    return torch.full_like(like, float(x))


def online_attention(q, k, v, score_mod, mask_mod, online_func, custom_fwd_inputs=None,
                     custom_tensors=(), block_n=64, mask_value="-inf", p_dtype=None):
    """Run the traced functions tile by tile.  Returns (out [B,Sq,Hq,DV] float64,
    {name: final rowscale [B,Hq,Sq] float64}).

    ``p_dtype``: if given (torch.float16 / bfloat16) the probabilities are rounded to it before
    the PV product, as the kernels do (attn_tl.py:153)."""
    from core.transform.core import CustomIO, SymbolicArray, SymbolScalar   # product tracer types
    from core.transform.graph import Var

    custom_fwd_inputs = custom_fwd_inputs if custom_fwd_inputs is not None else CustomIO()
    B, Sq, Hq, D = q.shape
    Skv, Hkv, DV = k.shape[1], k.shape[2], v.shape[3]
    G = Hq // Hkv
    qd, kd, vd = q.double(), k.double(), v.double()
    out = torch.zeros(B, Sq, Hq, DV, dtype=torch.float64)
    finals = {}

    def fresh_indices():
        return (SymbolScalar("b", Var("b"), shape_idx=[]), SymbolScalar("h", Var("h"), shape_idx=[]),
                SymbolScalar("q_idx", Var("q_idx"), shape_idx=["block_M"]),
                SymbolScalar("kv_idx", Var("kv_idx"), shape_idx=["block_N"]))

    # trace once
    sb, sh, sq, skv = fresh_indices()
    s_in = SymbolicArray("scores", Var("scores"), shape_idx=["block_M", "block_N"])
    s_out = score_mod(s_in, custom_fwd_inputs, sb, sh, sq, skv) if score_mod is not None else s_in
    ob, oh, oq, _ = fresh_indices()
    o_in = SymbolicArray("scores", Var("scores"), shape_idx=["block_M", "block_N"])
    rowscales = online_func.online_rowscales
    for r in rowscales.values():
        r.clear_codegen()
    o_scores, o_rows, o_scale = online_func.online_fwd(o_in, rowscales, ob, oh, oq)
    eb, eh, eq, _ = fresh_indices()
    acc_in = SymbolicArray("acc_o", Var("acc_o"), shape_idx=["block_M", "dimv"])
    e_out, e_finals = online_func.online_fwd_epilogue(acc_in, rowscales, eb, eh, eq)

    cust_syms = list(custom_fwd_inputs.input_tensors.values())
    qi = torch.arange(Sq, dtype=torch.float64).view(Sq, 1)

    def custom_env(b, h):
        env = {}
        for sym, t in zip(cust_syms, custom_tensors):
            t = t.double()
            idx = []
            for d in sym.shape_idx:
                idx.append({"batch": b, "heads": h}.get(d, slice(None) if d in ("seq_len", "seq_len_kv") else 0))
            val = t[tuple(idx)] if t.dim() == len(idx) else t.reshape(-1)[0]
            if "seq_len" in sym.shape_idx and "seq_len_kv" not in sym.shape_idx:
                val = val.reshape(Sq, 1)
            env[id(sym)] = val
        return env

    for b in range(B):
        for h in range(Hq):
            hk = h // G
            state = {n: torch.full((Sq, 1), _init_value(r.code.name), dtype=torch.float64)
                     for n, r in rowscales.items()}
            acc = torch.zeros(Sq, DV, dtype=torch.float64)
            cenv = custom_env(b, h)
            for j0 in range(0, Skv, block_n):
                j1 = min(Skv, j0 + block_n)
                s = qd[b, :, h] @ kd[b, j0:j1, hk].T
                kvi = torch.arange(j0, j1, dtype=torch.float64).view(1, -1)
                if mask_mod is not None and mask_value == "-inf":
                    vis = mask_mod(torch.tensor(b), torch.tensor(h), torch.arange(Sq).view(Sq, 1),
                                   torch.arange(j0, j1).view(1, -1))
                    vis = torch.as_tensor(vis, dtype=torch.bool).expand(Sq, j1 - j0)
                    s = s.masked_fill(~vis, float("-inf"))
                # custom tensors with a kv dimension contribute their columns of this tile
                tenv = {id(sym): (cenv[id(sym)][:, j0:j1] if "seq_len_kv" in sym.shape_idx else cenv[id(sym)])
                        for sym in cust_syms}
                env = {id(s_in): s, id(sb): float(b), id(sh): float(h), id(sq): qi, id(skv): kvi, **tenv}
                s = _as_tensor(evaluate(s_out, env), s)
                env = {id(o_in): s, id(ob): float(b), id(oh): float(h), id(oq): qi, **tenv}
                for n, r in rowscales.items():
                    env[id(r)] = state[n]
                memo = {}
                p = _as_tensor(evaluate(o_scores, env, memo), s)
                new_state = {n: evaluate(o_rows[n], env, memo) for n in o_rows}
                scale = evaluate(o_scale, env, memo)
                for n, val in new_state.items():
                    state[n] = _as_tensor(val, state[n]).clone()
                if p_dtype is not None:
                    p = p.to(p_dtype).double()
                acc = acc * scale + p @ vd[b, j0:j1, hk]
            env = {id(acc_in): acc, id(eb): float(b), id(eh): float(h), id(eq): qi, **cenv}
            for n, r in rowscales.items():
                env[id(r)] = state[n]
            memo = {}
            out[b, :, h] = _as_tensor(evaluate(e_out, env, memo), acc)
            for n, sym in e_finals.items():
                val = _as_tensor(evaluate(sym, env, memo), state[next(iter(state))] if state else acc[:, :1])
                finals.setdefault(n, torch.zeros(B, Hq, Sq, dtype=torch.float64))[b, h] = val.reshape(Sq)
    return out, finals


def combine_partials(online_func, partial_o, partial_rowscales):
    """Evaluate a traced ``OnlineFunc.combine`` (attn_script/gqa_inference.py:73-81):
    partial_o [n_split, rows, DV], partial_rowscales {name: [n_split, rows]} -> o [rows, DV]
    (= sum_k partial_o[k] * o_scale[k], attn_decode_tl.py:184-189)."""
    from core.transform.core import SymbolicColReduceArray
    from core.transform.graph import Var

    syms = {n: SymbolicColReduceArray(n, Var(n), shape_idx=["num_split", "block_M"])
            for n in partial_rowscales}
    o_scale = online_func.combine(syms)
    env = {id(syms[n]): partial_rowscales[n].double() for n in syms}
    w = evaluate(o_scale, env)
    w = w if isinstance(w, torch.Tensor) else torch.full_like(next(iter(env.values())), float(w))
    return (partial_o.double() * w.unsqueeze(-1)).sum(dim=0)
