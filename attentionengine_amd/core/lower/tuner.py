"""Measured choice between the tile configurations of the prefill kernels, with the reference's json cache.

The reference tunes (block_M, block_N, num_stages, thread_num, shared_fuse) of its TileLang kernel when an
engine is built with ``tune=True`` and keeps the winner in ``tune_file``: a json list of
``{"batch", "heads", "seq_len", "dim", "dimv", "tuned_config": [...]}`` records, looked up by the five
problem keys before anything is measured
(attention_engine/core/template/tl_template/attn/attn_tl.py:33-48 candidates, 465-500 cache, 503-521 use;
backward 538-552).  Here the candidates are the tile configurations the HIP templates can be compiled with
for the head dims at hand, the measurement is HIP events around back-to-back launches on the caller's own
tensors at the first call, and the file keeps the same records; ``tuned_config`` is
``[block_M, block_N, LDS stages, threads, waves per SIMD, template]`` for the forward and
``[q rows of a dq workgroup]`` for the backward.  A record whose configuration is not among the candidates
(e.g. written by the reference for another GPU) is ignored and measured again.
"""
from __future__ import annotations

import json
import os
import tempfile

import torch

from . import lower as L

# extents the reference assumes for dynamic (string) dims when it looks a problem up (attn_tl.py:465-472)
_DYNAMIC_DEFAULT = {"batch": 4, "heads": 32, "seq_len": 2048}


def problem_keys(q_shape, dim, dimv):
    """The five keys of a cache record from the declared q shape [batch, heads, seq_len, dim]."""
    def ext(x, name):
        return _DYNAMIC_DEFAULT[name] if isinstance(x, str) else int(x)
    return {"batch": ext(q_shape[0], "batch"), "heads": ext(q_shape[1], "heads"),
            "seq_len": ext(q_shape[2], "seq_len"), "dim": int(dim), "dimv": int(dimv)}


def _salvage(text):
    """The complete records of a damaged file (a write that was cut short, two writers): every json object
    that still parses and carries a ``tuned_config``."""
    dec, recs, pos = json.JSONDecoder(), [], 0
    while True:
        pos = text.find("{", pos)
        if pos < 0:
            return recs
        try:
            obj, end = dec.raw_decode(text, pos)
        except ValueError:
            pos += 1
            continue
        if isinstance(obj, dict) and "tuned_config" in obj:
            recs.append(obj)
        pos = end


def _records(tune_file):
    if not tune_file or not os.path.exists(tune_file):
        return []
    try:
        with open(tune_file) as f:
            text = f.read()
    except OSError:
        return []
    try:
        recs = json.loads(text)
    except ValueError:
        return _salvage(text)
    return recs if isinstance(recs, list) else []


def lookup(tune_file, pk):
    """tuned_config of the record with these problem keys, or None."""
    for rec in _records(tune_file):
        if isinstance(rec, dict) and all(rec.get(k) == v for k, v in pk.items()):
            return rec.get("tuned_config")
    return None


def store(tune_file, pk, tuned_config):
    """Adds (or replaces) the record of this problem; the other records of the file are kept.  The new contents
    go to a temporary file of this process in the same directory, which then replaces ``tune_file`` in one step:
    a reader never sees half a file, and a crash in the middle leaves the old one."""
    recs = [r for r in _records(tune_file)
            if not (isinstance(r, dict) and all(r.get(k) == v for k, v in pk.items()))]
    recs.append({**pk, "tuned_config": list(tuned_config)})
    d = os.path.dirname(os.path.abspath(tune_file))
    fd, tmp = tempfile.mkstemp(prefix=os.path.basename(tune_file) + ".", suffix=".tmp", dir=d)
    try:
        with os.fdopen(fd, "w") as f:
            json.dump(recs, f, indent=4)
        os.replace(tmp, tune_file)
    except BaseException:
        try:
            os.unlink(tmp)
        except OSError:
            pass
        raise


def prefill_candidates(d, dv, softmax, elementwise):
    """Every tile configuration the forward templates are built for at these head dims; the first one is
    what ``choose_prefill_tiles`` picks for a problem large enough to fill the chip."""
    if d in L.DIRECT_D and dv in L.DIRECT_DV:
        c = []
        if d in (64, 128) and dv in (64, 128) and (softmax is not None or elementwise):
            c.append(L.pipelined_tiles(d, dv))
        # two waves per SIMD while a wave may fit 256 registers (Q fragments of up to 192 columns, 128 value columns)
        shapes = [(2, 64), (2, 32), (1, 64)] if d <= 192 and dv <= 128 else [(1, 64), (1, 32)]
        if d > 128 and dv <= 128:
            shapes.append((1, 32))
        for wpe, bn in shapes:
            if L.direct_tile_ok(d, dv, bn) and not (bn == 64 and dv > 256):
                c.append(L.PrefillTiles(waves_per_eu=wpe, block_n=bn))
        return c
    base = L.choose_prefill_tiles(d, dv)
    c = [base]
    other, nt = 96 - base.block_n, 64 * base.n_waves          # the kv tile is 32 or 64 keys
    if (other * d // 8) % nt == 0 and (other * dv // 8) % nt == 0:
        c.append(L.PrefillTiles(template=base.template, n_waves=base.n_waves, block_n=other,
                                waves_per_eu=base.waves_per_eu, k_pad=base.k_pad, v_pad=base.v_pad))
    return c


def encode_tiles(t):
    return [t.block_m, t.block_n, t.kv_stages, 64 * t.n_waves, t.waves_per_eu, t.template]


def decode_tiles(tuned_config, candidates):
    """The candidate a cache record names, or None."""
    if not isinstance(tuned_config, (list, tuple)):
        return None
    for t in candidates:
        if list(tuned_config) == encode_tiles(t):
            return t
    return None


def time_call(fn, budget_ms=30.0, min_calls=3, max_calls=200):
    """Mean milliseconds of ``fn()`` on torch's current stream: two warm-up calls, a one-call estimate, then
    as many back-to-back calls as fit ``budget_ms`` between two events."""
    fn()
    fn()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    fn()
    end.record()
    end.synchronize()
    n = int(max(min_calls, min(max_calls, budget_ms / max(start.elapsed_time(end), 1e-3))))
    start.record()
    for _ in range(n):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / n


def pick(candidates, build, run, log=None):
    """Measures ``run(build(c))`` for every candidate; candidates that cannot be built or launched for this
    problem are passed over.  Returns (best candidate, what build() made of it, {candidate index: ms})."""
    best, times = None, {}
    for i, c in enumerate(candidates):
        try:
            made = build(c)
            ms = time_call(lambda: run(made))
        except (NotImplementedError, ValueError, RuntimeError) as e:
            if log is not None:
                log(f"tune: {c} not usable here ({e})")
            continue
        times[i] = ms
        if log is not None:
            log(f"tune: {c} {ms:.4f} ms")
        if best is None or ms < best[2]:
            best = (c, made, ms)
    if best is None:
        raise RuntimeError("no tile configuration could be launched for this problem")
    return best[0], best[1], times
