"""Benchmark of the fused attention path (forward; one extra workload for the backward) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-extra] [--no-cpu]

A "step" is one forward pass of the hot path over one batch of synthetic input that is already
resident in HBM.  The headline workload (default) is the configuration the metric is quoted on:
causal softmax prefill, fp16, B=2 H=32 S=4096 D=DV=128 ("c2_causal").  Rank 0 prints ONE JSON line.
Its `roofline` object prices the dominant kernel of the workload against MI355X's published peaks
(dense fp16/bf16 MFMA 2.5 PFLOP/s, HBM 8 TB/s) using the ALGORITHMIC flops / bytes of one launch and
the average launch duration measured with HIP events on the launch stream; `cpu_baseline` is the
CPU oracle (a restatement of the reference's eager PyTorch path) timed on the host cores on a
bounded sample of the same workload.  The remaining benchmark configurations are measured too and
reported inside the same line under `other_configs` (disable with --no-extra).

FLOP / byte conventions are the reference's: prefill 2*B*H*Sq*Skv*(D+DV), halved if causal
(attention_engine/benchmark/bench_utils.py:1185-1186); GQA decode bytes = K+V streamed; MLA
bytes = B*Skv*D*itemsize, flops = 2*B*H*Skv*(D+DV) (attn_script/mla_decode.py:129).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "attentionengine_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_MFMA_TFLOPS = 2500.0   # dense fp16 / bf16
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # name: (engine key in __graft_entry__.benchmark_engines, kind)
    "c2_causal": ("c2_softmax_causal", "prefill"),
    "c2_full": ("c2_softmax_full", "prefill"),
    "c3_sigmoid": ("c3_sigmoid", "prefill"),
    "c4_gqa_decode": ("c4_gqa_decode", "gqa_decode"),
    "c5_mla_decode": ("c5_mla_decode", "mla_decode"),
    # not a BASELINE configuration: the decode shape of the reference's own script (attn_script/gqa_inference.py,
    # batch 1: one launch whose last workgroup merges; the call is bound by latency, not by HBM)
    "gqa_decode_b1": ("gqa_decode_b1", "gqa_decode"),
    # not a BASELINE configuration: the backward of c2_causal (dq, dk, dv from dout; three launches)
    "c2_causal_bwd": ("c2_softmax_causal", "prefill_bwd"),
}


ONLY_ON_REQUEST = {"gqa_decode_b1"}      # measured with --workload, not part of the default line's other_configs


# HBM bytes per launch of each workload's dominant kernel, from the hardware counters FETCH_SIZE and
# WRITE_SIZE (rocprofv3 --pmc, one counter per run, `--copy-probe` in the same run so that a 256 MiB copy
# kernel calibrates the counter).  The figures live next to the profile summaries they were computed from,
# in profiles/traffic.json: {workload: {"kernel": ..., "fetch_bytes": ..., "write_bytes": ...}}; a workload
# without an entry reports null.
def measured_traffic(name):
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            e = json.load(f)[name]
        return float(e["fetch_bytes"]) + float(e["write_bytes"])
    except (OSError, KeyError, ValueError, TypeError):
        return None


def _inputs(name, device):
    """Synthetic N(0,1) inputs of the workload's shape, generated on the CPU with seed 0 in the
    order q, k, v (MLA: q, q_pe, kv, k_pe), rounded to the compute dtype, copied to the GPU."""
    import torch
    g = torch.Generator().manual_seed(0)

    def rn(*shape, dtype):
        return torch.randn(*shape, generator=g, dtype=torch.float32).to(dtype).to(device)
    f16, bf16 = torch.float16, torch.bfloat16
    if name in ("c2_causal", "c2_full", "c3_sigmoid", "c2_causal_bwd"):
        B, H, S, D = 2, 32, 4096, 128
        args = [rn(B, S, H, D, dtype=f16), rn(B, S, H, D, dtype=f16), rn(B, S, H, D, dtype=f16)]
        if name == "c3_sigmoid":
            args.append(torch.tensor([-math.log(S)], dtype=torch.float32, device=device))
        if name == "c2_causal_bwd":
            args.append(rn(B, S, H, D, dtype=f16))          # dout
        flops = 4.0 * B * H * S * S * D * (1.0 if name in ("c2_full", "c3_sigmoid") else 0.5)
        if name == "c2_causal_bwd":
            flops *= 2.5     # the reference's count: 4*B*H*S^2*DV + 6*B*H*S^2*D, halved (bench_utils.py:1199-1201)
        return args, {"flops": flops, "bytes": 4.0 * B * S * H * D * 2,
                      "shape": {"B": B, "H": H, "S": S, "D": D, "DV": D}, "dtype": "fp16"}
    if name in ("c4_gqa_decode", "gqa_decode_b1"):
        B, Hq, Hkv, Skv, D = (64 if name == "c4_gqa_decode" else 1), 32, 8, 8192, 128
        args = [rn(B, 1, Hq, D, dtype=f16), rn(B, Skv, Hkv, D, dtype=f16), rn(B, Skv, Hkv, D, dtype=f16)]
        return args, {"flops": 4.0 * B * Hq * Skv * D, "bytes": 2.0 * B * Skv * Hkv * D * 2,
                      "shape": {"B": B, "Hq": Hq, "Hkv": Hkv, "Skv": Skv, "D": D, "DV": D}, "dtype": "fp16"}
    if name == "c5_mla_decode":
        B, H, Skv, D, DV = 128, 128, 4096, 576, 512
        args = [rn(B, 1, H, DV, dtype=bf16), rn(B, 1, H, D - DV, dtype=bf16),
                rn(B, Skv, 1, DV, dtype=bf16), rn(B, Skv, 1, D - DV, dtype=bf16)]
        return args, {"flops": 2.0 * B * H * Skv * (D + DV), "bytes": 1.0 * B * Skv * D * 2,
                      "shape": {"B": B, "Hq": H, "Hkv": 1, "Skv": Skv, "D": D, "DV": DV}, "dtype": "bf16"}
    raise KeyError(name)


CLOCK_RAMP_MS = 60.0
CPU_BASELINE_SECONDS = 10.0   # the CPU oracle repeats its sample for about this long


def measure(name, steps, warmup):
    """Time `steps` forward passes of workload `name`; returns a result dict."""
    import torch
    import __graft_entry__ as G
    from core.runtime import hip_rt as rt
    dev = torch.device("cuda:0")
    key, kind = WORKLOADS[name]
    mod = G.benchmark_engines({key})[key]
    args, info = _inputs(name, dev)
    if kind == "prefill_bwd":
        # the timed step is the backward alone: dq, dk, dv from (q, k, v, out, lse, dout)
        q, k, v, dout = args
        with torch.no_grad():
            out = mod(q, k, v)
        lse = mod.final_rowscales["lse"]
        mod, args = mod._op.backward_op(), [q, k, v, out, lse, dout]
    # Untimed warm-up: the W steps asked for, continued until the launches have covered CLOCK_RAMP_MS.
    # The shader clock of an idle MI355X takes some tens of milliseconds of load to reach its working
    # point (measured: 0.335 ms per step after 10 warm-up steps, 0.29 ms after 50 or more), and the
    # reference's own harness warms up for 25 ms before it times anything (bench_utils.py:14-99).
    checked = verify(name, kind, mod, args)       # untimed: one slice against eager fp32 torch
    # MLA decode streams 0.6 GB, about twice the 256 MB of last-level cache: two copies of the KV cache
    # alternate between steps so that no step finds a part of its input cached by the previous one
    rotation = [args]
    if kind == "mla_decode":
        rotation.append([args[0], args[1], args[2].clone(), args[3].clone()])
    n_warm = 0
    t_w = time.perf_counter()
    while n_warm < max(1, warmup) or (time.perf_counter() - t_w) * 1e3 < CLOCK_RAMP_MS:
        for i in range(8):
            mod(*rotation[i % len(rotation)])
        n_warm += 8
        torch.cuda.synchronize()
    stream = torch.cuda.current_stream(dev).cuda_stream
    e0, e1 = rt.Event(), rt.Event()
    t0 = time.perf_counter()
    e0.record(stream)
    for i in range(steps):
        mod(*rotation[i % len(rotation)])
    e1.record(stream)
    ev_ms = e0.elapsed_ms(e1) / steps          # synchronises on e1
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    res = {"workload": name, "kind": kind, "ms_per_step": wall_ms, "kernel_ms": ev_ms, "warmup_launches": n_warm,
           "checked": checked, **info}
    res["tflops"] = info["flops"] / (wall_ms * 1e-3) / 1e12
    res["gbs"] = info["bytes"] / (wall_ms * 1e-3) / 1e9
    stamps = getattr(getattr(mod, "_op", None), "clock_stamps", None)     # builds with AE_CLOCK_STAMPS=1 only
    if stamps is not None:
        res["clock_mhz"] = _clock_mhz(stamps)
        ph = getattr(getattr(mod, "_op", None), "phase_ticks", None)
        if ph is not None:
            # where a workgroup's time goes, microseconds (100 MHz ticks): launch start = the earliest entry
            t = ph.cpu().double()
            t = t[t[:, 3] > 0]
            t0 = t[:, 0].min()
            res["phases_us"] = {"first_entry_to_last_exit": float((t[:, 3].max() - t0) / 100.0),
                                "entry_after_launch_start_max": float((t[:, 0].max() - t0) / 100.0),
                                "prologue_median": float((t[:, 1] - t[:, 0]).median() / 100.0),
                                "loop_median": float((t[:, 2] - t[:, 1]).median() / 100.0),
                                "epilogue_median": float((t[:, 3] - t[:, 2]).median() / 100.0),
                                "workgroup_median": float((t[:, 3] - t[:, 0]).median() / 100.0),
                                "workgroup_max": float((t[:, 3] - t[:, 0]).max() / 100.0)}
    if kind in ("prefill", "prefill_bwd"):
        ach = info["flops"] / (ev_ms * 1e-3) / 1e12
        res["roofline"] = {"bound": "mfma", "achieved": ach, "peak": PEAK_MFMA_TFLOPS, "unit": "TFLOP/s",
                           "frac": ach / PEAK_MFMA_TFLOPS, "traffic": measured_traffic(name)}
    else:
        ach = info["bytes"] / (ev_ms * 1e-3) / 1e9
        res["roofline"] = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                           "frac": ach / PEAK_HBM_GBS, "traffic": measured_traffic(name)}
        if kind == "mla_decode":
            res["mfma_frac"] = info["flops"] / (ev_ms * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS
    del args, mod, rotation
    torch.cuda.empty_cache()
    return res


def verify(name, kind, mod, args):
    """One untimed call of the workload, compared on a slice with eager fp32 torch evaluated on the GPU
    (closed forms of bench_utils.py:1250-1275 and mla_decode_tl.py:266-306 of the reference).  Bars as in
    the tests: out 2e-2 max-abs, lse 1e-3; gradients 2e-2 + 1 % of their largest magnitude."""
    import torch
    rep = {"against": "eager fp32 torch, one slice", "ok": False}
    with torch.no_grad():
        if kind == "prefill":
            q, k, v = args[:3]
            b, h = q.shape[0] - 1, q.shape[2] - 1
            out = mod(*args)
            D = q.shape[3]
            s = (q[b, :, h].float() @ k[b, :, h].float().T) / math.sqrt(D)
            if name == "c3_sigmoid":
                ref = torch.sigmoid(s + args[3].float()) @ v[b, :, h].float()
                rep["slice"] = f"b{b} h{h}"
                rep["max_abs_out"] = (out[b, :, h].float() - ref).abs().max().item()
                rep["ok"] = rep["max_abs_out"] <= 2e-2
                return rep
            if name == "c2_causal":
                s = s.masked_fill(~torch.ones_like(s, dtype=torch.bool).tril(), float("-inf"))
            ref = torch.softmax(s, -1) @ v[b, :, h].float()
            lse = mod.final_rowscales["lse"][b, h]
            rep["slice"] = f"b{b} h{h}"
            rep["max_abs_out"] = (out[b, :, h].float() - ref).abs().max().item()
            rep["max_abs_lse"] = (lse - torch.logsumexp(s, -1)).abs().max().item()
        elif kind == "gqa_decode":
            q, k, v = args
            b = q.shape[0] - 1
            out = mod(*args)
            g = q.shape[2] // k.shape[2]
            kk, vv = k[b].float().repeat_interleave(g, 1), v[b].float().repeat_interleave(g, 1)   # [Skv, Hq, D]
            s = torch.einsum("hd,khd->hk", q[b, 0].float(), kk) / math.sqrt(q.shape[3])
            ref = torch.einsum("hk,khd->hd", torch.softmax(s, -1), vv)
            rep["slice"] = f"batch entry {b}"
            rep["max_abs_out"] = (out[b, 0].float() - ref).abs().max().item()
            rep["max_abs_lse"] = (mod.final_rowscales["lse"][b, :, 0] - torch.logsumexp(s, -1)).abs().max().item()
        elif kind == "mla_decode":
            q, q_pe, kv, k_pe = args
            b = q.shape[0] - 1
            out = mod(*args)
            s = (q[b, 0].float() @ kv[b, :, 0].float().T + q_pe[b, 0].float() @ k_pe[b, :, 0].float().T) / math.sqrt(192)
            ref = torch.softmax(s, -1) @ kv[b, :, 0].float()
            rep["slice"] = f"batch entry {b}"
            rep["max_abs_out"] = (out[b, 0].float() - ref).abs().max().item()
            rep["max_abs_lse"] = (mod.final_rowscales["lse"][b, :, 0] - torch.logsumexp(s, -1)).abs().max().item()
        if kind != "prefill_bwd":
            rep["ok"] = rep["max_abs_out"] <= 2e-2 and rep["max_abs_lse"] <= 1e-3
            return rep
    # backward: (q, k, v, out, lse, dout) -> dq, dk, dv; autograd through the eager closed form on one slice
    q, k, v, out, lse, dout = args
    b, h = q.shape[0] - 1, q.shape[2] - 1
    dq, dk, dv = mod(*args)
    qs, ks, vs = (t[b, :, h].float().detach().requires_grad_(True) for t in (q, k, v))
    s = (qs @ ks.T) / math.sqrt(q.shape[3])
    s = s.masked_fill(~torch.ones_like(s, dtype=torch.bool).tril(), float("-inf"))
    (torch.softmax(s, -1) @ vs).backward(dout[b, :, h].float())
    rep["slice"] = f"b{b} h{h}"
    rep["ok"] = True
    for nm, got, want in (("dq", dq, qs.grad), ("dk", dk, ks.grad), ("dv", dv, vs.grad)):
        err = (got[b, :, h].float() - want).abs().max().item()
        rep[f"max_abs_{nm}"] = err
        rep["ok"] = rep["ok"] and err <= 2e-2 + 1e-2 * want.abs().max().item()
    return rep


COPY_PROBE_BYTES = 256 << 20


def copy_probe():
    """One launch of a plain copy kernel over COPY_PROBE_BYTES (reads that many bytes, writes that many)."""
    import ctypes
    import torch
    from core.runtime import hip_rt as rt

    class CopyParams(ctypes.Structure):
        _fields_ = [("src", ctypes.c_void_p), ("dst", ctypes.c_void_p), ("n_vec", ctypes.c_uint64)]
    src = torch.ones(COPY_PROBE_BYTES // 4, dtype=torch.float32, device="cuda:0")
    dst = torch.empty_like(src)
    kern = rt.compile_module("ae_copy_probe.hip", {}).kernel("ae_copy_probe_kernel")
    torch.cuda.synchronize()
    kern.launch(CopyParams(src.data_ptr(), dst.data_ptr(), COPY_PROBE_BYTES // 16), (4096, 1, 1), (256, 1, 1), 0,
                torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.equal(src, dst)


MFMA_FLOP_PER_CLK = 256 * 4 * 1024.0     # 256 CUs x 4 SIMDs x (32*32*16*2 flop per 32-cycle MFMA)


def _clock_mhz(stamps):
    """Shader clock from per-workgroup (s_memtime cycles, s_memrealtime 100 MHz ticks) pairs."""
    st = stamps.cpu().double()
    st = st[st[:, 1] > 0]
    return float(st[:, 0].sum() / st[:, 1].sum() * 100.0) if len(st) else float("nan")


# (label, configuration of ae_mfma_probe.hip) of the cases `--mfma-probe` reports; the first is the pure ceiling
PROBE_CASES = [
    ("fp16 MFMA only, 1 wave/SIMD", {}),
    ("fp16 MFMA only, 2 waves/SIMD", {"AE_PROBE_WAVES_PER_SIMD": 2}),
    ("bf16 MFMA only, 1 wave/SIMD", {"AE_PROBE_BF16": 1}),
    ("fp16 MFMA + 4 v_fma per MFMA", {"AE_PROBE_EXTRA_VALU": 4}),
    ("fp16 MFMA + half a 1 KiB LDS fragment read per MFMA", {"AE_PROBE_LDS": 1}),
    ("fp16 flash-attention mix per MFMA: 1 v_exp + 3 VALU + half a fragment read, 1 wave/SIMD",
     {"AE_PROBE_EXTRA_VALU": 2, "AE_PROBE_EXP": 1, "AE_PROBE_LDS": 1}),
    ("fp16 flash-attention mix per MFMA, 2 waves/SIMD",
     {"AE_PROBE_EXTRA_VALU": 2, "AE_PROBE_EXP": 1, "AE_PROBE_LDS": 1, "AE_PROBE_WAVES_PER_SIMD": 2}),
    ("bf16 flash-attention mix per MFMA, 1 wave/SIMD",
     {"AE_PROBE_EXTRA_VALU": 2, "AE_PROBE_EXP": 1, "AE_PROBE_LDS": 1, "AE_PROBE_BF16": 1}),
    ("fp16 MFMA only, 16x16x32 shape (two per 32x32x16), 1 wave/SIMD", {"AE_PROBE_M16": 1}),
    ("fp16 MFMA only, 16x16x32 shape, 2 waves/SIMD", {"AE_PROBE_M16": 1, "AE_PROBE_WAVES_PER_SIMD": 2}),
    ("fp16 flash-attention mix per two 16x16x32 MFMAs, 1 wave/SIMD",
     {"AE_PROBE_M16": 1, "AE_PROBE_EXTRA_VALU": 2, "AE_PROBE_EXP": 1, "AE_PROBE_LDS": 1}),
    ("fp16 flash-attention mix per two 16x16x32 MFMAs, 2 waves/SIMD",
     {"AE_PROBE_M16": 1, "AE_PROBE_EXTRA_VALU": 2, "AE_PROBE_EXP": 1, "AE_PROBE_LDS": 1, "AE_PROBE_WAVES_PER_SIMD": 2}),
    ("fp16 loop skeleton: the mix on MFMA results, their exponentials as operands, tile loads and a barrier per 32 MFMAs, "
     "1 wave/SIMD",
     {"AE_PROBE_EXTRA_VALU": 1, "AE_PROBE_EXP": 1, "AE_PROBE_LDS": 1, "AE_PROBE_SKELETON": 1}),
    ("fp16 loop skeleton, 2 waves/SIMD of half the rows (a fragment read per MFMA)",
     {"AE_PROBE_EXTRA_VALU": 1, "AE_PROBE_EXP": 1, "AE_PROBE_LDS": 2, "AE_PROBE_SKELETON": 1, "AE_PROBE_WAVES_PER_SIMD": 2}),
    ("fp16 loop skeleton on 16x16x32 MFMAs, 2 waves/SIMD of half the rows (a fragment read per pair)",
     {"AE_PROBE_EXTRA_VALU": 1, "AE_PROBE_EXP": 1, "AE_PROBE_LDS": 2, "AE_PROBE_SKELETON": 1, "AE_PROBE_WAVES_PER_SIMD": 2,
      "AE_PROBE_M16": 1}),
]


def probe_config_text(cfg):
    return "// configuration of ae_mfma_probe.hip\n" + "".join(f"#define {k} {v}\n" for k, v in sorted(cfg.items()))


def mfma_probe(cfg=None, launches=20, iters=250, operands=("zeros", "randn")):
    """The matrix-pipe ceiling of this chip, measured: ae_mfma_probe_kernel (32x32x16 MFMAs back to back, with
    the other work ``cfg`` asks for between them) on all-zero and on N(0,1) operands -- the same code object, so
    the difference is the chip's power management reacting to the operand data.  Returns {operands: {tflops,
    clock_mhz, cycles_per_mfma}}; clock from the kernel's own s_memtime / s_memrealtime stamps, cycles_per_mfma =
    the cycles of that clock one SIMD spent per MFMA over the launch (32 when the matrix pipe never idles)."""
    import ctypes
    import torch
    from core.runtime import hip_rt as rt

    class ProbeParams(ctypes.Structure):
        _fields_ = [("src", ctypes.c_void_p), ("sink", ctypes.c_void_p), ("stamps", ctypes.c_void_p),
                    ("n_src", ctypes.c_uint32), ("iters", ctypes.c_int32)]
    cfg = dict(cfg or {})
    waves_per_simd = int(cfg.get("AE_PROBE_WAVES_PER_SIMD", 1))
    kern = rt.compile_module("ae_mfma_probe.hip", {"ae_config.h": probe_config_text(cfg)}).kernel("ae_mfma_probe_kernel")
    dev = torch.device("cuda:0")
    n_src = 1 << 20
    grid = 256 * 8
    g = torch.Generator().manual_seed(0)
    dt = torch.bfloat16 if cfg.get("AE_PROBE_BF16") else torch.float16
    pools = {"zeros": torch.zeros(n_src, dtype=dt, device=dev),
             "randn": torch.randn(n_src, generator=g, dtype=torch.float32).to(dt).to(dev)}
    sink = torch.zeros(1024, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    out = {}
    for name, pool in pools.items():
        if name not in operands:
            continue
        stamps = torch.zeros((grid, 2), dtype=torch.int64, device=dev)
        prm = ProbeParams(pool.data_ptr(), sink.data_ptr(), stamps.data_ptr(), n_src, iters)
        threads = 256 * waves_per_simd

        def launch():
            kern.launch(prm, (grid, 1, 1), (threads, 1, 1), 0, stream)
        t_w = time.perf_counter()
        while (time.perf_counter() - t_w) * 1e3 < 2 * CLOCK_RAMP_MS:      # to the working clock first
            for _ in range(4):
                launch()
            torch.cuda.synchronize()
        e0, e1 = rt.Event(), rt.Event()
        e0.record(stream)
        for _ in range(launches):
            launch()
        e1.record(stream)
        ms = e0.elapsed_ms(e1) / launches
        flop = grid * 4.0 * waves_per_simd * iters * 32 * 32768.0
        tflops, clock = flop / (ms * 1e-3) / 1e12, _clock_mhz(stamps)
        # cycles one SIMD spends per MFMA over the whole launch: 32768 flop per MFMA, 1024 SIMDs
        out[name] = {"tflops": tflops, "ms": ms, "clock_mhz": clock,
                     "cycles_per_mfma": 32768.0 * 1024 * clock * 1e6 / (tflops * 1e12)}
    return out


def mfma_probe_report(steps, warmup):
    """`--mfma-probe`: the measured matrix ceiling (zeros / N(0,1) operands, one and two waves per SIMD, with
    and without other arithmetic between the MFMAs) and, beside it, the prefill and MLA kernels of the
    benchmark built with clock stamps: their TFLOP/s, the shader clock they ran at, and what the matrix pipes
    could deliver at that clock."""
    lines = ["# matrix-pipe ceiling probe (ae_mfma_probe_kernel: 32x32x16 MFMAs back to back, alone or with the named other work "
             "between them) and the clock the attention kernels run at",
             "# columns: case, operands, TFLOP/s, shader clock MHz (s_memtime / s_memrealtime inside the kernel), "
             "SIMD cycles per MFMA, share of 2500 TFLOP/s"]
    rec = {}
    for tag, cfg in PROBE_CASES:
        r = mfma_probe(cfg)
        rec[tag] = r
        for ops, v in r.items():
            lines.append(f"{tag}, {ops}, {v['tflops']:.0f}, {v['clock_mhz']:.0f}, {v['cycles_per_mfma']:.1f}, "
                         f"{v['tflops'] / PEAK_MFMA_TFLOPS:.3f}")
    os.environ["AE_CLOCK_STAMPS"] = "1"
    lines.append("# columns: workload, TFLOP/s (HIP events), ms per launch, shader clock MHz over the launch's workgroups, "
                 "matrix-pipe rate at that clock TFLOP/s, kernel's share of it, share of 2500 TFLOP/s")
    for name in ("c2_causal", "c2_full", "c3_sigmoid", "c5_mla_decode"):
        r = measure(name, steps, warmup)
        clk = r.get("clock_mhz", float("nan"))
        tf = r["flops"] / (r["kernel_ms"] * 1e-3) / 1e12
        at_clock = MFMA_FLOP_PER_CLK * clk * 1e6 / 1e12
        rec[name] = {"tflops": tf, "ms": r["kernel_ms"], "clock_mhz": clk}
        if "phases_us" in r:
            rec[name]["phases_us"] = r["phases_us"]
            lines.append(f"#   {name} workgroup phases, microseconds: " +
                         ", ".join(f"{k} {v:.1f}" for k, v in r["phases_us"].items()))
        lines.append(f"{name}, {tf:.0f}, {r['kernel_ms']:.4f}, {clk:.0f}, {at_clock:.0f}, {tf / at_clock:.3f}, "
                     f"{tf / PEAK_MFMA_TFLOPS:.3f}")
    print("\n".join(lines))
    print(json.dumps({"mfma_probe": rec}), flush=True)


def cpu_baseline(name):
    """The CPU oracle on a bounded sample of the workload (one batch entry; heads in chunks so the
    [heads, S, S] fp32 score tensor stays below ~1 GiB), fp32 compute on the rounded inputs."""
    import torch
    from oracle import attention_ref as R
    threads = torch.get_num_threads()
    g = torch.Generator().manual_seed(0)
    if name == "c2_causal_bwd":
        H, S, D, chunk = 32, 4096, 128, 2
        q, k, v, do = (torch.randn(1, S, H, D, generator=g).half().float() for _ in range(4))
        t0 = time.perf_counter()
        for h0 in range(0, H, chunk):
            sl = slice(h0, h0 + chunk)
            R.softmax_attention_grads(q[:, :, sl], k[:, :, sl], v[:, :, sl], do[:, :, sl], causal=True)
        dt = time.perf_counter() - t0
        return {"value": 10.0 * H * S * S * D * 0.5 / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": f"oracle gradients on 1 of 2 batch entries (32 heads, S=4096, D=128, fp32), {dt:.2f} s, "
                          "reference flop convention"}
    if name in ("c2_causal", "c2_full", "c3_sigmoid"):
        H, S, D, chunk = 32, 4096, 128, 4
        q = torch.randn(1, S, H, D, generator=g).half().float()
        k = torch.randn(1, S, H, D, generator=g).half().float()
        v = torch.randn(1, S, H, D, generator=g).half().float()
        causal = name == "c2_causal"

        def run():
            for h0 in range(0, H, chunk):
                sl = slice(h0, h0 + chunk)
                if name == "c3_sigmoid":
                    R.sigmoid_attention(q[:, :, sl], k[:, :, sl], v[:, :, sl], bias=-math.log(S))
                else:
                    R.softmax_attention(q[:, :, sl], k[:, :, sl], v[:, :, sl], causal=causal)
        flops = 4.0 * H * S * S * D * (0.5 if causal else 1.0)
        R.softmax_attention(q[:, :256, :1], k[:, :256, :1], v[:, :256, :1])   # warm the thread pool
        passes, t0 = 0, time.perf_counter()
        while passes == 0 or time.perf_counter() - t0 < CPU_BASELINE_SECONDS:
            run()
            passes += 1
        dt = time.perf_counter() - t0
        return {"value": passes * flops / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": f"oracle/attention_ref.py on 1 of 2 batch entries (32 heads, S=4096, D=128, "
                          f"fp32), {passes} passes in {dt:.1f} s, reference flop convention"}
    if name in ("c4_gqa_decode", "gqa_decode_b1"):
        nb, Hq, Hkv, Skv, D = (8 if name == "c4_gqa_decode" else 1), 32, 8, 8192, 128
        q = torch.randn(nb, 1, Hq, D, generator=g).half().float()
        k = torch.randn(nb, Skv, Hkv, D, generator=g).half().float()
        v = torch.randn(nb, Skv, Hkv, D, generator=g).half().float()
        R.softmax_attention(q[:1], k[:1], v[:1])
        t0 = time.perf_counter()
        R.softmax_attention(q, k, v)
        dt = time.perf_counter() - t0
        by = 2.0 * nb * Skv * Hkv * D * 2
        return {"value": by / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": f"oracle on {nb} of {64 if name == 'c4_gqa_decode' else 1} batch entries (fp32 compute, "
                          f"fp16-sized KV bytes), {dt:.2f} s"}
    if name == "c5_mla_decode":
        nb, H, Skv, D, DV = 8, 128, 4096, 576, 512
        q = torch.randn(nb, H, DV, generator=g).bfloat16().float()
        qpe = torch.randn(nb, H, D - DV, generator=g).bfloat16().float()
        kv = torch.randn(nb, Skv, 1, DV, generator=g).bfloat16().float()
        kpe = torch.randn(nb, Skv, 1, D - DV, generator=g).bfloat16().float()
        R.mla_decode(q[:1], qpe[:1], kv[:1], kpe[:1])
        t0 = time.perf_counter()
        R.mla_decode(q, qpe, kv, kpe, scale=1 / math.sqrt(192))
        dt = time.perf_counter() - t0
        by = 1.0 * nb * Skv * D * 2
        return {"value": by / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": f"oracle on 8 of 128 batch entries (fp32 compute, bf16-sized KV bytes), {dt:.2f} s"}
    raise KeyError(name)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2_causal", choices=sorted(WORKLOADS))
    ap.add_argument("--no-extra", action="store_true", help="measure only --workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="instead of the benchmark line: measure the matrix-pipe ceiling (a pure MFMA loop on zero and "
                         "on N(0,1) operands) and the shader clock the prefill / MLA kernels run at")
    ap.add_argument("--probe-case", type=int, default=None, metavar="I",
                    help="with --mfma-probe: only case I of PROBE_CASES, on --probe-operands, --steps launches of ~1 ms "
                         "back to back (a steady load to read socket power and clocks against, e.g. with amd-smi metric -p)")
    ap.add_argument("--probe-operands", default="randn", choices=["zeros", "randn"])
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch one plain 256 MiB copy kernel (ae_copy_probe_kernel) so that a "
                         "hardware-counter run can scale FETCH_SIZE / WRITE_SIZE by a known transfer")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the attention forward path on ONE GPU; "
              "--gpus N with N > 1 is not supported (the path shards over batch/heads with no "
              "exchange, so N GPUs are N independent copies of this measurement).", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; there is no CPU fallback for the measured path.", file=sys.stderr)
        sys.exit(3)
    from core.runtime import hip_rt as rt
    info = rt.device_info(0)
    if a.mfma_probe and a.probe_case is not None:
        tag, cfg = PROBE_CASES[a.probe_case]
        r = mfma_probe(cfg, launches=a.steps, operands=(a.probe_operands,))[a.probe_operands]
        print(json.dumps({"mfma_probe_case": tag, "operands": a.probe_operands, "launches": a.steps, **r}), flush=True)
        return
    if a.mfma_probe:
        mfma_probe_report(a.steps, a.warmup)
        return

    head = measure(a.workload, a.steps, a.warmup)
    if a.copy_probe:
        copy_probe()
    unit = head["roofline"]["unit"]
    value = head["tflops"] if unit == "TFLOP/s" else head["gbs"]
    line = {
        "metric": "prefill TFLOP/s (causal S=4096 D=128 fp16) + decode GB/s; % of MI355X peak",
        "value": value, "unit": unit, "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "warmup_launches": head["warmup_launches"], "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": head["dtype"], "data": "synthetic",
        "config": {"workload": a.workload, **head["shape"]},
        "roofline": head["roofline"],
        "checked": head["checked"],
        "device": {"name": info["name"], "arch": info["arch"], "compute_units": info["compute_units"],
                   "clock_khz": info["clock_khz"]},
    }
    if "mfma_frac" in head:
        line["mfma_frac"] = head["mfma_frac"]
    if head["roofline"]["bound"] == "mfma":
        # beside (never instead of) the fraction of the published peak: what a pure MFMA loop reaches on this
        # chip on the same kind of operand data, and on zeros
        pr = mfma_probe({}, launches=10)
        line["mfma_ceiling_measured"] = {k: {"tflops": v["tflops"], "clock_mhz": v["clock_mhz"]} for k, v in pr.items()}
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(a.workload)
    if not a.no_extra:
        others = {}
        for name in WORKLOADS:
            if name == a.workload or name in ONLY_ON_REQUEST:
                continue
            r = measure(name, max(5, a.steps // 2), max(2, a.warmup // 2))
            others[name] = {"ms_per_step": r["ms_per_step"], "kernel_ms": r["kernel_ms"],
                            "tflops": r["tflops"], "gbs": r["gbs"], "roofline": r["roofline"],
                            "checked": r["checked"],
                            **({"mfma_frac": r["mfma_frac"]} if "mfma_frac" in r else {})}
        line["other_configs"] = others
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
