#!/usr/bin/env python3
"""Benchmark of the block-scaled FP4 GEMM path on one MI355X.

Follows the reference harness (reference ``benchmark/gemm/bench_amdgpu_gemm.py:23-68``):
``flops = 2*M*N*K``, warm-up launches, ONE launch captured in a graph and replayed (``:36-52``),
device time between two events around the replays, optional validation on the CPU
(``:62-68``).  Extended with the FP4 configurations, roofline fractions and a CPU baseline.
Operands are drawn from CPU generators with fixed seeds (reproducible without a GPU) and
quantised on the device.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--all] [--no-cpu] [--rotated-only] [--no-live-counters]
    python bench.py --m M --n N --k K [--validate]      # one MXFP4 GEMM, the reference's CLI (:75-81)

Prints ONE JSON line.  ``value`` is the MXFP4 GEMM throughput (TFLOP/s) at
M=8192, N=14336, K=4096 with operands resident in HBM; the small-M decode GEMM
(M=16, N=28672, K=4096) is reported in ``decode`` as achieved HBM GB/s, the NVFP4 and the
grouped (MoE) configurations in ``nvfp4`` and ``grouped``.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from avelang_amd import (  # noqa: E402
    gather_rows_mxfp4,
    moe_combine_top2,
    gemm_mxfp4_blocked_scales_transposed_b,
    gemm_mxfp4_swiglu_quant_transposed_b,
    gemm_mxfp4_swiglu_transposed_b,
    pad_k_mxfp4,
    scales_to_blocked,
    grouped_gemm_mxfp4_swiglu_quant_transposed_b,
    moe_route_top2,
    quantize_mxfp4, quantize_nvfp4,
    gemm_mxfp4_transposed_b,
    gemm_nvfp4_transposed_b,
    grouped_gemm_mxfp4_transposed_b,
)
from avelang_amd import testing as synth  # noqa: E402

FP4_PEAK_TFLOPS = 10100.0   # MI355X dense FP4 MFMA, published
F16_PEAK_TFLOPS = 2500.0    # MI355X dense bf16/fp16 MFMA, published
HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published



COUNTERS_FILE = "profiles/traffic.json"


def _counters(kernel):
    try:
        with open(os.path.join(ROOT, COUNTERS_FILE)) as f:
            return json.load(f)[kernel]
    except (OSError, KeyError, ValueError):
        return {}


def measured_traffic(kernel):
    """HBM bytes per launch measured with rocprofv3 --pmc in a separate run (profiles/traffic.json);
    None when no measurement is on file."""
    t = _counters(kernel)
    return t["fetch_bytes"] + t["write_bytes"] if "fetch_bytes" in t and "write_bytes" in t else None


def _pmc_child(counters, bench_args, kernel, timeout_s=150):
    """Per-dispatch counter values of `kernel` from a child process: `rocprofv3 --pmc <counters> -- python3 bench.py
    <bench_args>` (the program directly behind `--`, counters in a run of their own).  Returns a list of dicts
    {counter: value, "ns": kernel duration}, or [] when the profiler is missing, fails or times out, or when this
    process is itself being profiled."""
    import csv
    import shutil
    import signal
    import subprocess
    import tempfile
    if shutil.which("rocprofv3") is None:
        return []
    if any(k.startswith("ROCPROF") or k.startswith("ROCP_") for k in os.environ) or "rocprofiler" in os.environ.get("LD_PRELOAD", ""):
        return []
    out = tempfile.mkdtemp(prefix="ave_fp4_pmc_", dir="/tmp")
    try:
        cmd = ["rocprofv3", "--pmc", *counters, "--output-format", "csv", "-d", out, "-o", "b", "--", sys.executable,
               os.path.join(ROOT, "bench.py"), *bench_args]
        # The profiler starts the benchmark as a child of its own.  Both run in a session (= process group) of their
        # own, so that on a time-out, an error or a helper the profiler leaves behind the WHOLE group can be ended:
        # killing the profiler alone would leave the benchmark holding the GPU next to the legs that follow.
        child = subprocess.Popen(cmd, cwd=ROOT, env=dict(os.environ, TMPDIR="/tmp"), stdout=subprocess.DEVNULL,
                                 stderr=subprocess.DEVNULL, start_new_session=True)
        try:
            rc = child.wait(timeout=timeout_s)
        except subprocess.TimeoutExpired:
            rc = None
        finally:
            try:
                os.killpg(child.pid, signal.SIGKILL)   # the group leader's pid is the group's id; gone already: fine
            except (ProcessLookupError, PermissionError):
                pass
            child.wait()
        if rc != 0:
            return []
        per = {}
        for root_dir, _, files in os.walk(out):
            for name in files:
                if not name.endswith("counter_collection.csv"):
                    continue
                with open(os.path.join(root_dir, name)) as f:
                    for r in csv.DictReader(f):
                        if kernel not in r["Kernel_Name"]:
                            continue
                        d = per.setdefault(r["Dispatch_Id"], {"ns": int(r["End_Timestamp"]) - int(r["Start_Timestamp"])})
                        d[r["Counter_Name"]] = float(r["Counter_Value"])
        return [d for d in per.values() if all(c in d for c in counters) and d["ns"] > 0]
    except (OSError, subprocess.SubprocessError, KeyError, ValueError):
        return []
    finally:
        shutil.rmtree(out, ignore_errors=True)


# what FETCH_SIZE and WRITE_SIZE (KiB per dispatch) read for a plain 256 MiB device copy, relative to the bytes moved
FETCH_SIZE_SCALE, WRITE_SIZE_SCALE = 2.0, 1.0
_SQ = ["SQ_VALU_MFMA_BUSY_CYCLES", "SQ_BUSY_CU_CYCLES"]


def live_leg_counters(device, leg, kernel, mfma=True, extra_args=()):
    """Counters of one leg's kernel measured NOW, in child processes of this run (`rocprofv3 --pmc ... -- python3
    bench.py --only <leg>`): the bytes that cross the L2 boundary per launch (FETCH_SIZE and WRITE_SIZE, which do not
    fit one pass: two children, scaled by the copy calibration) and, for the MFMA-bound legs, the matrix-core busy
    fraction and the average shader clock (busy = MFMA cycles / (4 SIMDs x CU-busy cycles); clock = CU-busy cycles /
    (compute units x kernel time); these two SQ counters ride with FETCH_SIZE's three TCC counters in the first child,
    and get a child of their own if that pass yields nothing).  {} for what could not be measured."""
    import statistics
    args = ["--only", leg, "--no-cpu", "--steps", "10", "--warmup", "5", *extra_args]
    out = {}
    first = _pmc_child(["FETCH_SIZE"] + (_SQ if mfma else []), args, kernel)
    sq_rows, fetch = (first, first) if mfma else ([], first)
    if mfma and len(first) < 5:
        sq_rows = _pmc_child(_SQ, args, kernel)
        fetch = _pmc_child(["FETCH_SIZE"], args, kernel) if sq_rows else []
    if len(sq_rows) >= 5:
        cus = torch.cuda.get_device_properties(device).multi_processor_count
        out.update({"mfma_busy_frac": statistics.median(d["SQ_VALU_MFMA_BUSY_CYCLES"] / (4.0 * d["SQ_BUSY_CU_CYCLES"]) for d in sq_rows),
                    "shader_clock_ghz": statistics.median(d["SQ_BUSY_CU_CYCLES"] / cus / d["ns"] for d in sq_rows),
                    "kernel_us_under_counters": statistics.median(d["ns"] for d in sq_rows) / 1e3, "dispatches": len(sq_rows),
                    "counters_from": "rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES in a child process of this run"})
    write = _pmc_child(["WRITE_SIZE"], args, kernel) if len(fetch) >= 5 else []
    if len(fetch) >= 5 and len(write) >= 5:
        f = statistics.median(d["FETCH_SIZE"] for d in fetch) * 1024.0 * FETCH_SIZE_SCALE
        w = statistics.median(d["WRITE_SIZE"] for d in write) * 1024.0 * WRITE_SIZE_SCALE
        out.update({"traffic": int(f + w), "fetch_bytes": int(f), "write_bytes": int(w),
                    "traffic_from": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE in child processes of this run "
                                    "(KiB per dispatch x 2.0 / x 1.0, the factors a 256 MiB device copy gives)"})
    return out


def apply_live_counters(roof, live):
    """Puts a leg's live counters into its roofline object; what the object quoted from the file on disk moves to
    `counters_on_file` / `traffic_on_file` so that both stay visible."""
    if "mfma_busy_frac" in live:
        on_file = {k: roof.pop(k) for k in ("mfma_busy_frac", "shader_clock_ghz", "counters_from") if k in roof}
        if on_file:
            roof["counters_on_file"] = on_file
        roof.update({k: live[k] for k in ("mfma_busy_frac", "shader_clock_ghz", "kernel_us_under_counters", "dispatches", "counters_from")})
    if "traffic" in live:
        roof["traffic_on_file"] = roof.get("traffic")
        roof.update({k: live[k] for k in ("traffic", "fetch_bytes", "write_bytes", "traffic_from")})
    elif roof.get("traffic") is not None:
        roof["traffic_from"] = COUNTERS_FILE


def measured_counters(kernel):
    """Matrix-core busy fraction and average shader clock from the rocprofv3 --pmc run on file for this kernel
    (profiles/traffic.json), tagged with where they come from: they describe the profiled run, not this one."""
    t = _counters(kernel)
    out = {k: t[k] for k in ("mfma_busy_frac", "shader_clock_ghz") if k in t}
    if t:
        out["counters_from"] = COUNTERS_FILE
    return out


METRIC = "MXFP4 GEMM TFLOP/s (% FP4 MFMA peak) at 8192x14336x4096; M=16 HBM GB/s"


def mx_bytes(m, n, k):
    return (m + n) * k // 2 + (m + n) * k // 32 + m * n * 2


def _events_ms(fn, steps, warmup):
    """Exactly `steps` launches between two events on the current stream, bracketed by syncs."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_time(e1) / steps, wall / steps


def _graph_us(calls, steps, warmup):
    """Per-call device time of short kernels: the calls (one per rotated buffer) are captured in one graph
    and replayed, so that host launch overhead (10-20 us per Python call) is not what gets measured."""
    for c in calls:
        c()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=torch.cuda.Stream()):
        for c in calls:
            c()
    torch.cuda.synchronize()
    ms, _ = _events_ms(graph.replay, max(1, steps // len(calls)), max(1, warmup // len(calls)))
    return ms * 1e3 / len(calls)


class GraphLeg:
    """The reference's protocol (bench_amdgpu_gemm.py:31-52) in two halves, so that several legs can be prepared first
    and then timed back to back with no capture, allocation or other host work between their launches: the
    constructor runs the launch once eagerly, captures ONE launch in a graph and replays it once (which uploads the
    graph); :meth:`time` replays it `warmup` times untimed and exactly `steps` times between two events, bracketed by
    synchronisation."""

    def __init__(self, fn):
        fn()
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=torch.cuda.Stream()):
            fn()
        torch.cuda.synchronize()
        self.graph.replay()
        torch.cuda.synchronize()

    def time(self, steps, warmup):
        return _events_ms(self.graph.replay, steps, warmup)


def _graph_replay_ms(fn, steps, warmup):
    return GraphLeg(fn).time(steps, warmup)


def cpu_randn(shape, seed, device, std=1.0, generator=None):
    """fp32 N(0, std) drawn on the CPU from a generator with a fixed seed, then uploaded: the same tensor on any
    machine, with or without a GPU."""
    g = generator or torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g, dtype=torch.float32)
    if std != 1.0:
        x *= std
    return x.to(device)


def make_prefill(device, m=8192, n=14336, k=4096, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = synth.activations_with_outliers(m, k, g, "cpu").to(device)
    w = cpu_randn((n, k), seed, device, std=0.02, generator=g)
    a, a_s = synth.quantize_mxfp4(x)
    b, b_s = synth.quantize_mxfp4(w)
    return a, a_s, b, b_s


def prepare_prefill(device, operands=None):
    m, n, k = 8192, 14336, 4096
    a, a_s, b, b_s = operands or make_prefill(device, m, n, k)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    return {"leg": GraphLeg(lambda: gemm_mxfp4_transposed_b(a, a_s, b, b_s, out=out)), "tensors": (a, a_s, b, b_s, out),
            "shape": (m, n, k)}


def bench_prefill(device, steps, warmup, operands=None, settle_steps=0, prepared=None):
    pre = prepared or prepare_prefill(device, operands)
    m, n, k = pre["shape"]
    ms, wall_ms = pre["leg"].time(steps, warmup)
    tflops = 2.0 * m * n * k / (ms * 1e-3) / 1e12
    res = {"ms": ms, "wall_ms": wall_ms, "tflops": tflops, "tensors": pre["tensors"], "shape": (m, n, k)}
    if settle_steps:
        # The same replays continued: the GPU's power management takes some 50-100 ms of a load to settle on its
        # clock for it (from idle it overshoots, throttles hard, then recovers), far longer than a few dozen steps.
        pre["leg"].time(settle_steps, 0)
        settled_ms, _ = pre["leg"].time(settle_steps, 0)
        res["settled"] = {"ms_per_step": settled_ms, "tflops": 2.0 * m * n * k / (settled_ms * 1e-3) / 1e12,
                          "steps": settle_steps, "after_untimed_steps": steps + settle_steps}
    return res


def prepare_prefill_cold(device, operands, copies=9):
    """The headline GEMM as a model's layers run it: every launch on a weight matrix that has left the caches --
    `copies` distinct B buffers (the quantised rows rolled by i; 9 x 31 MB is more than the 256 MB last-level cache
    holds, and each launch's 235 MB of C sweep it as well), one launch each, captured in ONE graph."""
    a, a_s, b, b_s = operands
    m, n, k = a.shape[0], b.shape[0], a.shape[1] * 2
    ws = [(b, b_s)] + [(torch.roll(b, i, 0), torch.roll(b_s, i, 0)) for i in range(1, copies)]
    out = torch.empty((m, n), dtype=torch.bfloat16, device=device)

    def launches():
        for w, w_s in ws:
            gemm_mxfp4_transposed_b(a, a_s, w, w_s, out=out)

    return {"leg": GraphLeg(launches), "copies": copies, "shape": (m, n, k), "keep": (ws, out)}


def bench_prefill_cold(pre, steps, warmup):
    copies = pre["copies"]
    m, n, k = pre["shape"]
    ms, _ = pre["leg"].time(max(1, steps // copies + 1), max(1, warmup // copies))
    per = ms / copies
    return {"workload": "the headline GEMM with its weights streamed from HBM: one graph of %d launches, each on a weight "
                        "buffer of its own (what a model's layers see; the headline replays ONE cache-resident matrix, "
                        "as the reference benchmark does)" % copies,
            "weight_buffers_rotated": copies, "ms_per_launch": per, "value": 2.0 * m * n * k / (per * 1e-3) / 1e12,
            "unit": "TFLOP/s", "frac_fp4_peak": 2.0 * m * n * k / (per * 1e-3) / 1e12 / FP4_PEAK_TFLOPS}


def prepare_k_tail(device, m=8192, n=14336, k=4128):
    """The headline shape with a K that is no multiple of the 256-element stage (one 32-element block more)."""
    a, a_s = synth.quantize_mxfp4(cpu_randn((m, k), 10, device))
    b, b_s = synth.quantize_mxfp4(cpu_randn((n, k), 11, device, std=0.02))
    out = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    # the same operands padded with zero blocks to a multiple of 512 (what a caller can do: weights once, activations
    # by the quantiser): same sums, rows that are whole cache lines
    k_pad = (k + 511) // 512 * 512
    pa, pa_s = pad_k_mxfp4(a, a_s, k_pad)
    pb, pb_s = pad_k_mxfp4(b, b_s, k_pad)
    return {"leg": GraphLeg(lambda: gemm_mxfp4_transposed_b(a, a_s, b, b_s, out=out)), "shape": (m, n, k), "k_pad": k_pad,
            "padded_leg": GraphLeg(lambda: gemm_mxfp4_transposed_b(pa, pa_s, pb, pb_s, out=out)),
            "keep": (a, a_s, b, b_s, out, pa, pa_s, pb, pb_s)}


def bench_k_tail(pre, steps, warmup):
    m, n, k = pre["shape"]
    ms, _ = pre["leg"].time(steps, warmup)
    ms_pad, _ = pre["padded_leg"].time(steps, warmup)
    tf = 2.0 * m * n * k / (ms * 1e-3) / 1e12
    return {"workload": "MXFP4 GEMM with a K tail: K = 4096 + 32, row pitch no multiple of the 128-byte line",
            "M": m, "N": n, "K": k, "ms_per_step": ms, "value": tf, "unit": "TFLOP/s",
            "operands_padded_with_zero_blocks": {"K_padded": pre["k_pad"], "ms_per_step": ms_pad,
                                                 "value": 2.0 * m * n * k / (ms_pad * 1e-3) / 1e12, "unit": "TFLOP/s of the unpadded problem"},
            "roofline": {"bound": "mfma", "achieved": tf, "peak": FP4_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tf / FP4_PEAK_TFLOPS,
                         "traffic": None, "kernel": "mx_tile_kernel (K tail form)", "flops_per_launch": 2.0 * m * n * k,
                         "algorithmic_bytes_per_launch": mx_bytes(m, n, k)}}


def bench_blocked_scales(device, operands, steps, warmup):
    """The headline GEMM and the decode GEMM with their scale tensors in the 128 x 4 blocked layout, read by the kernels
    directly, beside the same launches on row-major scales (alternately, same operands, graph replays)."""
    res = {}
    a, a_s, b, b_s = operands
    out = torch.empty((a.shape[0], b.shape[0]), dtype=torch.bfloat16, device=device)
    ab, bb = scales_to_blocked(a_s), scales_to_blocked(b_s)
    legs = {"row_major": GraphLeg(lambda: gemm_mxfp4_transposed_b(a, a_s, b, b_s, out=out)),
            "blocked": GraphLeg(lambda: gemm_mxfp4_blocked_scales_transposed_b(a, ab, b, bb, out=out))}
    for _ in range(2):
        for name, leg in legs.items():
            ms, _ = leg.time(steps, warmup)
            res.setdefault("prefill_8192x14336x4096_ms", {})[name] = ms
    m, n, k = 16, 28672, 4096
    x, x_s = synth.quantize_mxfp4(cpu_randn((m, k), 2, device))
    w, w_s = synth.quantize_mxfp4(cpu_randn((n, k), 3, device, std=0.02))
    ws = [(torch.roll(w, i, 0), torch.roll(w_s, i, 0)) for i in range(10)]
    wb = [scales_to_blocked(s_) for _, s_ in ws]
    xb = scales_to_blocked(x_s)
    o = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    res["decode_16x28672x4096_us"] = {
        "row_major": _graph_us([lambda q=q, s_=s_: gemm_mxfp4_transposed_b(x, x_s, q, s_, out=o) for q, s_ in ws], 400, 80),
        "blocked": _graph_us([lambda q=q, s_=s_: gemm_mxfp4_blocked_scales_transposed_b(x, xb, q, s_, out=o)
                              for (q, _), s_ in zip(ws, wb)], 400, 80)}
    return res


def bench_prefill_swiglu(device, steps, warmup):
    """Gate+up projection of the MLP with the SwiGLU activation: fused in the LDS-staged kernel's epilogue, and
    the same result by the plain GEMM over the 2 x 14336 weight rows followed by torch's silu and product."""
    m, n, k = 8192, 14336, 4096
    g = torch.Generator(device=device).manual_seed(5)
    a, a_s = synth.quantize_mxfp4(torch.randn((m, k), generator=g, device=device))
    w = torch.randn((2 * n, k), generator=g, device=device, dtype=torch.float32) * 0.02
    b, b_s = synth.quantize_mxfp4(w)
    del w
    out = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    fused_ms, _ = _events_ms(lambda: gemm_mxfp4_swiglu_transposed_b(a, a_s, b, b_s, out=out), steps, warmup)
    wide = torch.empty((m, 2 * n), dtype=torch.bfloat16, device=device)

    def unfused():
        gemm_mxfp4_transposed_b(a, a_s, b, b_s, out=wide)
        torch.mul(torch.nn.functional.silu(wide[:, :n]), wide[:, n:], out=out)

    unfused_ms, _ = _events_ms(unfused, max(10, steps // 4), max(2, warmup // 4))
    # the same with the next GEMM's MXFP4 quantiser behind it: one launch, and the fused GEMM followed by the quantiser
    q = torch.empty((m, n // 2), dtype=torch.uint8, device=device)
    q_s = torch.empty((m, n // 32), dtype=torch.uint8, device=device)
    fq_ms, _ = _events_ms(lambda: gemm_mxfp4_swiglu_quant_transposed_b(a, a_s, b, b_s, out=q, out_scale=q_s), steps, warmup)

    def two_calls():
        gemm_mxfp4_swiglu_transposed_b(a, a_s, b, b_s, out=out)
        quantize_mxfp4(out, q, q_s)

    two_ms, _ = _events_ms(two_calls, max(10, steps // 2), max(2, warmup // 2))
    flop = 2.0 * m * 2 * n * k
    return {"shape": (m, n, k), "fused_ms": fused_ms, "fused_tflops": flop / (fused_ms * 1e-3) / 1e12,
            "gemm_then_torch_silu_mul_ms": unfused_ms, "fused_with_quantiser_ms": fq_ms,
            "fused_with_quantiser_tflops": flop / (fq_ms * 1e-3) / 1e12, "fused_then_quantiser_kernel_ms": two_ms}


def bench_mfma_ceiling(device, operands, f16=False, settle_launches=0):
    """Rate of a loop of nothing but scaled FP4 MFMAs (two waves per SIMD, operands kept in registers), on
    fragments of zeros and on fragments of the GEMM's own quantised operands: the matrix-core clock under load
    depends on how many operand bits toggle, so the second figure is what a GEMM on this data can approach.
    With `settle_launches`, the probe on the GEMM's operands is then launched that many more times untimed (about
    8 ms each: several hundred ms of continuous matrix-core load, the treatment the GEMM's own `settled_clock`
    figure gets) and timed again: `gemm_operands_settled` is the ceiling at the clock the power management settles
    on, where the first figure may still sit in the transient after the idle period before it."""
    import ctypes
    from avelang_amd import _lib
    lib = _lib.load()
    sink = torch.zeros(1, dtype=torch.float32, device=device)
    workgroups, iters = 256 * 4, (1500 if f16 else 6000)
    probe = lib.ave_fp4_debug_mfma_rate_f16 if f16 else lib.ave_fp4_debug_mfma_rate
    flop = ctypes.c_double(0.0)
    out = {}
    a, b = operands
    mixed = torch.cat([a.reshape(-1)[: 4 << 20], b.reshape(-1)[: 4 << 20]]).contiguous()
    for name, codes in (("zeros", torch.zeros(1 << 20, dtype=torch.uint8, device=device)), ("gemm_operands", mixed)):
        def call():
            rc = probe(codes.data_ptr(), codes.numel(), workgroups, iters, sink.data_ptr(),
                       torch.cuda.current_stream().cuda_stream, ctypes.byref(flop))
            if rc != 0:
                raise RuntimeError(lib.ave_fp4_last_error().decode())
        ms, _ = _events_ms(call, 3, 1)
        out[name] = flop.value / (ms * 1e-3) / 1e12
        if name == "gemm_operands" and settle_launches:
            ms, _ = _events_ms(call, 10, settle_launches)
            out["gemm_operands_settled"] = flop.value / (ms * 1e-3) / 1e12
            out["settled_after_untimed_launches"] = settle_launches
            out["ms_per_probe_launch"] = ms
    return out


def bench_stream_read(device, algorithmic_bytes, total_bytes=1 << 30, copies=10, result_bytes=0):
    """What a kernel that only reads gets out of HBM on this GPU: (1) 1 GiB (four times the last-level cache) read
    once per launch, 16 bytes per lane -- the sustained rate; (2) the decode GEMM's own byte count read from `copies`
    rotated buffers, one launch each in a graph, exactly as the GEMM is timed -- the time per launch that a kernel of
    this size cannot go below, start-up and drain included; (3) with `result_bytes`, the same read followed by that many
    bytes of coalesced stores: the floor for a kernel that also has the GEMM's result to write."""
    from avelang_amd import _lib
    lib = _lib.load()
    sink = torch.zeros(1, dtype=torch.int32, device=device)

    def reader(buf, workgroups):
        def call():
            rc = lib.ave_fp4_debug_stream_read(buf.data_ptr(), buf.numel(), workgroups, sink.data_ptr(),
                                               torch.cuda.current_stream().cuda_stream)
            if rc != 0:
                raise RuntimeError(lib.ave_fp4_last_error().decode())
        return call

    src = torch.full((total_bytes,), 3, dtype=torch.uint8, device=device)
    ms, _ = _graph_replay_ms(reader(src, 256 * 16), 20, 5)
    del src
    gbs = total_bytes / (ms * 1e-3) / 1e9
    nbytes = algorithmic_bytes // 16 * 16
    bufs = [torch.full((nbytes,), i + 1, dtype=torch.uint8, device=device) for i in range(copies)]
    same_size = {}
    for workgroups in (256, 512, 4096):
        same_size[str(workgroups)] = _graph_us([reader(b, workgroups) for b in bufs], 40 * copies, 8 * copies)
    best = min(same_size.values())
    same = {"bytes": nbytes, "buffers_rotated": copies, "us_per_launch_by_workgroups": same_size,
            "us_per_launch": best, "gbs": nbytes / best / 1e3, "frac_hbm_peak": nbytes / best / 1e3 / HBM_PEAK_GBS}
    if result_bytes:
        result = torch.zeros(result_bytes // 16 * 16, dtype=torch.uint8, device=device)

        def read_write(buf, workgroups):
            def call():
                rc = lib.ave_fp4_debug_stream_read_write(buf.data_ptr(), buf.numel() - result.numel(), result.data_ptr(),
                                                         result.numel(), workgroups, sink.data_ptr(),
                                                         torch.cuda.current_stream().cuda_stream)
                if rc != 0:
                    raise RuntimeError(lib.ave_fp4_last_error().decode())
            return call

        with_result = {str(w): _graph_us([read_write(b, w) for b in bufs], 40 * copies, 8 * copies) for w in (256, 512, 4096)}
        same["result_bytes"] = result.numel()
        same["us_per_launch_with_result_by_workgroups"] = with_result
        same["us_per_launch_with_result"] = min(with_result.values())
    return {"kernel": "stream_read_kernel", "bytes": total_bytes, "gbs": gbs, "frac_hbm_peak": gbs / HBM_PEAK_GBS,
            "same_bytes_as_the_gemm": same}


def bench_shape_grouped(device, experts, rows, n, k, steps, warmup, variant=0):
    """One grouped MXFP4 GEMM: `experts` experts of `rows` rows each against weights [experts, n, k] of their own
    (--m ROWS --n N --k K --grouped E).  Random codes under scale bytes around 2^0: the timing needs no oracle."""
    g = torch.Generator(device=device).manual_seed(1)
    total = experts * rows
    a = torch.randint(0, 256, (total, k // 2), dtype=torch.uint8, device=device, generator=g)
    a_s = torch.randint(120, 130, (total, k // 32), dtype=torch.uint8, device=device, generator=g)
    b = torch.randint(0, 256, (experts, n, k // 2), dtype=torch.uint8, device=device, generator=g)
    b_s = torch.randint(120, 130, (experts, n, k // 32), dtype=torch.uint8, device=device, generator=g)
    ro = torch.arange(0, total + 1, rows, dtype=torch.int32, device=device)
    out = torch.empty((total, n), dtype=torch.bfloat16, device=device)
    ms, _ = _graph_replay_ms(lambda: grouped_gemm_mxfp4_transposed_b(a, a_s, b, b_s, ro, out=out, variant=variant), steps, warmup)
    weights = experts * n * (k // 2 + k // 32)
    return {"metric": "grouped MXFP4 GEMM", "experts": experts, "rows_per_expert": rows, "N": n, "K": k, "time_ms": ms,
            "ms_per_step": ms, "value": 2.0 * total * n * k / (ms * 1e-3) / 1e12, "unit": "TFLOP/s",
            "weights_gbs": weights / (ms * 1e-3) / 1e9, "steps": steps, "warmup": warmup, "variant": variant}


def bench_shape_nvfp4(device, m, n, k, steps, warmup, rotate=1, variant=0):
    """One NVFP4 GEMM of a given shape, timed like bench_shape (--m --n --k --nvfp4 [--rotate B --variant V])."""
    a, a_s, a_g = synth.quantize_nvfp4(cpu_randn((m, k), 0, device))
    b, b_s, b_g = synth.quantize_nvfp4(cpu_randn((n, k), 1, device, std=0.02))
    out = torch.zeros((m, n), dtype=torch.bfloat16, device=device)
    ws = [(b, b_s)] + [(torch.roll(b, i, 0), torch.roll(b_s, i, 0)) for i in range(1, rotate)]

    def launches():
        for w, w_s in reversed(ws):
            gemm_nvfp4_transposed_b(a, a_s, a_g, w, w_s, b_g, out=out, variant=variant)

    ms, _ = _graph_replay_ms(launches, max(1, steps // rotate), max(1, warmup // rotate))
    ms /= rotate
    nbytes = m * (k // 2 + k // 16) + n * (k // 2 + k // 16) + 2 * m * n + 8
    return {"metric": "NVFP4 GEMM", "M": m, "N": n, "K": k, "time_ms": ms, "ms_per_step": ms,
            "value": 2.0 * m * n * k / (ms * 1e-3) / 1e12, "unit": "TFLOP/s", "bandwidth_gbs": nbytes / (ms * 1e-3) / 1e9,
            "steps": steps, "warmup": warmup, "weight_buffers_rotated": rotate, "variant": variant}


def bench_shape(device, m, n, k, steps, warmup, validate, rotate=1, variant=0):
    """One MXFP4 GEMM of a given shape, the reference benchmark's command line (bench_amdgpu_gemm.py:23-68, :75-81):
    seeded N(0,1) x N(0,0.02) operands, warm-up, graph replay, 2*M*N*K flop; --validate compares with the CPU
    recipe (dequantise, fp32 matmul, bf16) as the reference does, and with the stated fp64 bound.  `rotate` > 1: the
    graph holds that many launches, each on a weight buffer of its own (the quantised rows rolled by i), so that the
    weights come from HBM and not from the last-level cache; `variant` forces a kernel (ave_fp4_variant)."""
    a, a_s = synth.quantize_mxfp4(cpu_randn((m, k), 0, device))
    b, b_s = synth.quantize_mxfp4(cpu_randn((n, k), 1, device, std=0.02))
    out = torch.zeros((m, n), dtype=torch.bfloat16, device=device)
    ws = [(b, b_s)] + [(torch.roll(b, i, 0), torch.roll(b_s, i, 0)) for i in range(1, rotate)]

    def launches():
        for w, w_s in reversed(ws):   # the last launch is the one on the unrolled weights, which --validate checks
            gemm_mxfp4_transposed_b(a, a_s, w, w_s, out=out, variant=variant)

    ms, _ = _graph_replay_ms(launches, max(1, steps // rotate), max(1, warmup // rotate))
    ms /= rotate
    res = {"metric": "MXFP4 GEMM", "M": m, "N": n, "K": k, "time_ms": ms, "ms_per_step": ms,
           "value": 2.0 * m * n * k / (ms * 1e-3) / 1e12, "unit": "TFLOP/s",
           "bandwidth_gbs": mx_bytes(m, n, k) / (ms * 1e-3) / 1e9, "steps": steps, "warmup": warmup,
           "weight_buffers_rotated": rotate, "variant": variant}
    res["frac_fp4_peak"] = res["value"] / FP4_PEAK_TFLOPS
    if validate:
        from oracle import fp4_oracle as orc
        import numpy as np
        a_np, as_np, b_np, bs_np = (t.cpu().numpy() for t in (a, a_s, b, b_s))
        adq, bdq = orc.dequantize_mxfp4(a_np, as_np), orc.dequantize_mxfp4(b_np, bs_np)
        expected = (torch.from_numpy(adq) @ torch.from_numpy(bdq).T).to(torch.bfloat16)
        actual = out.cpu()
        res["validation_max_abs_diff"] = (actual.float() - expected.float()).abs().max().item()
        if not torch.allclose(actual.float(), expected.float(), rtol=1e-1, atol=1e-1):      # the reference's test (:66)
            raise AssertionError(f"Validation failed (max abs diff {res['validation_max_abs_diff']}).")
        if m * n * k <= 1 << 34:   # the stated bound against fp64, where the fp64 product is affordable
            a64, b64 = adq.astype(np.float64), bdq.astype(np.float64)
            ok, rep = orc.check_bf16_against_fp64(actual.view(torch.uint16).numpy(), a64 @ b64.T, np.abs(a64) @ np.abs(b64).T, k)
            if not ok:
                raise AssertionError(f"Validation against fp64 failed: {rep}")
            res["validation_fp64_bound"] = "ok"
    return res


def bench_decode(device, steps, warmup, copies=10, shape=(16, 28672, 4096), swiglu=False, split_k=True, variant=0,
                 rotated_only=False):
    """M=16 decode GEMM.  The 62 MB of weights fit in the 256 MB last-level cache, so the graph
    walks over `copies` distinct weight buffers (>= 600 MB) and every launch reads from HBM;
    the single-buffer (cache-resident) figure is reported next to it."""
    m, n, k = shape
    g = torch.Generator().manual_seed(2)
    a, a_s = synth.quantize_mxfp4(cpu_randn((m, k), 2, device, generator=g))
    # one CPU-seeded weight matrix; the rotated buffers are its quantised rows rolled by i (distinct buffers are what
    # defeats the cache, and every one of them is reproducible from the seed)
    wq, wq_s = synth.quantize_mxfp4(cpu_randn((n, k), 2, device, std=0.02, generator=g))
    ws = [(wq, wq_s)] + [(torch.roll(wq, i, 0), torch.roll(wq_s, i, 0)) for i in range(1, copies)]
    out = torch.empty((m, n // 2 if swiglu else n), dtype=torch.bfloat16, device=device)
    if swiglu:
        def gemm(*operands, out):
            return gemm_mxfp4_swiglu_transposed_b(*operands, out=out, variant=variant)
    else:
        def gemm(*operands, out):
            return gemm_mxfp4_transposed_b(*operands, out=out, split_k=split_k, variant=variant)

    def capture(bufs):
        graph = torch.cuda.CUDAGraph()
        stream = torch.cuda.Stream()
        for b, b_s in bufs:  # warm every buffer once outside capture
            gemm(a, a_s, b, b_s, out=out)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            for b, b_s in bufs:
                gemm(a, a_s, b, b_s, out=out)
        torch.cuda.synchronize()
        return graph

    res = {}
    for name, bufs in (("hbm", ws),) + (() if rotated_only else (("cached", [ws[0]] * copies),)):
        graph = capture(bufs)
        reps = max(1, steps // copies)
        ms, _ = _events_ms(graph.replay, reps, max(1, warmup // copies))
        per_launch = ms / copies
        byts = mx_bytes(m, n, k) - (m * n if swiglu else 0)   # fused: half as many bf16 outputs
        res[name] = {"us": per_launch * 1e3, "gbs": byts / (per_launch * 1e-3) / 1e9}
    res["shape"] = (m, n, k)
    res["copies"] = copies
    return res


def bench_down_batched(device, rows=(128, 256, 512, 1024)):
    """A few hundred activation rows against the down projection's weights (16 output tiles of 256 x 256 for
    256 compute units): K split over the idle units through a workspace against one workgroup per tile."""
    res = {}
    for m in rows:
        split = bench_decode(device, 240, 48, copies=24, shape=(m, 4096, 14336))
        whole = bench_decode(device, 240, 48, copies=24, shape=(m, 4096, 14336), split_k=False)
        res["M=%d" % m] = {"us_per_launch": split["hbm"]["us"], "us_per_launch_unsplit": whole["hbm"]["us"],
                           "hbm_gbs": split["hbm"]["gbs"], "tflops": 2.0 * m * 4096 * 14336 / split["hbm"]["us"] / 1e6}
        torch.cuda.empty_cache()
    return res


def bench_gate_up_batched(device, rows=(128, 256)):
    """65..256 activation rows against the gate/up weights (N = 28672, K = 4096; 112 tiles of 256 x 256 for 256
    compute units): the narrow-tile kernel (128 x 128 tiles with four stage buffers up to 128 rows, 256 x 128 tiles
    with three above) against the 256 x 256 tile kernel."""
    res = {}
    for m in rows:
        narrow = bench_decode(device, 200, 40, shape=(m, 28672, 4096))
        wide = bench_decode(device, 200, 40, shape=(m, 28672, 4096), variant=2)
        res["M=%d" % m] = {"us_per_launch": narrow["hbm"]["us"], "us_per_launch_256x256_tiles": wide["hbm"]["us"],
                           "hbm_gbs": narrow["hbm"]["gbs"], "frac_hbm_peak": narrow["hbm"]["gbs"] / HBM_PEAK_GBS,
                           "tflops": 2.0 * m * 28672 * 4096 / narrow["hbm"]["us"] / 1e6}
        if m == 128:
            res["M=128"]["roofline"] = {"bound": "hbm", "achieved": narrow["hbm"]["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                        "frac": narrow["hbm"]["gbs"] / HBM_PEAK_GBS, "traffic": measured_traffic("mx_narrow_kernel"),
                                        "kernel": "mx_narrow_kernel", "algorithmic_bytes_per_launch": mx_bytes(m, 28672, 4096)}
        fused = bench_decode(device, 200, 40, shape=(m, 28672, 4096), swiglu=True)
        fused_wide = bench_decode(device, 200, 40, shape=(m, 28672, 4096), swiglu=True, variant=2)
        res["M=%d" % m]["fused_swiglu_us"] = fused["hbm"]["us"]
        res["M=%d" % m]["fused_swiglu_us_256x128_output_tiles"] = fused_wide["hbm"]["us"]
        torch.cuda.empty_cache()
    return res


def bench_nvfp4(device, steps, warmup):
    m, n, k = 4096, 4096, 14336
    g = torch.Generator().manual_seed(3)
    a, a_s, a_g = synth.quantize_nvfp4(cpu_randn((m, k), 3, device, generator=g))
    b, b_s, b_g = synth.quantize_nvfp4(cpu_randn((n, k), 3, device, std=0.02, generator=g))
    out = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    leg = GraphLeg(lambda: gemm_nvfp4_transposed_b(a, a_s, a_g, b, b_s, b_g, out=out))
    ceiling = bench_mfma_ceiling(device, (a, b), f16=True)   # also keeps the GPU loaded up to the timed steps
    ms, _ = leg.time(steps, warmup)
    return {"ms": ms, "tflops": 2.0 * m * n * k / (ms * 1e-3) / 1e12, "shape": (m, n, k), "f16_mfma_only": ceiling,
            "bytes": (m + n) * k // 2 + (m + n) * k // 16 + 2 * m * n + 8}


def bench_nvfp4_decode(device, rows=(16, 64, 128, 256)):
    """NVFP4 at decode batch sizes against the gate/up and down projection weights (rotated so that every call
    streams them from HBM): the weight-streaming kernel up to 64 rows, above that the tile kernel with K split
    over the compute units."""
    res = {}
    g = torch.Generator(device=device).manual_seed(3)
    for name, n, k, copies in (("gate_up 28672x4096", 28672, 4096, 8), ("down 4096x14336", 4096, 14336, 16)):
        ws = [synth.quantize_nvfp4(torch.randn((n, k), generator=g, device=device) * 0.02) for _ in range(copies)]
        res[name] = {}
        for m in rows:
            a, a_s, a_g = synth.quantize_nvfp4(torch.randn((m, k), generator=g, device=device))
            out = torch.empty((m, n), dtype=torch.bfloat16, device=device)
            us = _graph_us([lambda w=w: gemm_nvfp4_transposed_b(a, a_s, a_g, w[0], w[1], w[2], out=out) for w in ws], 10 * copies, 2 * copies)
            weight_bytes = n * k // 2 + n * k // 16
            res[name]["M=%d" % m] = {"us_per_launch": us, "weights_gbs": weight_bytes / (us * 1e-6) / 1e9}
        del ws
        torch.cuda.empty_cache()
    return res


def prepare_grouped(device):
    tokens, experts, top_k, n, k = 16384, 8, 2, 14336, 4096
    g = torch.Generator().manual_seed(4)
    x = cpu_randn((tokens, k), 4, device, generator=g)
    token_of_row, row_offsets = synth.moe_routing(tokens, experts, top_k, g, "cpu")
    token_of_row, row_offsets = token_of_row.to(device), row_offsets.to(device)
    a, a_s = synth.quantize_mxfp4(x[token_of_row])
    del x
    bs, bss = [], []
    for _ in range(experts):
        q, s = synth.quantize_mxfp4(cpu_randn((n, k), 4, device, std=0.02, generator=g))
        bs.append(q)
        bss.append(s)
    b, b_s = torch.stack(bs), torch.stack(bss)
    total_m = a.shape[0]
    out = torch.empty((total_m, n), dtype=torch.bfloat16, device=device)
    return {"leg": GraphLeg(lambda: grouped_gemm_mxfp4_transposed_b(a, a_s, b, b_s, row_offsets, out=out)),
            "tensors": (a, a_s, b, b_s, row_offsets, out), "shape": (total_m, n, k), "row_offsets": row_offsets.cpu().tolist(),
            "bytes": (total_m + experts * n) * k // 2 + (total_m + experts * n) * k // 32 + 2 * total_m * n + 4 * (experts + 1)}


def bench_grouped(device, steps, warmup, prepared=None):
    pre = prepared or prepare_grouped(device)
    total_m, n, k = pre["shape"]
    ms, _ = pre["leg"].time(steps, warmup)
    return {"ms": ms, "tflops": 2.0 * total_m * n * k / (ms * 1e-3) / 1e12, "shape": pre["shape"],
            "row_offsets": pre["row_offsets"], "bytes": pre["bytes"]}


def bench_mlp_block(device, steps, warmup):
    """A dense MLP block, 8192 tokens, 4096 -> 14336 -> 4096, bf16 in and out: activation quantiser, gate+up GEMM with
    SwiGLU and the quantiser of its result, down projection.  Three launches in one graph."""
    m, hidden, inter = 8192, 4096, 14336
    g = torch.Generator(device=device).manual_seed(7)
    x = torch.randn((m, hidden), generator=g, device=device, dtype=torch.bfloat16)
    w = torch.randn((2 * inter, hidden), generator=g, device=device, dtype=torch.float32) * 0.02
    w1, w1_s = synth.quantize_mxfp4(w)
    del w
    w = torch.randn((hidden, inter), generator=g, device=device, dtype=torch.float32) * 0.02
    w2, w2_s = synth.quantize_mxfp4(w)
    del w
    xa = torch.empty((m, hidden // 2), dtype=torch.uint8, device=device)
    xs = torch.empty((m, hidden // 32), dtype=torch.uint8, device=device)
    ha = torch.empty((m, inter // 2), dtype=torch.uint8, device=device)
    hs = torch.empty((m, inter // 32), dtype=torch.uint8, device=device)
    y = torch.empty((m, hidden), dtype=torch.bfloat16, device=device)

    def block():
        quantize_mxfp4(x, xa, xs)
        gemm_mxfp4_swiglu_quant_transposed_b(xa, xs, w1, w1_s, out=ha, out_scale=hs)
        gemm_mxfp4_transposed_b(ha, hs, w2, w2_s, out=y)

    block()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=torch.cuda.Stream()):
        block()
    torch.cuda.synchronize()
    ms, _ = _events_ms(graph.replay, max(10, steps // 2), 3)
    down_ms, _ = _events_ms(lambda: gemm_mxfp4_transposed_b(ha, hs, w2, w2_s, out=y), max(10, steps // 2), 3)
    flop = 2.0 * m * (2 * inter) * hidden + 2.0 * m * hidden * inter
    return {"shape": {"tokens": m, "hidden": hidden, "intermediate": inter}, "block_ms": ms,
            "block_tflops": flop / (ms * 1e-3) / 1e12, "down_ms": down_ms,
            "down_tflops": 2.0 * m * hidden * inter / (down_ms * 1e-3) / 1e12}


def bench_mlp_block_batched_decode(device, tokens=128, layers=6):
    """The same dense MLP block at a decode batch: `tokens` rows through `layers` blocks with weights of their own
    (88 MB each, more than the last-level cache holds in all), each block's bf16 output feeding the next: quantiser,
    gate+up GEMM with SwiGLU and quantiser (the narrow-tile kernel), down projection with K split
    over the compute units (two launches).  One graph; time per block."""
    m, hidden, inter = tokens, 4096, 14336
    g = torch.Generator(device=device).manual_seed(8)
    x0 = torch.randn((m, hidden), generator=g, device=device, dtype=torch.bfloat16)
    weights = []
    for _ in range(layers):
        w = torch.randn((2 * inter, hidden), generator=g, device=device, dtype=torch.float32) * 0.02
        w1 = synth.quantize_mxfp4(w)
        del w
        w = torch.randn((hidden, inter), generator=g, device=device, dtype=torch.float32) * 0.02
        w2 = synth.quantize_mxfp4(w)
        del w
        weights.append((w1, w2))
    xa = torch.empty((m, hidden // 2), dtype=torch.uint8, device=device)
    xs = torch.empty((m, hidden // 32), dtype=torch.uint8, device=device)
    ha = torch.empty((m, inter // 2), dtype=torch.uint8, device=device)
    hs = torch.empty((m, inter // 32), dtype=torch.uint8, device=device)
    ys = [torch.empty((m, hidden), dtype=torch.bfloat16, device=device) for _ in range(2)]

    def chain():
        x = x0
        for i, ((w1, w1_s), (w2, w2_s)) in enumerate(weights):
            quantize_mxfp4(x, xa, xs)
            gemm_mxfp4_swiglu_quant_transposed_b(xa, xs, w1, w1_s, out=ha, out_scale=hs)
            x = gemm_mxfp4_transposed_b(ha, hs, w2, w2_s, out=ys[i & 1])

    chain()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=torch.cuda.Stream()):
        chain()
    torch.cuda.synchronize()
    ms, _ = _events_ms(graph.replay, 40, 5)
    us = ms * 1e3 / layers
    weight_bytes = (2 * inter * hidden + hidden * inter) // 2 * 33 // 32
    return {"shape": {"tokens": m, "hidden": hidden, "intermediate": inter, "blocks": layers}, "block_us": us,
            "weights_gbs": weight_bytes / (us * 1e-6) / 1e9, "frac_hbm_peak": weight_bytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS,
            "block_tflops": (2.0 * m * (2 * inter) * hidden + 2.0 * m * hidden * inter) / (us * 1e-6) / 1e12}


def bench_moe_layer(device, steps, warmup, tokens=16384):
    """A whole MoE expert layer on the device, 16384 tokens, 8 experts top-2, hidden 4096, intermediate 14336:
    routing, activation quantiser, row gather, grouped gate+up GEMM with SwiGLU and the quantiser of its result,
    grouped down projection, weighted combine back into token order.  Six launches, captured in one graph; also
    each GEMM and the combine on their own."""
    experts, hidden, inter = 8, 4096, 14336
    g = torch.Generator(device=device).manual_seed(6)
    x = torch.randn((tokens, hidden), generator=g, device=device, dtype=torch.bfloat16)
    logits = torch.randn((tokens, experts), generator=g, device=device, dtype=torch.float32)

    def expert_weights(rows, k):
        qs, ss = [], []
        for _ in range(experts):
            w = torch.randn((rows, k), generator=g, device=device, dtype=torch.float32) * 0.02
            q, s_ = synth.quantize_mxfp4(w)
            qs.append(q)
            ss.append(s_)
            del w
        return torch.stack(qs), torch.stack(ss)

    w1, w1_s = expert_weights(2 * inter, hidden)   # gate rows, then up rows
    w2, w2_s = expert_weights(hidden, inter)
    rows = 2 * tokens
    tok = torch.empty(rows, dtype=torch.int32, device=device)
    off = torch.empty(experts + 1, dtype=torch.int32, device=device)
    wgt = torch.empty(rows, dtype=torch.float32, device=device)
    xa = torch.empty((tokens, hidden // 2), dtype=torch.uint8, device=device)
    xs = torch.empty((tokens, hidden // 32), dtype=torch.uint8, device=device)
    ga = torch.empty((rows, hidden // 2), dtype=torch.uint8, device=device)
    gs = torch.empty((rows, hidden // 32), dtype=torch.uint8, device=device)
    ha = torch.empty((rows, inter // 2), dtype=torch.uint8, device=device)
    hs = torch.empty((rows, inter // 32), dtype=torch.uint8, device=device)
    y = torch.empty((rows, hidden), dtype=torch.bfloat16, device=device)
    inv = torch.empty((tokens, 2), dtype=torch.int32, device=device)
    out = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=device)

    def combine():
        moe_combine_top2(y, inv, wgt, out=out, renormalize=True)

    def up():
        grouped_gemm_mxfp4_swiglu_quant_transposed_b(ga, gs, w1, w1_s, off, out=ha, out_scale=hs)

    def down():
        grouped_gemm_mxfp4_transposed_b(ha, hs, w2, w2_s, off, out=y)

    def layer():
        moe_route_top2(logits, token_of_row=tok, row_offsets=off, row_weight=wgt, rows_of_token=inv)
        quantize_mxfp4(x, xa, xs)
        gather_rows_mxfp4(xa, xs, tok, out=ga, out_scale=gs)
        up()
        down()
        combine()

    layer()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=torch.cuda.Stream()):
        layer()
    torch.cuda.synchronize()
    n = max(10, steps // 5)
    layer_ms, _ = _events_ms(graph.replay, n, 3)
    up_ms, _ = _events_ms(up, n, 3)
    down_ms, _ = _events_ms(down, n, 3)
    combine_us = _graph_us([combine] * 4, n, 3)
    flop = 2.0 * rows * (2 * inter) * hidden + 2.0 * rows * hidden * inter
    return {"shape": {"tokens": tokens, "experts": experts, "top_k": 2, "hidden": hidden, "intermediate": inter},
            "layer_ms": layer_ms, "layer_tflops": flop / (layer_ms * 1e-3) / 1e12,
            "gate_up_swiglu_quant_ms": up_ms, "gate_up_tflops": 2.0 * rows * (2 * inter) * hidden / (up_ms * 1e-3) / 1e12,
            "down_ms": down_ms, "down_tflops": 2.0 * rows * hidden * inter / (down_ms * 1e-3) / 1e12,
            "combine_us": combine_us, "combine_gbs": 3.0 * tokens * hidden * 2 / (combine_us * 1e-6) / 1e9}


def bench_quantize(device, steps, warmup):
    """Device-side MXFP4 quantiser on the prefill activations (8192 x 4096), fp32 and bf16 input.
    HBM-bound: bytes = input + packed codes + scales."""
    m, k = 8192, 4096
    g = torch.Generator(device=device).manual_seed(0)
    x = synth.activations_with_outliers(m, k, g, device)
    packed = torch.empty((m, k // 2), dtype=torch.uint8, device=device)
    scales = torch.empty((m, k // 32), dtype=torch.uint8, device=device)
    res = {"shape": (m, k), "input_buffers_rotated": 4}
    for name, t in (("f32", x), ("bf16", x.to(torch.bfloat16))):
        # four copies of the input (> 256 MB for fp32) so that launches do not re-read the last-level cache
        ts = [t] + [t.clone() for _ in range(3)]
        us = _graph_us([lambda src=src: quantize_mxfp4(src, packed=packed, scales=scales) for src in ts], steps, warmup)
        ms = us * 1e-3
        del ts
        byts = t.numel() * t.element_size() + packed.numel() + scales.numel()
        res[name] = {"us": ms * 1e3, "gbs": byts / (ms * 1e-3) / 1e9, "frac_hbm_peak": byts / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
    # the NVFP4 quantiser on the same activations, for a calibrated per-tensor scale
    gscale = (x.abs().amax() / (448 * 6)).reshape(1)
    nv_scales = torch.empty((m, k // 16), dtype=torch.uint8, device=device)
    for name, t in (("nvfp4_f32", x), ("nvfp4_bf16", x.to(torch.bfloat16))):
        ts = [t] + [t.clone() for _ in range(3)]
        us = _graph_us([lambda src=src: quantize_nvfp4(src, gscale, packed=packed, scales=nv_scales) for src in ts], steps, warmup)
        del ts
        byts = t.numel() * t.element_size() + packed.numel() + nv_scales.numel()
        res[name] = {"us": us, "gbs": byts / (us * 1e-6) / 1e9, "frac_hbm_peak": byts / (us * 1e-6) / 1e9 / HBM_PEAK_GBS}
    return res


def bench_moe_front(device, steps, warmup):
    """Routing (16384 tokens, 8 experts, one workgroup: latency-bound) and the row gather that builds
    the grouped GEMM's A operand (32768 rows of K = 4096: HBM-bound, bytes = read + written rows)."""
    tokens, experts, k = 16384, 8, 4096
    g = torch.Generator(device=device).manual_seed(4)
    logits = torch.randn((tokens, experts), generator=g, device=device, dtype=torch.float32)
    tok, off, w = moe_route_top2(logits)
    ms_route = _graph_us([lambda: moe_route_top2(logits, tok, off, w)] * 4, steps, warmup) * 1e-3
    srcs = [synth.quantize_mxfp4(torch.randn((tokens, k), generator=g, device=device)) for _ in range(4)]
    ga = torch.empty((2 * tokens, k // 2), dtype=torch.uint8, device=device)
    gs = torch.empty((2 * tokens, k // 32), dtype=torch.uint8, device=device)
    ms_gather = _graph_us([lambda a=a, a_s=a_s: gather_rows_mxfp4(a, a_s, tok, ga, gs) for a, a_s in srcs],
                          steps, warmup) * 1e-3
    row = k // 2 + k // 32
    byts = tokens * row + 2 * tokens * row + 2 * tokens * 4   # every source row once, every routed row written
    return {"shape": (tokens, experts, k), "route_us": ms_route * 1e3, "gather_us": ms_gather * 1e3,
            "gather_gbs": byts / (ms_gather * 1e-3) / 1e9,
            "gather_frac_hbm_peak": byts / (ms_gather * 1e-3) / 1e9 / HBM_PEAK_GBS}


def cpu_baseline(prefill, repeats=15):
    """The reference's validation recipe (dequantise -> fp32 matmul -> bf16,
    test/examples/gemm/amdgpu/test_amdgpu_gemm.py:27) on the host cores for the whole problem: operands are
    dequantised once (numpy oracle) and the fp32 matmul is timed `repeats` times; the throughput is that of
    one dequantisation plus one matmul.  The GPU result is checked against it on the way."""
    from oracle import fp4_oracle as orc

    a, a_s, b, b_s, out = prefill["tensors"]
    m, n, k = prefill["shape"]
    cores = torch.get_num_threads()
    a_np, as_np = a.cpu().numpy(), a_s.cpu().numpy()
    b_np, bs_np = b.cpu().numpy(), b_s.cpu().numpy()
    t0 = time.perf_counter()
    adq = torch.from_numpy(orc.dequantize_mxfp4(a_np, as_np))
    bdq = torch.from_numpy(orc.dequantize_mxfp4(b_np, bs_np))
    t1 = time.perf_counter()
    for _ in range(repeats):
        c = (adq @ bdq.T).to(torch.bfloat16)
    t2 = time.perf_counter()
    dequant_s, matmul_s = t1 - t0, (t2 - t1) / repeats
    flops = 2.0 * m * n * k
    ref = c.float()
    del c
    got = out.float().cpu()
    row_max = ref.abs().amax(dim=1).clamp_min(1e-30)
    rel = ((got - ref).abs().amax(dim=1) / row_max).max().item()
    return {
        "value": flops / (dequant_s + matmul_s) / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"the whole problem ({m}x{n}x{k}): operands dequantised once, fp32 matmul timed {repeats} times",
        "dequant_s": dequant_s,
        "matmul_s": matmul_s,
        "cpu_seconds_total": t2 - t0,
        "gpu_vs_cpu_max_row_rel": rel,
    }


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--all", action="store_true", help="also time the legs beyond the four GPU configurations: fused SwiGLU, "
                    "quantisers, MLP block, MoE layer, decode batches")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-live-counters", action="store_true",
                    help="do not start the child rocprofv3 run that measures the prefill GEMM's MFMA-busy fraction and clock")
    ap.add_argument("--rotated-only", action="store_true",
                    help="decode leg: time the launches over rotated weight buffers only (no cache-resident launches), "
                         "so that a kernel trace of the run shows HBM-streamed launches alone")
    ap.add_argument("--m", type=int, default=None, help="with --n and --k: time one MXFP4 GEMM of this shape "
                    "(the reference benchmark's command line)")
    ap.add_argument("--n", type=int, default=None)
    ap.add_argument("--k", type=int, default=None)
    ap.add_argument("--validate", action="store_true", help="with --m --n --k: check the result on the CPU")
    ap.add_argument("--grouped", type=int, default=0, help="with --m --n --k: the grouped GEMM of this many experts with --m rows "
                    "and [n, k] weights each")
    ap.add_argument("--nvfp4", action="store_true", help="with --m --n --k: the NVFP4 GEMM instead of the MXFP4 one (no --validate)")
    ap.add_argument("--repeat", type=int, default=None, help="with --m --n --k: the reference's pair of loop counts "
                    "(bench_amdgpu_gemm.py:78-80): repeat x iters graph replays between the two events; replaces --steps")
    ap.add_argument("--iters", type=int, default=None, help="graph replays per timing repeat (with --repeat)")
    ap.add_argument("--rotate", type=int, default=1, help="with --m --n --k: launches per graph, each on a weight buffer of its "
                    "own (weights from HBM instead of the last-level cache)")
    ap.add_argument("--variant", type=int, default=0, help="with --m --n --k: force a kernel (ave_fp4_variant: 1 generic, 2 tile, "
                    "3 decode, 4 narrow, 6 tile with look-ahead touches)")
    ap.add_argument("--rows", type=int, default=None, help="with --only down_batched, gate_up_batched, mlp_block_decode, nvfp4_decode: a single batch size; with --only moe_layer: the number of tokens")
    ap.add_argument("--only", choices=["stream_read", "prefill", "decode", "decode_down", "copy", "nvfp4", "grouped", "quantize", "moe_front", "mfma_ceiling", "prefill_swiglu", "moe_layer", "mlp_block", "down_batched", "gate_up_batched", "mlp_block_decode", "nvfp4_decode", "blocked_scales"], default=None,
                    help="time one kernel only (profiling); 'copy' runs a plain 256 MiB device copy, the known-size "
                         "kernel the FETCH_SIZE / WRITE_SIZE counters are calibrated against")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).")
    if not synth.has_rocm():
        sys.exit("bench.py needs a ROCm GPU.")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    line = {"metric": METRIC, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "mxfp4 (e2m1 x e8m0), fp32 accumulate",
            "data": "synthetic"}
    prefill = None
    if args.m is not None or args.n is not None or args.k is not None:
        if None in (args.m, args.n, args.k):
            sys.exit("--m, --n and --k go together.")
        steps = args.steps
        if args.repeat is not None or args.iters is not None:
            steps = (args.repeat or 100) * (args.iters or 100)   # the reference's defaults (:78-79)
        if args.grouped:
            res = bench_shape_grouped(device, args.grouped, args.m, args.n, args.k, steps, args.warmup, args.variant)
        elif args.nvfp4:
            res = bench_shape_nvfp4(device, args.m, args.n, args.k, steps, args.warmup, max(1, args.rotate), args.variant)
        else:
            res = bench_shape(device, args.m, args.n, args.k, steps, args.warmup, args.validate, max(1, args.rotate), args.variant)
        if steps != args.steps:
            res.update({"repeat": args.repeat or 100, "iters": args.iters or 100})
        print(json.dumps(res))
        return
    if args.only == "stream_read":
        print(json.dumps({"metric": "plain streaming read of 1 GiB from HBM", "unit": "GB/s",
                          **bench_stream_read(device, mx_bytes(16, 28672, 4096), result_bytes=16 * 28672 * 2)}))
        return
    if args.only == "copy":
        src = torch.full((256 << 20,), 7, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        ms, _ = _events_ms(lambda: dst.copy_(src), args.steps, args.warmup)
        print(json.dumps({"metric": "device copy", "bytes_read": src.numel(), "bytes_written": src.numel(),
                          "ms_per_step": ms, "value": 2 * src.numel() / (ms * 1e-3) / 1e9, "unit": "GB/s"}))
        return
    if args.only == "nvfp4":
        nv = bench_nvfp4(device, args.steps, args.warmup)
        print(json.dumps({"metric": "NVFP4 GEMM", "shape": nv["shape"], "ms_per_step": nv["ms"], "value": nv["tflops"],
                          "unit": "TFLOP/s", "frac_f16_peak": nv["tflops"] / F16_PEAK_TFLOPS}))
        return
    if args.only == "decode_down":
        dd = bench_decode(device, 240, 48, copies=24, shape=(16, 4096, 14336))
        print(json.dumps({"metric": "MXFP4 decode GEMM, down projection", "shape": dd["shape"],
                          "us_per_launch": dd["hbm"]["us"], "value": dd["hbm"]["gbs"], "unit": "GB/s",
                          "cache_resident_us": dd["cached"]["us"]}))
        return
    if args.only == "down_batched":
        print(json.dumps({"metric": "MXFP4 down projection at batch 128..1024, N=4096, K=14336", **bench_down_batched(device, (args.rows,) if args.rows else (128, 256, 512, 1024))}))
        return
    if args.only == "nvfp4_decode":
        print(json.dumps({"metric": "NVFP4 GEMM at decode batch sizes", **bench_nvfp4_decode(device, (args.rows,) if args.rows else (16, 64, 128, 256))}))
        return
    if args.only == "mlp_block_decode":
        print(json.dumps({"metric": "dense MLP block at decode batch, one graph over six blocks",
                          **bench_mlp_block_batched_decode(device, args.rows or 128)}))
        return
    if args.only == "gate_up_batched":
        print(json.dumps({"metric": "MXFP4 gate/up projection at batch 128 and 256, N=28672, K=4096",
                          **bench_gate_up_batched(device, (args.rows,) if args.rows else (128, 256))}))
        return
    if args.only == "moe_front":
        mf = bench_moe_front(device, args.steps, args.warmup)
        print(json.dumps({"metric": "top-2 routing and row gather", **mf}))
        return
    if args.only == "quantize":
        q = bench_quantize(device, args.steps, args.warmup)
        print(json.dumps({"metric": "device MXFP4 quantiser, 8192x4096", **q}))
        return
    if args.only == "grouped":
        gr = bench_grouped(device, args.steps, args.warmup)
        print(json.dumps({"metric": "grouped MXFP4 GEMM", "shape": gr["shape"], "ms_per_step": gr["ms"],
                          "value": gr["tflops"], "unit": "TFLOP/s", "frac_fp4_peak": gr["tflops"] / FP4_PEAK_TFLOPS}))
        return
    if args.only == "mlp_block":
        mb = bench_mlp_block(device, args.steps, args.warmup)
        print(json.dumps({"metric": "dense MLP block, three launches in one graph", "unit": "TFLOP/s",
                          "value": mb["block_tflops"], "ms_per_step": mb["block_ms"], **mb}))
        return
    if args.only == "moe_layer":
        ml = bench_moe_layer(device, args.steps, args.warmup, args.rows or 16384)
        print(json.dumps({"metric": "MoE expert layer, six launches in one graph", "unit": "TFLOP/s",
                          "value": ml["layer_tflops"], "ms_per_step": ml["layer_ms"], **ml}))
        return
    if args.only == "prefill_swiglu":
        ps = bench_prefill_swiglu(device, args.steps, args.warmup)
        print(json.dumps({"metric": "MXFP4 gate+up GEMM with fused SwiGLU", "unit": "TFLOP/s", "value": ps["fused_tflops"],
                          "ms_per_step": ps["fused_ms"], **ps}))
        return
    if args.only == "blocked_scales":
        print(json.dumps({"metric": "MXFP4 GEMM on blocked (128 x 4) scale tensors against row-major ones",
                          **bench_blocked_scales(device, make_prefill(device), args.steps, args.warmup)}))
        return
    if args.only == "mfma_ceiling":
        a, _, b, _ = make_prefill(device)
        print(json.dumps({"metric": "scaled FP4 MFMA loop, nothing else running", "unit": "TFLOP/s",
                          **bench_mfma_ceiling(device, (a, b), settle_launches=45)}))
        return
    if args.only in (None, "prefill"):
        # The matrix-core rate this GPU sustains on these very operands when it does nothing else comes first: it
        # also brings the GPU out of its idle clocks before the timed launches, as the reference's warm-up is
        # meant to (bench_amdgpu_gemm.py:31-34: "stabilize clocks").
        # Everything that takes host time (operands, graph capture) is prepared first, so that the GPU is not left
        # idle between the legs that follow.
        operands = make_prefill(device)
        prepared = prepare_prefill(device, operands)
        prepared_grouped = prepare_grouped(device) if args.only is None else None
        prepared_cold = prepare_prefill_cold(device, operands) if args.only is None else None
        prepared_tail = prepare_k_tail(device) if args.only is None else None
        ceiling = bench_mfma_ceiling(device, (operands[0], operands[2]), settle_launches=0 if args.only else 45)
        if args.only is None:
            # The grouped (MoE) configuration runs on the same kernel as the headline GEMM; measured ahead of it, its
            # launches keep the GPU under this kernel's load until the timed steps of the headline begin.
            gr = bench_grouped(device, args.steps, args.warmup, prepared_grouped)
            del prepared_grouped
            m, n, k = gr["shape"]
            line["grouped"] = {"workload": "MoE grouped MXFP4 GEMM, 8 experts top-2 (BASELINE configs[4])", "total_M": m,
                               "N": n, "K": k, "row_offsets": gr["row_offsets"], "ms_per_step": gr["ms"],
                               "value": gr["tflops"], "unit": "TFLOP/s",
                               "roofline": {"bound": "mfma", "achieved": gr["tflops"], "peak": FP4_PEAK_TFLOPS, "unit": "TFLOP/s",
                                            "frac": gr["tflops"] / FP4_PEAK_TFLOPS, "traffic": measured_traffic("mx_tile_kernel_grouped"),
                                            "kernel": "mx_tile_kernel (grouped)", "flops_per_launch": 2.0 * m * n * k,
                                            "algorithmic_bytes_per_launch": gr["bytes"],
                                            **measured_counters("mx_tile_kernel_grouped")}}
            del gr
        prefill = bench_prefill(device, args.steps, args.warmup, settle_steps=0 if args.only else 150, prepared=prepared)
        m, n, k = prefill["shape"]
        line.update({
            "value": prefill["tflops"],
            "ms_per_step": prefill["ms"],
            "timing": "one launch captured in a graph, `steps` replays between two events (reference protocol)",
            "config": {"workload": "MXFP4 prefill MLP up-projection GEMM (BASELINE configs[1])", "M": m, "N": n, "K": k,
                       "A": "N(0,1), 1% of K channels x20", "B": "N(0,0.02)", "block": 32, "out": "bf16",
                       "seeds": "CPU generators, fixed seeds"},
            "roofline": {"bound": "mfma", "achieved": prefill["tflops"], "peak": FP4_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": prefill["tflops"] / FP4_PEAK_TFLOPS, "traffic": measured_traffic("mx_tile_kernel"),
                         "kernel": "mx_tile_kernel", "flops_per_launch": 2.0 * m * n * k,
                         "algorithmic_bytes_per_launch": mx_bytes(m, n, k), **measured_counters("mx_tile_kernel")},
        })
        if prepared_cold is not None:
            # right behind the headline's replays, at the same clock
            line["cold_weights"] = bench_prefill_cold(prepared_cold, args.steps, args.warmup)
            line["cold_weights"]["frac_of_cache_resident_rate"] = line["cold_weights"]["value"] / prefill["tflops"]
            line["k_tail"] = bench_k_tail(prepared_tail, args.steps, args.warmup)
            line["k_tail"]["time_vs_k4096"] = line["k_tail"]["ms_per_step"] / prefill["ms"]
            del prepared_cold, prepared_tail
        if "settled" in prefill:
            line["settled_clock"] = {"workload": "the same graph replayed on, timed after the GPU's power management has "
                                                 "settled on this load", **prefill["settled"],
                                     "frac_fp4_peak": prefill["settled"]["tflops"] / FP4_PEAK_TFLOPS}
        line["roofline"]["mfma_only_measured"] = {"unit": "TFLOP/s", **ceiling,
                                                  "frac_of_gemm_operands_rate": prefill["tflops"] / ceiling["gemm_operands"]}
        if "gemm_operands_settled" in ceiling:
            line["roofline"]["mfma_only_measured"]["frac_of_settled_rate"] = prefill["tflops"] / ceiling["gemm_operands_settled"]
    if args.only in (None, "decode"):
        dec = bench_decode(device, max(args.steps, 10) * 4, args.warmup * 4, rotated_only=args.rotated_only)
        m, n, k = dec["shape"]
        line["decode"] = {
            "workload": "MXFP4 decode GEMM (BASELINE configs[2])", "M": m, "N": n, "K": k,
            "us_per_launch": dec["hbm"]["us"], "value": dec["hbm"]["gbs"], "unit": "GB/s",
            "weight_buffers_rotated": dec["copies"],
            "roofline": {"bound": "hbm", "achieved": dec["hbm"]["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": dec["hbm"]["gbs"] / HBM_PEAK_GBS, "traffic": measured_traffic("mx_decode_ring_kernel"),
                         "kernel": "mx_decode_ring_kernel",
                         "algorithmic_bytes_per_launch": mx_bytes(m, n, k),
                         **({"counters_from": COUNTERS_FILE} if measured_traffic("mx_decode_ring_kernel") else {})},
        }
        if "cached" in dec:
            line["decode"]["cache_resident"] = {"us_per_launch": dec["cached"]["us"], "gbs": dec["cached"]["gbs"]}
        if prefill is None:
            line.update({"value": dec["hbm"]["gbs"], "unit": "GB/s", "ms_per_step": dec["hbm"]["us"] * 1e-3,
                         "config": {"workload": line["decode"]["workload"]}})
        else:
            line["decode"]["stream_read_floor"] = bench_stream_read(device, mx_bytes(m, n, k), result_bytes=m * n * 2)
            floor_us = line["decode"]["stream_read_floor"]["same_bytes_as_the_gemm"]["us_per_launch_with_result"]
            line["decode"]["frac_of_stream_read_floor"] = floor_us / dec["hbm"]["us"]
    if args.only is None:
        # the other two GPU configurations, each with its own roofline object
        torch.cuda.empty_cache()
        nv = bench_nvfp4(device, args.steps, args.warmup)
        m, n, k = nv["shape"]
        line["nvfp4"] = {"workload": "NVFP4 down-projection GEMM (BASELINE configs[3])", "M": m, "N": n, "K": k,
                         "ms_per_step": nv["ms"], "value": nv["tflops"], "unit": "TFLOP/s",
                         "roofline": {"bound": "mfma", "achieved": nv["tflops"], "peak": FP4_PEAK_TFLOPS, "unit": "TFLOP/s",
                                      "frac": nv["tflops"] / FP4_PEAK_TFLOPS,
                                      "peak_f16": F16_PEAK_TFLOPS, "frac_f16": nv["tflops"] / F16_PEAK_TFLOPS,
                                      "note": "operands are dequantised to f16 in registers and multiplied at the f16 MFMA rate",
                                      "traffic": measured_traffic("nv_tile4_kernel"), "kernel": "nv_tile4_kernel",
                                      "flops_per_launch": 2.0 * m * n * k, "algorithmic_bytes_per_launch": nv["bytes"],
                                      "f16_mfma_only_measured": {"unit": "TFLOP/s", **nv["f16_mfma_only"],
                                                                 "frac_of_gemm_operands_rate": nv["tflops"] / nv["f16_mfma_only"]["gemm_operands"]},
                                      **measured_counters("nv_tile4_kernel")}}
        del nv
    if args.all:
        torch.cuda.empty_cache()
        q = bench_quantize(device, max(20, args.steps), args.warmup)
        line["quantize_mxfp4"] = {"workload": "device MXFP4 quantiser, 8192x4096 activations", **q}
        torch.cuda.empty_cache()
        ps = bench_prefill_swiglu(device, max(20, args.steps // 2), args.warmup)
        line["prefill_swiglu"] = {"workload": "MXFP4 gate+up GEMM with fused SwiGLU, 8192 x (2 x 14336) x 4096", **ps,
                                  "frac_fp4_peak": ps["fused_tflops"] / FP4_PEAK_TFLOPS}
        torch.cuda.empty_cache()
        line["mlp_block"] = {"workload": "dense MLP block in one graph: quantiser, gate+up+SwiGLU+quantiser, down projection",
                             **bench_mlp_block(device, args.steps, args.warmup)}
        torch.cuda.empty_cache()
        line["moe_layer"] = {"workload": "MoE expert layer in one graph: routing, quantiser, gather, grouped gate+up+SwiGLU+"
                                         "quantiser, grouped down projection, combine", **bench_moe_layer(device, args.steps, args.warmup)}
        torch.cuda.empty_cache()
        line["blocked_scales"] = {"workload": "the headline and the decode GEMM on blocked (128 x 4) scale tensors, read directly",
                                  **bench_blocked_scales(device, make_prefill(device), args.steps, args.warmup)}
        torch.cuda.empty_cache()
        ds = bench_decode(device, 400, 80, swiglu=True)
        line["decode_swiglu"] = {"workload": "MXFP4 gate+up decode GEMM with fused SwiGLU, M=16, 2x14336 weight rows, K=4096",
                                 "us_per_launch": ds["hbm"]["us"], "hbm_gbs": ds["hbm"]["gbs"],
                                 "frac_hbm_peak": ds["hbm"]["gbs"] / HBM_PEAK_GBS}
        torch.cuda.empty_cache()
        line["decode_batched"] = {"workload": "MXFP4 decode GEMM at larger batch, N=28672, K=4096 (weights rotated over 10 buffers)"}
        for m in (32, 64):
            db = bench_decode(device, 400, 80, shape=(m, 28672, 4096))
            line["decode_batched"]["M=%d" % m] = {"us_per_launch": db["hbm"]["us"], "hbm_gbs": db["hbm"]["gbs"],
                                                   "frac_hbm_peak": db["hbm"]["gbs"] / HBM_PEAK_GBS}
        torch.cuda.empty_cache()
        mf = bench_moe_front(device, max(20, args.steps), args.warmup)
        line["moe_front"] = {"workload": "top-2 routing and row gather in front of the grouped GEMM", **mf}
        torch.cuda.empty_cache()
        line["nvfp4_decode"] = {"workload": "NVFP4 GEMM at decode batch sizes, weights rotated", **bench_nvfp4_decode(device)}
        torch.cuda.empty_cache()
        line["mlp_block_decode"] = {"workload": "dense MLP block at decode batch 128: quantiser, gate+up+SwiGLU+quantiser, down projection "
                                                "with K split; six blocks with weights of their own in one graph",
                                    **bench_mlp_block_batched_decode(device)}
        torch.cuda.empty_cache()
        line["gate_up_batched"] = {"workload": "MXFP4 gate/up projection at batch 128 and 256, N=28672, K=4096: the narrow-tile kernel "
                                               "(128x128 tiles up to 128 rows, 256x128 above) against 256x256 tiles", **bench_gate_up_batched(device)}
        torch.cuda.empty_cache()
        line["down_batched"] = {"workload": "MXFP4 down projection at batch 128..1024, N=4096, K=14336: K split over idle "
                                            "compute units through a workspace, against one workgroup per tile",
                                **bench_down_batched(device)}
        torch.cuda.empty_cache()
        dd = bench_decode(device, 240, 48, copies=24, shape=(16, 4096, 14336))
        line["decode_down"] = {"workload": "MXFP4 decode GEMM, down projection (K = 14336, four K panels)",
                               "shape": dd["shape"], "us_per_launch": dd["hbm"]["us"], "hbm_gbs": dd["hbm"]["gbs"],
                               "frac_hbm_peak": dd["hbm"]["gbs"] / HBM_PEAK_GBS,
                               "cache_resident_gbs": dd["cached"]["gbs"]}
    if prefill is not None and args.only is None and not args.no_live_counters:
        # every leg's counters in this run, on this box (child processes under rocprofv3, two per leg; the figures from
        # the file on disk are kept beside them)
        apply_live_counters(line["roofline"], live_leg_counters(device, "prefill", "mx_tile_kernel"))
        apply_live_counters(line["grouped"]["roofline"], live_leg_counters(device, "grouped", "mx_tile_kernel"))
        apply_live_counters(line["decode"]["roofline"],
                            live_leg_counters(device, "decode", "mx_decode_ring_kernel", mfma=False, extra_args=("--rotated-only",)))
        apply_live_counters(line["nvfp4"]["roofline"], live_leg_counters(device, "nvfp4", "nv_tile4_kernel"))
    if prefill is not None and not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(prefill)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
