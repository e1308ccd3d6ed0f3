#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

Default workload (`--workload layer_m1`): the linears of one Qwen3.8-27B-shaped
decoder layer at M=1 — q 5120->6144, k and v 5120->1024, o 6144->5120, gate and
up 5120->17408, down 17408->5120 — in affine-Q4 group-64 with bf16 scale/bias,
fp16 activations and fp16 outputs, on seeded synthetic weights (N(0,0.02)
before quantization) and activations (N(0,1)).  One step is one pass over the
seven linears of one weight copy (four launches: q|k|v and gate|up share their
activations and go out as one launch each, then o and down); successive steps
rotate over `--copies` distinct prepared copies (>= 1.5 GB in total) so that the
256 MB memory-side cache cannot serve the weights and the figure is an HBM figure.

Prints ONE JSON line.  `value` is algorithmic bytes (N*K/2 + N*(K/64)*4 +
M*K*2 + M*N*2 per linear) per second of wall time over the timed steps, with
all inputs resident in HBM before the clock starts.  `roofline` prices the
dominant kernel (the weight-streaming Q4 kernel) against HBM: algorithmic bytes
per launch over the kernel's own average duration (HIP events bound to each
dispatch, measured in a second pass of the same steps).  Before anything is
timed the GPU runs the same steps untimed until at least `--preheat-ms` of GPU
time have passed (clocks and power state settle; `config.preheat_ms` says how
long it ran): a 20-step run then reads like a 400-step run.  `cpu_baseline` is the
CPU oracle (a C restatement of the reference's scalar loop, row-parallel with
OpenMP as the reference parallelises its GEMV) timed on this host on the same
layer, with the CPU model, the threads used and the host's read bandwidth.

The default line also carries `secondary`: the other configurations of the
headline metric, each measured briefly in the same process on the same weights —
the speculative-verify batches (M = 2, 4, 8: HBM roofline), the prefill GEMMs of
the MLP at M = 512 (gate, up, down: fp16 matrix-instruction roofline) and the
W8A8 encoder projections (M=64, K=1024, N=4096: int8 roofline, accumulators
compared bit for bit with the CPU oracle).  `--no-secondary` leaves them out.

Other workloads (never the default; each prints its own JSON line of the same
shape): `--workload prefill --rows 512`, `--workload w8a8`, `--workload lm_head`,
`--workload config1`; `--rows 2..8` turns the default workload into the
small-M verify case.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT / "cpu-llms-in-c_amd"))
sys.path.insert(0, str(ROOT / "oracle"))

HBM_PEAK_GBPS = 8000.0  # MI355X datasheet: 8 TB/s HBM3E
# HBM bytes moved per algorithmic byte by the streaming kernel on the default workload: FETCH_SIZE and
# WRITE_SIZE of rocprofv3 --pmc, scaled by a plain read/fill of known size in the same runs
# (profiles/q4_stream_kernel_layer_m1.md, the section on the current library: 193,100,800 HBM bytes a
# step against 191,897,600 algorithmic); a counter reading, not something this script can measure
MEASURED_TRAFFIC_RATIO_LAYER_M1 = 1.006
F16_MFMA_PEAK_TFLOPS = 2500.0  # dense fp16 matrix instructions
I8_MFMA_PEAK_TOPS = 5000.0  # dense int8 matrix instructions

LAYER = [  # name, N (output rows), K (input columns)
    ("q_proj", 6144, 5120),
    ("k_proj", 1024, 5120),
    ("v_proj", 1024, 5120),
    ("o_proj", 5120, 6144),
    ("gate_proj", 17408, 5120),
    ("up_proj", 17408, 5120),
    ("down_proj", 5120, 17408),
]
CONFIG1 = [("linear_0p8b", 3584, 1024)]
LM_HEAD = [("lm_head", 248320, 5120)]  # the largest linear of the model: 698 MB, once per token
PREFILL = [("gate_proj", 17408, 5120), ("up_proj", 17408, 5120), ("down_proj", 5120, 17408)]
W8A8 = {"M": 64, "K": 1024, "N": 4096, "projections": 3}


def q4_bytes(N, K, M, y_bytes=2):
    return N * K // 2 + N * (K // 64) * 4 + M * K * 2 + M * N * y_bytes


# ---- host context ------------------------------------------------------------------------------

def host_threads():
    """Threads for the CPU baseline: every CPU this process may run on, but no more than the job's
    share when the launcher has set one (OMP_NUM_THREADS)."""
    try:
        allowed = len(os.sched_getaffinity(0))
    except AttributeError:
        allowed = os.cpu_count() or 1
    cap = os.environ.get("OMP_NUM_THREADS", "")
    threads = min(allowed, int(cap)) if cap.isdigit() and int(cap) > 0 else allowed
    return max(threads, 1), allowed


def cpu_model():
    try:
        with open("/proc/cpuinfo") as stream:
            for line in stream:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def host_fields(oracle, threads, allowed):
    """CPU model, thread counts and the host's read bandwidth at 1 and `threads` threads (the
    reference's target-probe measurement, tools/target_probe.c)."""
    return {
        "cpu_model": cpu_model(),
        "cores": threads,
        "host_cpus_online": os.cpu_count(),
        "host_cpus_allowed": allowed,
        "omp_num_threads_env": os.environ.get("OMP_NUM_THREADS"),
        # a 2 GiB buffer: far beyond the last-level caches of any host
        "host_read_gib_per_s": {"threads_1": round(oracle.probe_read_gib_per_s(2 << 30, 1, 0.5), 2),
                                "threads_%d" % threads: round(oracle.probe_read_gib_per_s(2 << 30, threads, 0.5), 2)},
        "host_read_what": "sum over the threads of the bytes each reads per second from a 2 GiB buffer of 64-bit "
                          "words (four accumulators per thread, 0.5 s); every pass a thread moves on to the share "
                          "its neighbour read last, so over the passes each thread walks the whole buffer and no "
                          "cache holds its working set: a DRAM figure",
    }


# ---- timing helpers ----------------------------------------------------------------------------

def preheat(ctx, run_steps, minimum_ms, batch):
    """Runs steps untimed until `minimum_ms` of GPU time have passed; returns the GPU ms it took."""
    total = 0.0
    while total < minimum_ms:
        ctx.timer_begin()
        run_steps(batch)
        total += ctx.timer_end()
    return total


def time_steps(ctx, run_steps, steps, warmup, preheat_ms=0.0, preheat_batch=50):
    """Wall and event time of `steps` steps after `warmup`, then the same steps again with an
    event pair around every dispatch: dict(wall s, gpu ms, kernel ms, launches, per-launch us)."""
    heated = preheat(ctx, run_steps, preheat_ms, preheat_batch) if preheat_ms > 0 else 0.0
    run_steps(warmup)
    ctx.sync()
    t0 = time.perf_counter()
    ctx.timer_begin()
    run_steps(steps)
    gpu_ms = ctx.timer_end()  # waits for the stream
    ctx.sync()
    wall = time.perf_counter() - t0
    # per-dispatch pass: the warm-up steps run in the same mode first (it launches through another
    # runtime call and creates its events on first use), then the counted steps follow at once
    ctx.profile_begin()
    run_steps(max(warmup, 2))
    ctx.profile_end()
    ctx.profile_begin()
    run_steps(steps)
    kernel_ms, launches = ctx.profile_end()
    return {"wall": wall, "gpu_ms": gpu_ms, "kernel_ms": kernel_ms, "launches": int(launches),
            "per_launch_us": ctx.profile_durations(), "preheat_ms": heated}


def common_fields(args, wall):
    return {
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3 / args.steps, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
    }


def device_fields(info):
    name = info.name.decode(errors="replace").strip()
    arch = info.arch.decode(errors="replace")
    return {"device": name or "(the runtime reports no product name; arch %s)" % arch,
            "arch": arch,
            "max_clock_mhz": info.clock_mhz, "memory_clock_mhz": info.memory_clock_mhz,
            "memory_bus_bits": info.memory_bus_bits, "compute_units": info.compute_units}


# ---- Q4 layer workloads ------------------------------------------------------------------------

class LayerWorkload:
    """`copies` prepared device copies of every matrix of `shapes` plus activations/outputs."""

    def __init__(self, engine, ctx, shapes, copies, meta_kind, max_rows, verbose=False):
        self.engine, self.ctx, self.shapes, self.copies, self.meta_kind = engine, ctx, shapes, copies, meta_kind
        self.host, self.weights, self.x_ptr, self.y_ptr = {}, [[] for _ in range(copies)], {}, {}
        for index, (name, N, K) in enumerate(shapes):
            t0 = time.perf_counter()
            self.host[name] = engine.synth_q4_affine(1000 + index, 0.02, N, K, meta_kind)
            for copy in range(copies):
                self.weights[copy].append(ctx.q4_prepare(*self.host[name], N, K, meta_kind))
            if K not in self.x_ptr:
                rows = [engine.synth_normal_f16(77 + 1000 * m + K, 1.0, K) for m in range(max_rows)]
                self.host[("x", K)] = np.stack(rows)
                self.x_ptr[K] = ctx.to_device(self.host[("x", K)])
            self.y_ptr[name] = ctx.alloc(max(max_rows * N * 2, 16))
            if verbose:
                print(f"# prepared {name} {N}x{K} x{copies} in {time.perf_counter() - t0:.2f}s",
                      file=sys.stderr, flush=True)

    def calls(self, M, fuse=True, silu=False):
        """One call array per copy: linears that read the same activations go out as one launch
        (q|k|v, gate|up); rows 0..M-1 of the activations.  silu: the gate|up launch writes
        h = silu(gate . x) * (up . x) into gate's output buffer and down_proj reads that h (the MLP
        as a layer runs it) instead of its own synthetic activations."""
        engine, out = self.engine, []
        for copy in range(self.copies):
            groups = []
            for i, (name, N, K) in enumerate(self.shapes):
                target = (self.weights[copy][i], self.y_ptr[name])
                share = fuse and groups and groups[-1][1] == K and name.split("_")[0] in ("k", "v", "up")
                if share:
                    groups[-1][0].append(target)
                else:
                    groups.append(([target], K, name))
            items = []
            for targets, K, name in groups:
                fused = silu and len(targets) == 2
                x = self.y_ptr["gate_proj"] if silu and name == "down_proj" and "gate_proj" in self.y_ptr else self.x_ptr[K]
                items.append((targets, x, engine.F16, M, engine.F16, engine.F32, engine.FUSE_GATE_UP_SILU if fused else 0))
            out.append(engine.make_calls(items))
        return out

    def digest(self):
        """SHA-256 over the packed synthetic weights (codes, then metadata planes, matrix by matrix)."""
        import hashlib
        digest = hashlib.sha256()
        for name, _, _ in self.shapes:
            for plane in self.host[name]:
                if plane is not None:
                    digest.update(np.ascontiguousarray(plane).view(np.uint8))
        return digest.hexdigest()

    def destroy(self):
        for copy in self.weights:
            for weight in copy:
                weight.destroy()


def measure_layer(ctx, work, M, steps, warmup, preheat_ms, fuse=True, silu=False, graph=False):
    """Times `steps` layer steps at M rows; returns the figures of one layer line."""
    calls = work.calls(M, fuse=fuse, silu=silu)
    copies = work.copies
    launches_per_step = len(calls[0])
    step_bytes = sum(q4_bytes(N, K, M) for _, N, K in work.shapes)

    def run_steps(count):
        for step in range(count):
            ctx.q4_sequence(calls[step % copies])

    graphs = [ctx.q4_sequence_record(c) for c in calls] if graph else None

    def run_timed(count):
        if graphs is None:
            return run_steps(count)
        for step in range(count):
            ctx.graph_launch(graphs[step % copies])

    heated = preheat(ctx, run_timed, preheat_ms, 100) if preheat_ms > 0 else 0.0
    run_timed(warmup)
    ctx.sync()
    t0 = time.perf_counter()
    ctx.timer_begin()
    run_timed(steps)
    gpu_ms = ctx.timer_end()  # waits for the stream
    ctx.sync()
    wall = time.perf_counter() - t0

    # second pass of the same steps with an event pair bound to every dispatch (after the
    # warm-up steps in the same mode, see time_steps)
    ctx.profile_begin()
    run_steps(max(warmup, 2))
    ctx.profile_end()
    ctx.profile_begin()
    run_steps(steps)
    kernel_ms, launches = ctx.profile_end()
    per_launch = ctx.profile_durations()
    if launches % steps == 0:  # calls that went out together as one kernel count as one launch
        launches_per_step = int(launches) // steps
    for g in graphs or []:
        ctx.graph_destroy(g)
    # kernel time of each step (its launches, and the slice reductions some of them carry)
    per_step = per_launch[:len(per_launch) // steps * steps].reshape(steps, -1).sum(axis=1)
    p10, p50, p90 = (float(np.percentile(per_step, q)) for q in (10, 50, 90))
    launch_p50 = None  # median duration of each launch of a step, in launch order
    if len(per_launch) == steps * launches_per_step:
        launch_p50 = [round(float(v), 2) for v in np.median(per_launch.reshape(steps, launches_per_step), axis=0)]
    bytes_per_launch = step_bytes / launches_per_step
    avg_kernel_us = kernel_ms * 1e3 / max(launches, 1)
    return {
        "calls": calls, "run_steps": run_steps, "wall": wall, "gpu_ms": gpu_ms, "preheat_ms": heated,
        "step_bytes": step_bytes, "launches_per_step": launches_per_step, "launches": int(launches),
        "value": step_bytes * steps / wall / 1e9,
        "kernel_us_per_step": (p10, p50, p90), "launch_p50": launch_p50,
        "bytes_per_launch": bytes_per_launch, "avg_kernel_us": avg_kernel_us,
        "achieved": bytes_per_launch / (avg_kernel_us * 1e-6) / 1e9,
    }


def cpu_baseline_layer(oracle, shapes, host, M, meta_kind, budget_s=10.0):
    """The oracle's reference-faithful flavour (fp32, k order) on the host's threads: passes over
    the layer for about `budget_s` seconds (at least 5, at most 200), the median taken."""
    threads, allowed = host_threads()
    total_bytes = sum(q4_bytes(N, K, M) for _, N, K in shapes)

    def one_pass(count):
        t0 = time.perf_counter()
        for name, N, K in shapes:
            quants, meta_a, meta_b = host[name]
            oracle.q4_linear(quants, meta_a, meta_b, meta_kind, N, K, host[("x", K)][:M], oracle.X_F16,
                             M, oracle.W_EXACT, oracle.ACC_F32_SEQUENTIAL, threads=count)
        return time.perf_counter() - t0

    times, repeats, rep = [], 5, 0
    while rep < repeats + 1:
        seconds = one_pass(threads)
        if rep:
            times.append(seconds)
        if rep == 1:  # the first pass warms up; the second sizes the sample
            repeats = max(5, min(200, int(budget_s / max(times[0], 1e-4))))
        rep += 1
    median = sorted(times)[len(times) // 2]
    four = one_pass(4)  # the reference's deployment width: four threads (one pass)
    return {
        "value": round(total_bytes / median / 1e9, 3),
        "value_at_4_threads": round(total_bytes / four / 1e9, 3),
        "unit": "GB/s",
        **host_fields(oracle, threads, allowed),
        "kind": "port",
        "sample": f"{repeats} passes over the same layer (median), oracle restatement of "
                  f"cpu_row_dot, OpenMP static over rows, {median * 1e3:.1f} ms per pass",
    }


# ---- prefill -----------------------------------------------------------------------------------

def measure_prefill(engine, ctx, M, steps, warmup, preheat_ms, weights=None, host=None, with_cpu=True):
    """gate, up (one call, shared activations) and down at M rows: fp16 matrix-instruction GEMMs.
    `weights`: per copy [gate, up, down] prepared weights to reuse (and `host` their images)."""
    meta_kind = engine.META_BF16_PLANES
    own = weights is None
    if own:
        weights, host = [[] for _ in range(2)], {}
        for index, (name, N, K) in enumerate(PREFILL):
            host[name] = engine.synth_q4_affine(1004 + index, 0.02, N, K, meta_kind)
            for copy in range(2):
                weights[copy].append(ctx.q4_prepare(*host[name], N, K, meta_kind))
    copies = len(weights)
    x_host, x_ptr, y_ptr = {}, {}, {}
    for name, N, K in PREFILL:
        if K not in x_ptr:
            x_host[K] = engine.synth_normal_f16(77 + K, 1.0, M * K).reshape(M, K)
            x_ptr[K] = ctx.to_device(x_host[K])
        y_ptr[name] = ctx.alloc(M * N * 2)
    calls = []
    for copy in range(copies):
        gate, up, down = weights[copy]
        calls.append(engine.make_calls([
            ([(gate, y_ptr["gate_proj"]), (up, y_ptr["up_proj"])], x_ptr[5120], engine.F16, M, engine.F16),
            ((down, y_ptr["down_proj"]), x_ptr[17408], engine.F16, M, engine.F16)]))

    def run_steps(count):
        for step in range(count):
            ctx.q4_sequence(calls[step % copies])

    timed = time_steps(ctx, run_steps, steps, warmup, preheat_ms, preheat_batch=10)
    step_flops = sum(2.0 * M * N * K for _, N, K in PREFILL)
    value = step_flops * steps / timed["wall"] / 1e12
    achieved = step_flops * steps / (timed["kernel_ms"] * 1e-3) / 1e12
    # kernel time per linear: launches of a step in order are gate, up, down (+ a reduction kernel
    # behind any of them that is cut in K splits)
    result = {
        "tflops": round(value, 2),
        "percent_of_f16_peak": round(100.0 * value / F16_MFMA_PEAK_TFLOPS, 2),
        "wall": timed["wall"], "gpu_ms": timed["gpu_ms"], "preheat_ms": round(timed["preheat_ms"], 1),
        "step_flops": step_flops,
        "roofline": {
            "bound": "mfma",
            "achieved": round(achieved, 2),
            "peak": F16_MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / F16_MFMA_PEAK_TFLOPS, 4),
            "traffic": None,
            "kernel": "q4_gemm_pipe_kernel (with the K-split reduction where one runs)",
            "launches": timed["launches"],
            "kernel_us_per_linear": round(timed["kernel_ms"] * 1e3 / (3 * steps), 3),
            "kernel_us_per_step": round(timed["kernel_ms"] * 1e3 / steps, 3),
            "algorithmic_flops_per_linear": step_flops / 3,
        },
    }
    if with_cpu:
        import oracle  # test infrastructure, used here only as the timed CPU baseline
        threads, allowed = host_threads()
        rows = min(M, 4)  # bounded sample: the first rows of the same activations
        t0 = time.perf_counter()
        for name, N, K in PREFILL:
            oracle.q4_linear(*host[name], meta_kind, N, K, x_host[K][:rows], oracle.X_F16, rows,
                             oracle.W_EXACT, oracle.ACC_F32_SEQUENTIAL, threads=threads)
        seconds = time.perf_counter() - t0
        result["cpu_baseline"] = {
            "value": round(step_flops * rows / M / seconds / 1e12, 5), "unit": "TFLOP/s",
            "cores": threads, "kind": "port",
            "sample": "the first %d of the %d rows through the three linears, oracle restatement of "
                      "cpu_row_dot, OpenMP static over output rows, %.2f s" % (rows, M, seconds)}
    for pointer in list(x_ptr.values()) + list(y_ptr.values()):
        ctx.free(pointer)
    if own:
        for copy in weights:
            for weight in copy:
                weight.destroy()
    return result


def bench_prefill(engine, ctx, args):
    M = args.rows
    r = measure_prefill(engine, ctx, M, args.steps, args.warmup, args.preheat_ms, with_cpu=not args.no_cpu)
    result = {
        "metric": "q4_prefill_tflops_m%d_27b_mlp" % M,
        "value": r["tflops"],
        "unit": "TFLOP/s",
        **common_fields(args, r["wall"]),
        "dtype": "u4 codes dequantized to f16, f16 matrix instructions, f32 accumulate",
        "data": "synthetic (seeded N(0,0.02) weights min/max-quantized to affine-Q4 g64, N(0,1) "
                "fp16 activations)",
        "config": {
            "workload": "27B-shaped MLP linears gate/up (5120->17408) and down (17408->5120) at M=%d, "
                        "affine-Q4 g64, bf16 scale+bias, fp16 x and y" % M,
            "linears_per_step": 3,
            "algorithmic_flops_per_step": r["step_flops"],
            "percent_of_f16_peak": r["percent_of_f16_peak"],
            "preheat_ms": r["preheat_ms"],
            # what the matrix instruction sustains here from registers: alone, and with two or
            # three packed-fp16 vector instructions per matrix instruction (in-register dequantization)
            "measured_mfma_tflops": {"alone": round(ctx.probe_mfma_rate(0), 1),
                                     "with_2_valu": round(ctx.probe_mfma_rate(2), 1),
                                     "with_3_valu": round(ctx.probe_mfma_rate(3), 1)},
            "gpu_event_ms_per_step": round(r["gpu_ms"] / args.steps, 5),
            **device_fields(ctx.info()),
        },
        "roofline": r["roofline"],
    }
    if "cpu_baseline" in r:
        result["cpu_baseline"] = r["cpu_baseline"]
    print(json.dumps(result), flush=True)
    return 0


# ---- W8A8 --------------------------------------------------------------------------------------

def measure_w8a8(engine, ctx, steps, warmup, preheat_ms, with_cpu=True):
    """One step: quantize the activations once, then three projections that share them."""
    M, K, N, count = W8A8["M"], W8A8["K"], W8A8["N"], W8A8["projections"]
    rows = [engine.synth_w8_rows(2000 + i, 0.02, N, K) for i in range(count)]
    weights = [ctx.w8a8_prepare(r, N, K) for r in rows]
    x = engine.synth_normal_f32(31, 1.0, M * K).reshape(M, K)
    bias = [engine.synth_normal_f32(41 + i, 0.1, N) for i in range(count)]
    x_ptr, q_ptr, s_ptr = ctx.to_device(x), ctx.alloc(M * K), ctx.alloc(M * 4)
    bias_ptr = [ctx.to_device(b) for b in bias]
    out_ptr = [ctx.alloc(M * N * 4) for _ in range(count)]
    acc_ptr = [ctx.alloc(M * N * 4) for _ in range(count)]

    def run_steps(n):
        for _ in range(n):
            ctx.quantize_i8_device(x_ptr, M, K, q_ptr, s_ptr)
            ctx.w8a8_linear_multi_device(weights, q_ptr, s_ptr, M, bias_ptr, out_ptr, acc_ptr)

    timed = time_steps(ctx, run_steps, steps, warmup, preheat_ms, preheat_batch=200)
    step_ops = 2.0 * M * K * N * count
    value = step_ops * steps / timed["wall"] / 1e12
    achieved = step_ops * steps / (timed["kernel_ms"] * 1e-3) / 1e12
    per_launch = timed["per_launch_us"]
    gemm_us = float(np.median(per_launch[1::2])) if len(per_launch) == 2 * steps else None
    weight_bytes = count * N * (4 + K)
    result = {
        "tops": round(value, 3), "wall": timed["wall"], "gpu_ms": timed["gpu_ms"],
        "preheat_ms": round(timed["preheat_ms"], 1), "step_ops": step_ops,
        "projection_launch_us_p50": round(gemm_us, 2) if gemm_us else None,
        "weight_gb_per_s_at_p50": round(weight_bytes / (gemm_us * 1e-6) / 1e9, 1) if gemm_us else None,
        "roofline": {
            "bound": "mfma",
            "achieved": round(achieved, 3),
            "peak": I8_MFMA_PEAK_TOPS,
            "unit": "TOP/s",
            "frac": round(achieved / I8_MFMA_PEAK_TOPS, 5),
            "traffic": None,
            "kernel": "w8a8_kernel (quantize_i8_kernel included in the time)",
            "launches": timed["launches"],
            "avg_kernel_us": round(timed["kernel_ms"] * 1e3 / max(timed["launches"], 1), 3),
        },
    }
    if with_cpu:
        import oracle  # test infrastructure: the timed CPU baseline and the bit-exactness check
        threads, _ = host_threads()
        q_ref, s_ref = oracle.quantize_i8(x)
        repeats, t0 = 20, time.perf_counter()
        for _ in range(repeats):
            oracle.quantize_i8(x)
            refs = [oracle.w8a8_linear(rows[i], N, K, q_ref, s_ref, bias[i], threads=threads)
                    for i in range(count)]
        seconds = (time.perf_counter() - t0) / repeats
        exact = bool(np.array_equal(ctx.download(q_ptr, (M, K), np.int8), q_ref))
        for i in range(count):
            exact &= bool(np.array_equal(ctx.download(acc_ptr[i], (M, N), np.int32), refs[i][1]))
            exact &= bool(np.array_equal(ctx.download(out_ptr[i], (M, N), np.float32), refs[i][0]))
        result["bit_exact_vs_oracle"] = exact
        result["cpu_baseline"] = {
            "value": round(step_ops / seconds / 1e12, 5), "unit": "TOP/s", "cores": threads, "kind": "port",
            "sample": "%d passes of the same step (mean), oracle restatement of quantize_i8 and "
                      "matrix_sequence_i8_quantized, OpenMP static over output rows, %.2f ms per pass"
                      % (repeats, seconds * 1e3)}
    for pointer in [x_ptr, q_ptr, s_ptr] + bias_ptr + out_ptr + acc_ptr:
        ctx.free(pointer)
    for weight in weights:
        ctx.w8a8_destroy(weight)
    return result


Q8_AFFINE = {"N": 25600, "K": 5120}  # gate/up projection of the H3 text conditioner (minimax_h3_m3_e2e.m:2197-2205)


def measure_q8_affine(engine, ctx, rows_list=(1, 256), copies=3):
    """Affine-Q8 g64 linear (minimax_h3_q8_gemm_bf16_meta's format) of the conditioner's gate shape:
    GB/s of the weight image at M = 1, TFLOP/s at prefill M.  Up to 16 rows the weight is one Q4
    weight of twice the columns (high nibbles | low nibbles) whose second half meets the activation
    row again from its start, so a linear is one Q4 streaming linear; above, the pipelined GEMM
    kernel multiplies the bytes themselves (a second copy of the weight, in GEMM tiles).  Random
    codes and metadata: timing only, parity is the GPU tests' business."""
    N, K = Q8_AFFINE["N"], Q8_AFFINE["K"]
    rng = np.random.default_rng(77)
    quants = rng.integers(0, 256, size=N * K, dtype=np.uint8)
    scales = (rng.random(N * (K // 64), dtype=np.float32) * 2e-4 + 2e-4)
    biases = -scales * 128.0
    to_bf16 = lambda v: (v.view(np.uint32) >> 16).astype(np.uint16)
    weights = [ctx.q8_prepare(quants, to_bf16(scales), to_bf16(biases), N, K, engine.META_BF16_PLANES)
               for _ in range(copies)]
    image_bytes = N * K + N * (K // 64) * 4
    out = {}
    for M in rows_list:
        x_ptr = ctx.to_device(engine.synth_normal_f16(5, 1.0, M * K).reshape(M, K))
        y_ptr = ctx.alloc(M * N * 2)
        state = {"i": 0}

        def run_steps(n):
            for _ in range(n):
                ctx.q8_linear_device(weights[state["i"] % copies], x_ptr, engine.F16, M, y_ptr, engine.F16)
                state["i"] += 1

        steps = 60 if M == 1 else 20
        timed = time_steps(ctx, run_steps, steps, 6, 20.0, preheat_batch=20)
        kernel_s = timed["kernel_ms"] * 1e-3 / steps
        entry = {"rows": M, "steps": steps, "launches_per_linear": timed["launches"] // steps,
                 "kernel_us_per_linear": round(kernel_s * 1e6, 2),
                 "wall_us_per_linear": round(timed["wall"] / steps * 1e6, 2)}
        if M <= 16:
            achieved = (image_bytes + M * K * 2 + M * N * 2) / kernel_s / 1e9
            entry.update({"gb_per_s": round(achieved, 1),
                          "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                                       "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                                       "kernel": "q4_stream_kernel over [high | low nibbles] x [x | x]"}})
        else:
            achieved = 2.0 * M * N * K / kernel_s / 1e12
            entry.update({"tflops": round(achieved, 1),
                          "roofline": {"bound": "mfma", "achieved": round(achieved, 1), "peak": F16_MFMA_PEAK_TFLOPS,
                                       "unit": "TFLOP/s", "frac": round(achieved / F16_MFMA_PEAK_TFLOPS, 4),
                                       "kernel": "q4_gemm_pipe_kernel<128, 3, true, false, true>: 8-bit codes, "
                                                 "13 tiles per workgroup (16 where they fill the compute units better)"}})
        out["q8_affine_g64_m%d" % M] = entry
        ctx.free(x_ptr)
        ctx.free(y_ptr)
    for weight in weights:
        ctx.q8_destroy(weight)
    return out


def bench_w8a8(engine, ctx, args):
    M, K, N, count = W8A8["M"], W8A8["K"], W8A8["N"], W8A8["projections"]
    r = measure_w8a8(engine, ctx, args.steps, args.warmup, args.preheat_ms, with_cpu=not args.no_cpu)
    result = {
        "metric": "w8a8_tops_m64_k1024_n4096",
        "value": r["tops"],
        "unit": "TOP/s",
        **common_fields(args, r["wall"]),
        "dtype": "i8 x i8, i32 accumulate, f32 epilogue",
        "data": "synthetic (seeded N(0,0.02) weights absmax-quantized per row, N(0,1) fp32 activations "
                "quantized per token on the GPU)",
        "config": {
            "workload": "per-token int8 quantization then %d projections M=%d K=%d N=%d with bias"
                        % (count, M, K, N),
            "launches_per_step": 2,
            "projections_share_one_launch": True,
            "algorithmic_ops_per_step": r["step_ops"],
            "preheat_ms": r["preheat_ms"],
            "projection_launch_us_p50": r["projection_launch_us_p50"],
            "weight_gb_per_s_at_p50": r["weight_gb_per_s_at_p50"],
            "gpu_event_ms_per_step": round(r["gpu_ms"] / args.steps, 5),
            **device_fields(ctx.info()),
        },
        "roofline": r["roofline"],
    }
    if "cpu_baseline" in r:
        result["config"]["bit_exact_vs_oracle"] = r["bit_exact_vs_oracle"]
        result["cpu_baseline"] = r["cpu_baseline"]
    print(json.dumps(result), flush=True)
    return 0


# ---- configuration 1 ----------------------------------------------------------------------------

def sym128_records(weights):
    """fp32 [N][K] -> the symmetric group-128 records of compiler/q4_image.py as the C runtimes read
    them (qwen35_task.c:286-303,426-450): per (row, 128 columns) a bf16 scale and 64 code bytes, element
    j in byte j/2, even j in the low nibble, a two's complement value in [-8, 7]."""
    N, K = weights.shape
    blocks = weights.reshape(N, K // 128, 128)
    scale = np.maximum(-blocks.min(axis=-1) / np.float32(8.0), blocks.max(axis=-1) / np.float32(7.0))
    scale[scale == 0] = np.float32(1.0)
    bits = scale.astype(np.float32).view(np.uint32).astype(np.uint64)
    bf16 = (((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)
    scale = (bf16.astype(np.uint32) << 16).view(np.float32)
    nibbles = (np.clip(np.rint(blocks / scale[..., None]), -8, 7).astype(np.int16) & 0xF).astype(np.uint8)
    records = np.empty((N, K // 128, 66), dtype=np.uint8)
    records[..., :2] = bf16.view(np.uint8).reshape(N, K // 128, 2)
    records[..., 2:] = nibbles[..., 0::2] | (nibbles[..., 1::2] << 4)
    return np.ascontiguousarray(records).reshape(-1)


def measure_config1(engine, ctx, with_cpu=True, copies=600, steps=1200):
    """BASELINE configuration 1: the 0.8B-scale linear K=1024, N=3584 at M=1, affine-Q4 g64 with fp16
    scale+bias, fp16 x and y (2,073,600 algorithmic bytes a call), rotating over `copies` prepared
    copies; and the same shape in the symmetric group-128 format with fp32 x and y, which is what the
    reference's portable runtime runs on CPU (q4_gemv, qwen35_task.c:318-362)."""
    (name, N, K), = CONFIG1
    work = LayerWorkload(engine, ctx, CONFIG1, copies, engine.META_F16_INTERLEAVED, 1)
    r = measure_layer(ctx, work, 1, steps, 100, 20.0)
    out = {
        "workload": "affine-Q4 g64 GEMV K=%d N=%d M=1, fp16 scale+bias, fp16 x and y" % (K, N),
        "gb_per_s": round(r["value"], 1), "steps": steps, "weight_copies_rotated": copies,
        "rotated_bytes": r["step_bytes"] * copies, "kernel_us_per_launch_p50": round(r["kernel_us_per_step"][1], 2),
        "wall_us_per_call": round(r["wall"] / steps * 1e6, 2),
        "roofline": {"bound": "hbm", "achieved": round(r["achieved"], 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(r["achieved"] / HBM_PEAK_GBPS, 4), "kernel": "q4_stream_kernel",
                     "avg_kernel_us": round(r["avg_kernel_us"], 3),
                     "algorithmic_bytes_per_launch": round(r["bytes_per_launch"], 1)},
    }
    # the same shape as symmetric group-128 records: prepared once per copy, fp32 in and out
    weights32 = engine.synth_normal_f32(4242, 0.02, N * K).reshape(N, K)
    records = sym128_records(weights32)
    x32 = engine.synth_normal_f32(4243, 1.0, K)
    sym_copies = 64
    sym = [ctx.sym128_prepare(records, N, K) for _ in range(sym_copies)]
    x_ptr, y_ptr = ctx.to_device(x32), ctx.alloc(N * 4)
    state = {"i": 0}

    def run_steps(n):
        for _ in range(n):
            ctx.q4_linear_device(sym[state["i"] % sym_copies], x_ptr, engine.F32, 1, y_ptr, engine.F32)
            state["i"] += 1

    timed = time_steps(ctx, run_steps, 400, 40, 10.0, preheat_batch=100)
    out["sym128_m1"] = {"workload": "symmetric Q4 g128 records (66 bytes a group), fp32 x and y, same shape",
                        "record_bytes": int(records.size), "launches_per_call": timed["launches"] // 400,
                        "kernel_us_per_call": round(timed["kernel_ms"] * 1e3 / 400, 2),
                        "wall_us_per_call": round(timed["wall"] / 400 * 1e6, 2)}
    if with_cpu:
        import oracle  # test infrastructure, used here only as the timed CPU baseline
        threads, allowed = host_threads()
        quants, meta_a, meta_b = work.host[name]
        x16 = work.host[("x", K)][:1]

        def median_seconds(call, repeats=200):
            call()
            times = []
            for _ in range(repeats):
                t0 = time.perf_counter()
                call()
                times.append(time.perf_counter() - t0)
            return sorted(times)[len(times) // 2]

        affine = lambda n: oracle.q4_linear(quants, meta_a, meta_b, engine.META_F16_INTERLEAVED, N, K, x16, oracle.X_F16,
                                            1, oracle.W_EXACT, oracle.ACC_F32_SEQUENTIAL, threads=n)
        seconds, seconds4 = median_seconds(lambda: affine(threads)), median_seconds(lambda: affine(4))
        bytes_call = q4_bytes(N, K, 1)
        out["cpu_baseline"] = {
            "value": round(bytes_call / seconds / 1e9, 3), "value_at_4_threads": round(bytes_call / seconds4 / 1e9, 3),
            "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "200 calls (median), oracle restatement of cpu_row_dot, OpenMP static over rows, %.1f us a call"
                      % (seconds * 1e6)}
        sym_bytes = records.size + K * 4 + N * 4
        restated = median_seconds(lambda: oracle.sym128_gemv(records, 0, N, K, x32, threads=threads))
        column = {"value": round(sym_bytes / restated / 1e9, 3), "unit": "GB/s of the record image", "cores": threads,
                  "kind": "port", "us_per_call": round(restated * 1e6, 1),
                  "sample": "200 calls (median), oracle restatement of q4_gemv (qwen35_task.c:318-362), OpenMP static "
                            "over rows"}
        reference = oracle.ref_qwen35()
        if reference is not None:  # the reference's own q4_gemv compiled from where it lies (oracle/_ref)
            y = np.empty(N, dtype=np.float32)
            own = median_seconds(lambda: reference.ref_qwen35_q4_gemv(records.ctypes.data, 0, N, K, x32.ctypes.data,
                                                                      y.ctypes.data))
            column["reference_build"] = {
                "value": round(sym_bytes / own / 1e9, 3), "unit": "GB/s of the record image", "kind": "reference",
                "us_per_call": round(own * 1e6, 1), "cores": os.environ.get("OMP_NUM_THREADS") or allowed,
                "sample": "200 calls (median) of the reference's own q4_gemv (its OpenMP pragma, the process's "
                          "thread count)"}
        out["sym128_m1"]["cpu_baseline"] = column
    for pointer in (x_ptr, y_ptr):
        ctx.free(pointer)
    for weight in sym:
        weight.destroy()
    work.destroy()
    return out


# ---- the secondary figures of the default line --------------------------------------------------

def secondary_figures(engine, ctx, work, args):
    """The other configurations of the headline metric, measured briefly on the same weights."""
    out = {}
    for M in (2, 4, 8):
        r = measure_layer(ctx, work, M, 100, 10, 20.0)
        out["verify_m%d" % M] = {
            "gb_per_s": round(r["value"], 1),
            "percent_of_hbm_peak": round(100.0 * r["value"] / HBM_PEAK_GBPS, 2),
            "steps": 100, "warmup": 10,
            "roofline": {"bound": "hbm", "achieved": round(r["achieved"], 1), "peak": HBM_PEAK_GBPS,
                         "unit": "GB/s", "frac": round(r["achieved"] / HBM_PEAK_GBPS, 4),
                         "kernel": "q4_stream_kernel", "avg_kernel_us": round(r["avg_kernel_us"], 3),
                         "algorithmic_bytes_per_launch": round(r["bytes_per_launch"], 1)},
            "kernel_us_per_step_p50": round(r["kernel_us_per_step"][1], 2),
            "kernel_us_per_launch_p50_in_launch_order": r["launch_p50"],
        }
    # decode-identical verify (option "batch_invariant"): every row count takes the one-row launch's
    # waves and K slices, so a row's bits do not depend on the batch; what that costs per row count
    ctx.set_option("batch_invariant", "1")
    invariant = {}
    for M in (1, 2, 4, 8):
        r = measure_layer(ctx, work, M, 100, 10, 10.0)
        invariant["m%d" % M] = {"kernel_us_per_step_p50": round(r["kernel_us_per_step"][1], 2),
                                "kernel_us_per_launch_p50_in_launch_order": r["launch_p50"],
                                "hbm_frac_of_kernel_time": round(r["achieved"] / HBM_PEAK_GBPS, 4)}
    ctx.set_option("batch_invariant", None)
    out["verify_batch_invariant"] = {
        "what": "the layer with option batch_invariant = 1: row m of an M-row call equals the one-row call on "
                "x[m] bit for bit (compare kernel_us_per_step_p50 with verify_m* and the headline)",
        **invariant}
    # prefill: the MLP weights of the layer (every copy), M = 512
    mlp = [[copy[4], copy[5], copy[6]] for copy in work.weights]
    host = {name: work.host[name] for name, _, _ in PREFILL}
    p = measure_prefill(engine, ctx, 512, 30, 5, 50.0, weights=mlp, host=host, with_cpu=not args.no_cpu)
    out["prefill_m512"] = {"tflops": p["tflops"], "percent_of_f16_peak": p["percent_of_f16_peak"],
                           "steps": 30, "warmup": 5, "linears_per_step": 3,
                           "algorithmic_flops_per_step": p["step_flops"], "roofline": p["roofline"],
                           # what the matrix instruction sustains here from registers (power-limited clock):
                           # alone, and with two or three packed-fp16 vector instructions between two of them
                           "measured_mfma_tflops": {"alone": round(ctx.probe_mfma_rate(0), 1),
                                                    "with_2_valu": round(ctx.probe_mfma_rate(2), 1),
                                                    "with_3_valu": round(ctx.probe_mfma_rate(3), 1)}}
    if "cpu_baseline" in p:
        out["prefill_m512"]["cpu_baseline"] = p["cpu_baseline"]
    # the same three linears at M = 2048 (the shape divides evenly over the compute units from there on)
    p = measure_prefill(engine, ctx, 2048, 10, 3, 20.0, weights=mlp, host=host, with_cpu=False)
    out["prefill_m2048"] = {"tflops": p["tflops"], "percent_of_f16_peak": p["percent_of_f16_peak"],
                            "steps": 10, "warmup": 3, "linears_per_step": 3,
                            "algorithmic_flops_per_step": p["step_flops"], "roofline": p["roofline"]}
    w = measure_w8a8(engine, ctx, 200, 20, 20.0, with_cpu=not args.no_cpu)
    out["w8a8_m64_k1024_n4096"] = {"tops": w["tops"], "steps": 200, "warmup": 20, "projections_per_step": 3,
                                   "projection_launch_us_p50": w["projection_launch_us_p50"],
                                   "weight_gb_per_s_at_p50": w["weight_gb_per_s_at_p50"],
                                   "roofline": w["roofline"]}
    if "cpu_baseline" in w:
        out["w8a8_m64_k1024_n4096"]["bit_exact_vs_oracle"] = w["bit_exact_vs_oracle"]
        out["w8a8_m64_k1024_n4096"]["cpu_baseline"] = w["cpu_baseline"]
    out.update(measure_q8_affine(engine, ctx))
    out["config1_m1"] = measure_config1(engine, ctx, with_cpu=not args.no_cpu)
    return out


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=400)
    parser.add_argument("--warmup", type=int, default=40)
    parser.add_argument("--copies", type=int, default=8)
    parser.add_argument("--rows", type=int, default=None,
                        help="activation rows M (default 1; 512 for --workload prefill)")
    parser.add_argument("--workload", default="layer_m1", choices=["layer_m1", "config1", "lm_head", "prefill", "w8a8", "q8"])
    parser.add_argument("--preheat-ms", type=float, default=100.0,
                        help="GPU time of untimed steps before anything is timed (0: none)")
    parser.add_argument("--unfused", action="store_true",
                        help="one launch per linear instead of shared-x launches for q|k|v and gate|up")
    parser.add_argument("--graph", action="store_true",
                        help="replay each step from a recorded HIP graph (one host call per step) in "
                             "the timed pass; the per-kernel pass stays eager")
    parser.add_argument("--fused-mlp", action="store_true",
                        help="gate|up launch applies silu(gate)*up (one output instead of two) and down_proj "
                             "reads that output")
    parser.add_argument("--chain", action="store_true",
                        help="with --fused-mlp: context option chain = 1, the gate|up-SiLU launch and "
                             "down_proj go out as one kernel (three launches a step)")
    parser.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline legs")
    parser.add_argument("--no-secondary", action="store_true",
                        help="default workload only: leave out the verify / prefill / W8A8 figures")
    parser.add_argument("--verbose", action="store_true")
    args = parser.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (--gpus 1); nothing in it uses a second "
              "GPU", file=sys.stderr)
        return 2

    import mi355q as engine  # raises if the library is not built

    if args.rows is None:
        args.rows = 512 if args.workload == "prefill" else 1
    if args.workload == "q8":  # the affine-Q8 figures alone (for profiling); no line of the contract's shape
        with engine.Context(0) as ctx:
            print(json.dumps(measure_q8_affine(engine, ctx)), flush=True)
        return 0
    if args.workload in ("prefill", "w8a8"):
        if args.steps == 400 and args.warmup == 40:
            args.steps, args.warmup = 100, 10
        with engine.Context(0) as ctx:  # raises without a GPU
            return (bench_prefill if args.workload == "prefill" else bench_w8a8)(engine, ctx, args)
    shapes = {"layer_m1": LAYER, "config1": CONFIG1, "lm_head": LM_HEAD}[args.workload]
    meta_kind = engine.META_BF16_PLANES if args.workload == "layer_m1" else engine.META_F16_INTERLEAVED
    M = args.rows
    copies = {"layer_m1": args.copies, "config1": max(args.copies, 600), "lm_head": 2}[args.workload]
    if args.workload == "lm_head" and args.steps == 400 and args.warmup == 40:
        args.steps, args.warmup = 60, 6
    if args.chain:
        args.fused_mlp = True
    headline = args.workload == "layer_m1" and M == 1 and not (args.unfused or args.graph or args.fused_mlp)
    with_secondary = headline and not args.no_secondary
    ctx = engine.Context(0)  # raises without a GPU
    if args.chain:
        ctx.set_option("chain", "1")
    info = ctx.info()
    work = LayerWorkload(engine, ctx, shapes, copies, meta_kind, max(M, 8) if with_secondary else M,
                         args.verbose)
    r = measure_layer(ctx, work, M, args.steps, args.warmup, args.preheat_ms, fuse=not args.unfused,
                      silu=args.fused_mlp, graph=args.graph)
    step_bytes, launches_per_step = r["step_bytes"], r["launches_per_step"]

    # the same steps over one copy only: what a cache-resident weight set would show
    hot_steps = min(args.steps, 200)
    for step in range(args.warmup):
        ctx.q4_sequence(r["calls"][0])
    ctx.timer_begin()
    for step in range(hot_steps):
        ctx.q4_sequence(r["calls"][0])
    hot_ms = ctx.timer_end()

    # measured plain-read ceiling: whole 2 GiB pass, and launches the size of one weight matrix
    read_long = ctx.probe_read_bandwidth(2 << 30, 3, 1, 0)
    read_short = ctx.probe_read_bandwidth(2 << 30, 3, 1, int(step_bytes / launches_per_step))

    value, p = r["value"], r["kernel_us_per_step"]
    result = {
        "metric": {"layer_m1": "q4_gemv_hbm_gb_per_s_m%d_27b_layer",
                   "config1": "q4_gemv_hbm_gb_per_s_m%d_k1024_n3584",
                   "lm_head": "q4_gemv_hbm_gb_per_s_m%d_lm_head_248320x5120"}[args.workload] % M,
        "value": round(value, 2),
        "unit": "GB/s",
        **common_fields(args, r["wall"]),
        "dtype": "u4 codes x f16, f32 accumulate",
        "data": "synthetic (seeded N(0,0.02) weights min/max-quantized to affine-Q4 g64, N(0,1) "
                "fp16 activations)",
        "config": {
            "workload": ("27B-shaped decoder layer linears q/k/v/o/gate/up/down at M=%d, affine-Q4 "
                         "g64, bf16 scale+bias, fp16 x and y" % M) if args.workload == "layer_m1"
                        else "affine-Q4 g64 GEMV %s M=%d, fp16 scale+bias, fp16 x and y"
                             % (" ".join("K=%d N=%d" % (K, N) for _, N, K in shapes), M),
            "linears_per_step": len(shapes),
            "launches_per_step": launches_per_step,
            "gate_up_silu_fused": bool(args.fused_mlp),
            "mlp_as_one_launch": bool(args.chain),
            "steps_replayed_from_graph": bool(args.graph),
            "algorithmic_bytes_per_step": step_bytes,
            "weight_copies_rotated": copies,
            "rotated_bytes": step_bytes * copies,
            "preheat_ms": round(r["preheat_ms"], 1),
            "single_copy_gb_per_s": round(step_bytes * hot_steps / (hot_ms * 1e-3) / 1e9, 1),
            "percent_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
            "gpu_event_ms_per_step": round(r["gpu_ms"] / args.steps, 5),
            "kernel_us_per_step_p10_p50_p90": [round(p[0], 2), round(p[1], 2), round(p[2], 2)],
            "gb_per_s_at_p50_kernel_time": round(step_bytes / (p[1] * 1e-6) / 1e9, 1),
            "kernel_us_per_launch_p50_in_launch_order": r["launch_p50"],
            "weights_sha256": work.digest(),
            **device_fields(info),
            "measured_read_gb_per_s": {"one_2GiB_pass": round(read_long, 1),
                                       "matrix_sized_launches": round(read_short, 1)},
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(r["achieved"], 2),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(r["achieved"] / HBM_PEAK_GBPS, 4),
            "traffic": round(r["bytes_per_launch"] * MEASURED_TRAFFIC_RATIO_LAYER_M1) if headline else None,
            "traffic_source": ("rocprofv3 FETCH_SIZE + WRITE_SIZE per algorithmic byte = %.3f, read from "
                               "profiles/q4_stream_kernel_layer_m1.md (not measured in this run)"
                               % MEASURED_TRAFFIC_RATIO_LAYER_M1) if headline else None,
            "kernel": "q4_stream_kernel",
            "launches": r["launches"],
            "avg_kernel_us": round(r["avg_kernel_us"], 3),
            "algorithmic_bytes_per_launch": round(r["bytes_per_launch"], 1),
        },
    }
    if not args.no_cpu:
        import oracle  # test infrastructure, used here only as the timed CPU baseline
        result["cpu_baseline"] = cpu_baseline_layer(oracle, shapes, work.host, M, meta_kind)
    if with_secondary:
        result["secondary"] = secondary_figures(engine, ctx, work, args)
    print(json.dumps(result), flush=True)
    work.destroy()
    ctx.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
