#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

Default workload (`--workload layer_m1`): the linears of one Qwen3.8-27B-shaped
decoder layer at M=1 — q 5120->6144, k and v 5120->1024, o 6144->5120, gate and
up 5120->17408, down 17408->5120 — in affine-Q4 group-64 with bf16 scale/bias,
fp16 activations and fp16 outputs, on seeded synthetic weights (N(0,0.02)
before quantization) and activations (N(0,1)).  One step is one pass over the
seven linears of one weight copy (four launches: q|k|v and gate|up share their
activations and go out as one launch each, then o and down); successive steps rotate over `--copies`
distinct prepared copies (>= 1.5 GB in total) so that the 256 MB memory-side
cache cannot serve the weights and the figure is an HBM figure.

Prints ONE JSON line.  `value` is algorithmic bytes (N*K/2 + N*(K/64)*4 +
M*K*2 + M*N*2 per linear) per second of wall time over the timed steps, with
all inputs resident in HBM before the clock starts.  `roofline` prices the
dominant kernel (the weight-streaming Q4 kernel) against HBM: algorithmic bytes
per launch over the kernel's own average duration (HIP events bound to each
dispatch, measured in a second pass of the same steps).  `cpu_baseline` is the
CPU oracle (a C restatement of the reference's scalar loop, row-parallel with
OpenMP as the reference parallelises its GEMV) timed on this host on the same
layer.
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


def q4_bytes(N, K, M, y_bytes=2):
    return N * K // 2 + N * (K // 64) * 4 + M * K * 2 + M * N * y_bytes


def build_workload(engine, ctx, shapes, M, copies, meta_kind, verbose, fuse=True):
    """Prepares `copies` device copies of every matrix plus activations/outputs."""
    x_ptr, y_ptr, weights, host = {}, {}, [[] for _ in range(copies)], {}
    for index, (name, N, K) in enumerate(shapes):
        t0 = time.perf_counter()
        quants, meta_a, meta_b = engine.synth_q4_affine(1000 + index, 0.02, N, K, meta_kind)
        host[name] = (quants, meta_a, meta_b)
        for copy in range(copies):
            weights[copy].append(ctx.q4_prepare(quants, meta_a, meta_b, N, K, meta_kind))
        if K not in x_ptr:
            rows = [engine.synth_normal_f16(77 + 1000 * m + K, 1.0, K) for m in range(M)]
            host[("x", K)] = np.stack(rows)
            x_ptr[K] = ctx.to_device(host[("x", K)])
        y_ptr[name] = ctx.alloc(max(M * N * 2, 16))
        if verbose:
            print(f"# prepared {name} {N}x{K} x{copies} in {time.perf_counter() - t0:.2f}s",
                  file=sys.stderr, flush=True)
    calls = []
    for copy in range(copies):
        # linears that read the same activations go out as one launch (q|k|v, gate|up)
        groups = []
        for i, (name, N, K) in enumerate(shapes):
            target = (weights[copy][i], y_ptr[name])
            share = fuse and groups and groups[-1][1] == K and name.split("_")[0] in ("k", "v", "up")
            if share:
                groups[-1][0].append(target)
            else:
                groups.append(([target], K))
        calls.append(engine.make_calls([(targets, x_ptr[K], engine.F16, M, engine.F16)
                                        for targets, K in groups]))
    return calls, weights, host, x_ptr, y_ptr


def cpu_baseline(oracle, shapes, host, M, meta_kind, repeats=5):
    """The oracle's reference-faithful flavour (fp32, k order) on all host threads."""
    threads = min(os.cpu_count() or 1, 16)
    os.environ.setdefault("OMP_NUM_THREADS", str(threads))
    total_bytes = sum(q4_bytes(N, K, M) for _, N, K in shapes)
    times = []
    for rep in range(repeats + 1):
        t0 = time.perf_counter()
        for name, N, K in shapes:
            quants, meta_a, meta_b = host[name]
            oracle.q4_linear(quants, meta_a, meta_b, meta_kind, N, K, host[("x", K)], oracle.X_F16,
                             M, oracle.W_EXACT, oracle.ACC_F32_SEQUENTIAL, threads=threads)
        if rep:
            times.append(time.perf_counter() - t0)
    median = sorted(times)[len(times) // 2]
    return {
        "value": round(total_bytes / median / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{repeats} passes over the same layer (median), oracle restatement of "
                  f"cpu_row_dot, OpenMP static over rows, {median * 1e3:.1f} ms per pass",
    }


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=400)
    parser.add_argument("--warmup", type=int, default=40)
    parser.add_argument("--copies", type=int, default=8)
    parser.add_argument("--rows", type=int, default=1, help="activation rows M (1..8)")
    parser.add_argument("--workload", default="layer_m1", choices=["layer_m1", "config1"])
    parser.add_argument("--unfused", action="store_true",
                        help="one launch per linear instead of shared-x launches for q|k|v and gate|up")
    parser.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    parser.add_argument("--verbose", action="store_true")
    args = parser.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (--gpus 1); nothing in it uses a second "
              "GPU", file=sys.stderr)
        return 2

    import mi355q as engine  # raises if the library is not built

    shapes = LAYER if args.workload == "layer_m1" else CONFIG1
    meta_kind = engine.META_BF16_PLANES if args.workload == "layer_m1" else engine.META_F16_INTERLEAVED
    M = args.rows
    copies = args.copies if args.workload == "layer_m1" else max(args.copies, 600)
    ctx = engine.Context(0)  # raises without a GPU
    info = ctx.info()
    calls, weights, host, x_ptr, y_ptr = build_workload(engine, ctx, shapes, M, copies, meta_kind,
                                                        args.verbose, fuse=not args.unfused)
    launches_per_step = len(calls[0])
    step_bytes = sum(q4_bytes(N, K, M) for _, N, K in shapes)

    def run_steps(count):
        for step in range(count):
            ctx.q4_sequence(calls[step % copies])

    run_steps(args.warmup)
    ctx.sync()
    t0 = time.perf_counter()
    ctx.timer_begin()
    run_steps(args.steps)
    gpu_ms = ctx.timer_end()  # waits for the stream
    ctx.sync()
    wall = time.perf_counter() - t0

    # second pass of the same steps with an event pair bound to every dispatch
    ctx.profile_begin()
    run_steps(args.steps)
    kernel_ms, launches = ctx.profile_end()

    # measured plain-read ceiling: whole 2 GiB pass, and launches the size of one weight matrix
    read_long = ctx.probe_read_bandwidth(2 << 30, 3, 1, 0)
    read_short = ctx.probe_read_bandwidth(2 << 30, 3, 1, int(step_bytes / launches_per_step))

    value = step_bytes * args.steps / wall / 1e9
    bytes_per_launch = step_bytes / launches_per_step
    avg_kernel_us = kernel_ms * 1e3 / max(launches, 1)
    achieved = bytes_per_launch / (avg_kernel_us * 1e-6) / 1e9
    result = {
        "metric": "q4_gemv_hbm_gb_per_s_m1_27b_layer" if args.workload == "layer_m1"
                  else "q4_gemv_hbm_gb_per_s_m1_k1024_n3584",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3 / args.steps, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u4 codes x f16, f32 accumulate",
        "data": "synthetic (seeded N(0,0.02) weights min/max-quantized to affine-Q4 g64, N(0,1) "
                "fp16 activations)",
        "config": {
            "workload": ("27B-shaped decoder layer linears q/k/v/o/gate/up/down at M=%d, affine-Q4 "
                         "g64, bf16 scale+bias, fp16 x and y" % M) if args.workload == "layer_m1"
                        else "affine-Q4 g64 GEMV K=1024 N=3584 M=%d, fp16 scale+bias, fp16 x and y" % M,
            "linears_per_step": len(shapes),
            "launches_per_step": launches_per_step,
            "algorithmic_bytes_per_step": step_bytes,
            "weight_copies_rotated": copies,
            "rotated_bytes": step_bytes * copies,
            "percent_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
            "gpu_event_ms_per_step": round(gpu_ms / args.steps, 5),
            "device": info.name.decode(errors="replace").strip(),
            "arch": info.arch.decode(errors="replace"),
            "compute_units": info.compute_units,
            "measured_read_gb_per_s": {"one_2GiB_pass": round(read_long, 1),
                                       "matrix_sized_launches": round(read_short, 1)},
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": None,
            "kernel": "q4_stream_kernel",
            "launches": int(launches),
            "avg_kernel_us": round(avg_kernel_us, 3),
            "algorithmic_bytes_per_launch": round(bytes_per_launch, 1),
        },
    }
    if not args.no_cpu:
        import oracle  # test infrastructure, used here only as the timed CPU baseline
        result["cpu_baseline"] = cpu_baseline(oracle, shapes, host, M, meta_kind)
    print(json.dumps(result), flush=True)
    for copy in weights:
        for weight in copy:
            weight.destroy()
    ctx.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
