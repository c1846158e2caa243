#!/usr/bin/env python3
"""Benchmark of the HIP hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]

Prints ONE JSON line.  A "step" is one pass of the primary workload's kernel over one
batch of synthetic input already resident in HBM.  The line carries, next to the primary
record, an `also` list with the same measurements for the other headline workloads, each
with its own roofline object.

Timing: HIP events recorded on the library's own stream (the stream every kernel of the
device is queued on) around exactly K launches after W warm-ups; roofline.achieved is the
workload's ALGORITHMIC bytes (or flops) divided by that average launch duration.
cpu_baseline: the CPU oracle (restated Clang-backend kernels) timed on this host with the
reference's protocol - 1 warm-up, 3 runs, minimum (runtime/src/benchmark.rs:23-27) - on a
bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
BF16_PEAK_TFLOPS = 2500.0    # MI355X dense bf16 MFMA, published
METRIC = "bf16 GEMM TFLOP/s & flash-attn fwd TFLOP/s (% of peak); softmax HBM GB/s"


def _cpu_time(fn):
    fn()  # warm-up
    best = float("inf")
    for _ in range(3):
        t0 = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t0)
    return best


def bench_softmax(m, dev, steps, warmup, cpu):
    """configs[1]: row softmax over f32 [8192 x 8192], inputs normal(0, 2) from seed 2."""
    from morok_amd import ops, synth

    rows = cols = 8192
    n = rows * cols
    bx = dev.buffer(n * 4).ensure_allocated()
    by = dev.buffer(n * 4).ensure_allocated()
    ops.fill_normal(bx, n, sigma=2.0, seed=2, tensor_id=0)
    ms = m.time_launches(lambda: ops.softmax_f32(bx, by, rows, cols), steps, warmup)
    algo_bytes = 2 * n * 4  # one read + one write of the matrix
    gbs = algo_bytes / (ms * 1e-3) / 1e9
    rec = {
        "metric": "softmax HBM GB/s", "value": gbs, "unit": "GB/s", "ms_per_step": ms, "dtype": "f32",
        "config": {"workload": "row softmax f32 [8192x8192], normal(0,2), one fused kernel (configs[1])"},
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gbs / HBM_PEAK_GBS, "traffic": None, "kernel": "softmax_rows_in_regs<256,8,1>",
                     "algorithmic_bytes_per_launch": algo_bytes},
    }
    if cpu:
        from tests.oracle_lib import Oracle

        orc = Oracle()
        srows = 2048  # a quarter of the rows: ~1 s of CPU work per run
        x = synth.normal((srows, cols), 2, 0, sigma=2.0)
        t = orc.thread_count(srows * cols, srows)
        sec = _cpu_time(lambda: orc.softmax_f32(x, threads=t))
        # the oracle runs the reference's 3-kernel schedule; its algorithmic bytes are the same 2*n*4
        rec["cpu_baseline"] = {"value": 2 * srows * cols * 4 / sec / 1e9, "unit": "GB/s", "cores": t, "kind": "port",
                               "sample": f"{srows} of 8192 rows x 8192 cols, 3-kernel Clang-backend schedule, "
                                         f"{t} threads, min of 3 after 1 warm-up"}
    return rec


WORKLOADS = {"softmax": bench_softmax}
PRIMARY_ORDER = ["gemm", "flash", "softmax"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all", help="all | " + " | ".join(sorted(WORKLOADS)))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (every kernel shards into "
                 "independent units); run with --gpus 1")

    import morok_amd as m

    dev = m.Device("HIP:0")
    names = [w for w in PRIMARY_ORDER if w in WORKLOADS] if args.workload == "all" else [args.workload]
    recs = []
    for name in names:
        recs.append(WORKLOADS[name](m, dev, args.steps, args.warmup, not args.no_cpu_baseline))
        dev.synchronize()
        dev.lru_clear()
    primary = recs[0]
    line = {
        "metric": METRIC if args.workload == "all" else primary["metric"],
        "primary_metric": primary["metric"],
        "value": primary["value"], "unit": primary["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": primary["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": primary["dtype"], "data": "synthetic", "config": primary["config"],
        "roofline": primary["roofline"],
    }
    if "cpu_baseline" in primary:
        line["cpu_baseline"] = primary["cpu_baseline"]
    if len(recs) > 1:
        line["also"] = recs[1:]
    print(json.dumps(line))


if __name__ == "__main__":
    main()
