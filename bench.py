#!/usr/bin/env python3
"""Benchmark of the HIP hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]

Prints ONE JSON line.  A "step" is one pass of the primary workload's kernel over one
batch of synthetic input already resident in HBM.  The line carries, next to the primary
record, an `also` list with the same measurements for the other headline workloads, each
with its own roofline object.

Timing: HIP events recorded on the library's own stream (the stream every kernel of the
device is queued on) around exactly K launches after W warm-ups (and, before those, 300 ms of
untimed launches that let clocks and page mappings settle, reported as settle_ms);
roofline.achieved is the
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
MIB = 1 << 20
# roofline.traffic is not measured by this run (counters need a profiler run of their own): it is
# read from the committed rocprofv3 summary of the same workload, i.e. from the FETCH_SIZE and
# WRITE_SIZE passes recorded there, each scaled by what the same counter read for the 256 MiB copy
# kernel, and only when that summary names the kernel this run launched; otherwise null.
PROFILE_OF = {"softmax": "softmax_rows_in_regs_8192x8192_f32.txt", "gemm": "gemm_bf16_tile256_4096cubed.txt",
              "flash": "flash_fwd_d128_causal_8x32x4096x128.txt", "decoder": "decoder_block_4x2048_h4096.txt",
              "generated_tc": "generated_tensor_core_gemm_4096cubed.txt", "matmul_f32": "generated_f32_matmul_1024cubed.txt",
              "gemm_f16": "gemm_f16_tile256_4096cubed.txt", "flash_options": "flash_fwd_ext_d128_8x32x4096x128.txt",
              "linear_decode": "gemm_nt_skinny_1x12288x4096_x8.txt", "linear_decode_16": "gemm_nt_rows_16x12288x4096_x8.txt",
              "decoder_decode": "decoder_block_decode_16tokens_linear_layout.txt", "flash_decode": "flash_decode_1x32x1x4096_d128_x8.txt"}


def _profiled_traffic(workload, kernel):
    """(bytes per launch, source) for `kernel` from profiles/<summary>, or (None, reason)."""
    import re

    path = os.path.join(ROOT, "profiles", PROFILE_OF.get(workload, ""))
    if not os.path.isfile(path):
        return None, "no committed profile summary at run time"
    base = kernel.split("<")[0]
    for line in open(path):
        mt = re.match(r"\s*(\S.*?)\s+n=\s*\d+\s+FETCH.*->\s*([0-9.]+) MiB \| WRITE.*->\s*([0-9.]+) MiB", line)
        if mt and mt.group(1).split("<")[0] == base:
            return (float(mt.group(2)) + float(mt.group(3))) * MIB, "profiles/" + PROFILE_OF[workload]
    return None, "profiles/%s does not list kernel %s" % (PROFILE_OF[workload], base)


def _roofline(workload, bound, achieved, peak, unit, kernel, **extra):
    traffic, source = _profiled_traffic(workload, kernel)
    r = {"bound": bound, "achieved": achieved, "peak": peak, "unit": unit, "frac": achieved / peak, "traffic": traffic,
         "traffic_source": source, "kernel": kernel}
    r.update(extra)
    return r


METRIC = "bf16 GEMM TFLOP/s & flash-attn fwd TFLOP/s (% of peak); softmax HBM GB/s"


def _cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


SETTLE_MS = 300.0  # untimed launches before the W warm-up steps, see _settle()
REFERENCE_LEGS = True


def _settle(m, fn):
    """The first launches after idle run at ramping clocks and touch freshly mapped memory:
    on this part the same kernel measures 10-20 % slower in its first milliseconds than at the
    rate it then sustains indefinitely.  Every workload is therefore run untimed for SETTLE_MS
    of wall time before the W warm-up steps and the K timed steps."""
    import morok_amd

    dev = morok_amd.Device("HIP:0")
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < SETTLE_MS:
        for _ in range(10):
            fn()
        dev.synchronize()


def _launch_stats(m, fn, steps, warmup):
    """Average over exactly `steps` launches (one event pair around all of them), then a second
    pass with one event pair per launch for the median and the minimum."""
    _settle(m, fn)
    ms = m.time_launches(fn, steps, warmup)
    med, mn = m.time_each_launch(fn, max(steps, 20), 0)
    return ms, {"median_ms": med, "min_ms": mn}


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
    ms, stats = _launch_stats(m, lambda: ops.softmax_f32(bx, by, rows, cols), steps, warmup)
    algo_bytes = 2 * n * 4  # one read + one write of the matrix
    gbs = algo_bytes / (ms * 1e-3) / 1e9
    rec = {
        "metric": "softmax HBM GB/s", "value": gbs, "unit": "GB/s", "ms_per_step": ms, "dtype": "f32",
        "config": {"workload": "row softmax f32 [8192x8192], normal(0,2), one fused kernel (configs[1])"},
        "roofline": _roofline("softmax", "hbm", gbs, HBM_PEAK_GBS, "GB/s", "softmax_rows_in_regs<256,8,1>",
                              algorithmic_bytes_per_launch=algo_bytes),
    }
    rec.update(stats)
    if cpu:
        from tests.oracle_lib import Oracle

        orc = Oracle()
        srows = 8192  # the whole matrix; 4 passes of it (1 warm-up + 3 timed)
        x = synth.normal((srows, cols), 2, 0, sigma=2.0)
        t = orc.thread_count(srows * cols, srows)
        sec = _cpu_time(lambda: orc.softmax_f32(x, threads=t))
        # the oracle runs the reference's 3-kernel schedule; its algorithmic bytes are the same 2*n*4
        rec["cpu_baseline"] = {"value": 2 * srows * cols * 4 / sec / 1e9, "unit": "GB/s", "cores": t, "kind": "port",
                               "sample": f"all {srows} rows x 8192 cols, 3-kernel Clang-backend schedule, "
                                         f"{t} threads, min of 3 after 1 warm-up"}
    return rec


_CEILING = {}  # TFLOP/s of the MFMA-only calibration kernel, measured once per run


def _mfma_ceiling_tflops(m, dev, random_operands=True):
    """Rate of the register-only MFMA kernel at the size of the 4096^3 product (256 workgroups x 64
    K steps of a 256 x 256 tile), with the same settle / warm-up discipline as the workloads.
    random_operands: operand registers hold hashed values in [-1.7, 1.7) (the default: what a
    product of random matrices feeds the pipes) or small smooth values; the part is power-managed
    and sustains a lower clock the more the operand bits toggle."""
    from morok_amd import ops

    key = "f16" if random_operands == "f16" else "random" if random_operands else "smooth"
    if key not in _CEILING:
        scratch = dev.buffer(256).ensure_allocated()
        ms, _ = _launch_stats(m, lambda: ops.mfma_ceiling(scratch, 256, 64, random_operands=random_operands), 50, 5)
        _CEILING[key] = 2.0 * 4096 ** 3 / (ms * 1e-3) / 1e12
    return _CEILING[key]


def _gemm_cpu_baseline(M, N, K):
    from morok_amd import synth
    from tests.oracle_lib import Oracle

    orc = Oracle()
    a = synth.normal_bf16((M, K), 3, 0)
    b = synth.normal_bf16((K, N), 3, 1)
    t = orc.thread_count(M * N * K, M)
    sec = _cpu_time(lambda: orc.gemm_bf16(a, b, threads=t))
    return {"value": 2.0 * M * N * K / sec / 1e12, "unit": "TFLOP/s", "cores": t, "kind": "port",
            "sample": f"all {M} output rows (K=N=4096), f32-accumulate bf16 matmul kernel, "
                      f"{t} threads, min of 3 after 1 warm-up"}


def _vendor_gemm_tflops(n, steps, warmup):
    """torch.matmul (hipBLASLt) on the same shape and dtype, same settle discipline: a reference
    point outside the product path, reported when torch imports on this box."""
    try:
        import torch
    except Exception:
        return None
    if not torch.cuda.is_available():
        return None
    a = torch.randn(n, n, device="cuda", dtype=torch.bfloat16)
    b = torch.randn(n, n, device="cuda", dtype=torch.bfloat16)
    c = torch.empty(n, n, device="cuda", dtype=torch.bfloat16)
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < SETTLE_MS:
        for _ in range(10):
            torch.matmul(a, b, out=c)
        torch.cuda.synchronize()
    for _ in range(warmup):
        torch.matmul(a, b, out=c)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        torch.matmul(a, b, out=c)
    e1.record()
    torch.cuda.synchronize()
    return 2.0 * n ** 3 / (e0.elapsed_time(e1) / steps * 1e-3) / 1e12


def bench_gemm(m, dev, steps, warmup, cpu):
    """configs[2]: bf16 GEMM M=N=K=4096, inputs normal(0,1) rounded to bf16, f32 accumulate, bf16 out,
    through the caller path: Tensor::matmul -> prepare (schedule, kernel cache, plan) -> execute."""
    from morok_amd import ops, tensor, uop

    M = N = K = 4096
    ba = dev.buffer(M * K * 2).ensure_allocated()
    bb = dev.buffer(K * N * 2).ensure_allocated()
    ops.fill_normal(ba, M * K, seed=3, tensor_id=0, bf16=True)
    ops.fill_normal(bb, K * N, seed=3, tensor_id=1, bf16=True)
    c = tensor.Tensor.from_buffer(ba, (M, K), uop.BF16).matmul(tensor.Tensor.from_buffer(bb, (K, N), uop.BF16))
    plan = c.prepare()
    program = plan.kernel_name(0)  # the plan's one item: the hand-written kernel behind the Program interface
    if not program.startswith("gemm_bf16"):
        raise RuntimeError("Tensor::matmul did not select the hand-written bf16 GEMM: " + program)
    kernel = "gemm_bf16_tile256"     # the device function that Program launches for this shape
    ms, stats = _launch_stats(m, plan.execute, steps, warmup)
    flops = 2.0 * M * N * K
    tf = flops / (ms * 1e-3) / 1e12
    rec = {
        "metric": "bf16 GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "dtype": "bf16",
        "config": {"workload": "bf16 GEMM M=N=K=4096, normal(0,1) inputs, f32 accumulate, bf16 out, via "
                               "Tensor::matmul -> prepare -> execute (configs[2])"},
        "roofline": _roofline("gemm", "mfma", tf, BF16_PEAK_TFLOPS, "TFLOP/s", kernel, algorithmic_flops_per_launch=flops),
        "plan_item": program,
    }
    rec.update(stats)
    if REFERENCE_LEGS:
        # the same kernel called straight through the C ABI (no plan): shows what the plan costs
        bc = dev.buffer(M * N * 2).ensure_allocated()
        rec["direct_abi_ms_per_step"], _ = _launch_stats(m, lambda: ops.gemm_bf16(ba, bb, bc, M, N, K), steps, warmup)
        ceiling = _mfma_ceiling_tflops(m, dev)
        rec["roofline"].update(mfma_only_ceiling=ceiling, frac_of_ceiling=tf / ceiling,
                               mfma_only_ceiling_smooth_operands=_mfma_ceiling_tflops(m, dev, False))
        vendor = _vendor_gemm_tflops(M, steps, warmup)
        if vendor is not None:
            rec["vendor_reference"] = {"value": vendor, "unit": "TFLOP/s", "library": "torch.matmul (hipBLASLt), not on the "
                                       "product path", "ratio": tf / vendor}
    if cpu:
        rec["cpu_baseline"] = _gemm_cpu_baseline(M, N, K)
    return rec


def bench_gemm_f16(m, dev, steps, warmup, cpu):
    """The 4096^3 product in IEEE half precision through the same caller path: the f16 instantiation of
    the hand-written kernel (v_mfma_f32_16x16x32_f16), inputs normal(0,1) * 0.25 rounded to f16."""
    import numpy as np

    from morok_amd import synth, tensor, uop

    M = N = K = 4096
    a = (synth.normal((M, K), 3, 0) * np.float32(0.25)).astype(np.float16)
    b = synth.normal((K, N), 3, 1).astype(np.float16)
    ba, bb = m.Buffer.from_numpy(a.view(np.uint16)), m.Buffer.from_numpy(b.view(np.uint16))
    c = tensor.Tensor.from_buffer(ba, (M, K), uop.F16).matmul(tensor.Tensor.from_buffer(bb, (K, N), uop.F16))
    plan = c.prepare()
    program = plan.kernel_name(0)
    if not program.startswith("gemm_f16"):
        raise RuntimeError("Tensor::matmul did not select the hand-written f16 GEMM: " + program)
    ms, stats = _launch_stats(m, plan.execute, steps, warmup)
    flops = 2.0 * M * N * K
    tf = flops / (ms * 1e-3) / 1e12
    rec = {
        "metric": "f16 GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "dtype": "f16",
        "config": {"workload": "f16 GEMM M=N=K=4096, f32 accumulate, f16 out, via Tensor::matmul -> prepare -> execute"},
        # the dense f16 MFMA peak is the bf16 one
        "roofline": _roofline("gemm_f16", "mfma", tf, BF16_PEAK_TFLOPS, "TFLOP/s", "gemm_f16_tile256", algorithmic_flops_per_launch=flops),
        "plan_item": program,
    }
    rec.update(stats)
    if REFERENCE_LEGS:
        # register-only stream of the f16 instruction on the same values, and of the bf16 one beside it
        ceiling = _mfma_ceiling_tflops(m, dev, "f16")
        rec["roofline"].update(mfma_only_ceiling=ceiling, frac_of_ceiling=tf / ceiling, mfma_only_ceiling_bf16_instruction=_mfma_ceiling_tflops(m, dev))
    if cpu:
        from tests.oracle_lib import Oracle

        orc = Oracle()
        rows = 256
        sec = _cpu_time(lambda: orc.gemm_f16(a[:rows], b))
        rec["cpu_baseline"] = {"value": 2.0 * rows * N * K / sec / 1e12, "unit": "TFLOP/s", "cores": orc.max_threads, "kind": "port",
                               "sample": f"{rows} of the {M} output rows (K=N=4096), f32-accumulate f16 matmul, min of 3 after 1 warm-up"}
    return rec


def bench_flash(m, dev, steps, warmup, cpu):
    """configs[3]: causal flash-attention forward, bf16 Q/K/V [8, 32, 4096, 128], scale 1/sqrt(128)."""
    from morok_amd import ops, synth

    B, H, S, D = 8, 32, 4096, 128
    n = B * H * S * D
    bq, bk, bv, bo = (dev.buffer(n * 2).ensure_allocated() for _ in range(4))
    for i, b in enumerate((bq, bk, bv)):
        ops.fill_normal(b, n, seed=4, tensor_id=i, bf16=True)
    scale = 1.0 / np.sqrt(D)
    steps = max(1, min(steps, 20))
    ms, stats = _launch_stats(m, lambda: ops.flash_attn_fwd_bf16(bq, bk, bv, bo, B, H, S, S, D, scale, True), steps,
                              warmup)
    flops = 0.5 * 4.0 * B * H * S * S * D  # causal convention: half of the dense 4*B*H*S^2*D
    tf = flops / (ms * 1e-3) / 1e12
    rec = {
        "metric": "flash-attn fwd TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "dtype": "bf16",
        "steps": steps,
        "config": {"workload": "causal flash-attention fwd, bf16 [8,32,4096,128], scale 1/sqrt(128) (configs[3])"},
        "roofline": _roofline("flash", "mfma", tf, BF16_PEAK_TFLOPS, "TFLOP/s", "flash_fwd_d128",
                              algorithmic_flops_per_launch=flops),
    }
    rec.update(stats)
    if cpu:
        from tests.oracle_lib import Oracle

        orc = Oracle()
        sl = 16  # 16 of the 256 (batch, head) slices at full sequence length
        q = synth.normal_bf16((1, sl, S, D), 4, 0)
        k = synth.normal_bf16((1, sl, S, D), 4, 1)
        v = synth.normal_bf16((1, sl, S, D), 4, 2)
        t = orc.max_threads
        sec = _cpu_time(lambda: orc.sdpa_bf16(q, k, v, scale, causal=True, threads=t))
        rec["cpu_baseline"] = {"value": 0.5 * 4.0 * sl * S * S * D / sec / 1e12, "unit": "TFLOP/s", "cores": t,
                               "kind": "port",
                               "sample": f"{sl} of the 256 (batch, head) slices at S=4096, D=128, causal, one slice per "
                                         f"thread over {t} threads, min of 3 after 1 warm-up"}
    return rec


def bench_flash_options(m, dev, steps, warmup, cpu):
    """The attention of configs[3] with the options of tensor/src/transformer.rs:112-132 inside the fused
    kernel: a key-padding Bool mask [B, 1, 1, S] together with the causal rule, and (second figure) an additive
    bf16 mask [S, S] with a softcap, which makes the kernel visit every key tile."""
    import numpy as np

    from morok_amd import ops, synth

    B, H, S, D = 8, 32, 4096, 128
    n = B * H * S * D
    bq, bk, bv, bo = (dev.buffer(n * 2).ensure_allocated() for _ in range(4))
    for i, b in enumerate((bq, bk, bv)):
        ops.fill_normal(b, n, seed=4, tensor_id=i, bf16=True)
    pad = np.ones((B, S), np.uint8)
    for bi in range(B):
        pad[bi, S - 128 * bi:] = 0            # the last 128 * b keys of batch b are padding
    bpad = m.Buffer.from_numpy(pad)
    badd = dev.buffer(S * S * 2).ensure_allocated()
    ops.fill_normal(badd, S * S, seed=4, tensor_id=9, bf16=True)
    scale = 1.0 / np.sqrt(D)
    steps = max(1, min(steps, 20))
    ms, stats = _launch_stats(m, lambda: ops.flash_attn_fwd_bf16_ex(bq, bk, bv, bo, B, H, S, S, D, scale, True, bpad, 1, (S, 0, 0), 0.0), steps, warmup)
    flops = 0.5 * 4.0 * B * H * S * S * D
    tf = flops / (ms * 1e-3) / 1e12
    rec = {
        "metric": "flash-attn fwd TFLOP/s (causal + Bool key-padding mask)", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "dtype": "bf16",
        "steps": steps,
        "config": {"workload": "causal flash-attention fwd with a Bool key-padding mask [8,1,1,4096], bf16 [8,32,4096,128]"},
        "roofline": _roofline("flash_options", "mfma", tf, BF16_PEAK_TFLOPS, "TFLOP/s", "flash_fwd_ext_d128_bool", algorithmic_flops_per_launch=flops),
    }
    rec.update(stats)
    ms2, _ = _launch_stats(m, lambda: ops.flash_attn_fwd_bf16_ex(bq, bk, bv, bo, B, H, S, S, D, scale, False, badd, 2, (0, 0, S), 30.0), steps, warmup)
    rec["additive_mask_softcap"] = {"ms_per_step": ms2, "value": 4.0 * B * H * S * S * D / (ms2 * 1e-3) / 1e12, "unit": "TFLOP/s",
                                    "kernel": "flash_fwd_ext_d128_add_cap", "workload": "every key tile: additive bf16 mask [4096,4096] + softcap 30"}
    if cpu:
        from tests.oracle_lib import Oracle

        orc = Oracle()
        sl, Sc = 16, 1024
        q, k, v = (synth.normal_bf16((1, sl, Sc, D), 4, i) for i in range(3))
        mask = np.ones((1, 1, 1, Sc), bool)
        mask[..., Sc - 128:] = False
        sec = _cpu_time(lambda: orc.sdpa_bf16_ex(q, k, v, scale, causal=True, mask=mask))
        rec["cpu_baseline"] = {"value": 0.5 * 4.0 * sl * Sc * Sc * D / sec / 1e12, "unit": "TFLOP/s", "cores": orc.max_threads, "kind": "port",
                               "sample": f"{sl} (batch, head) slices at S={Sc}, D=128, causal + key-padding mask (the oracle visits every key), min of 3 after 1 warm-up"}
    return rec


def bench_decoder(m, dev, steps, warmup, cpu):
    """configs[4]: decoder transformer block from the tensor API, bf16, hidden 4096, 32 heads x 128,
    SwiGLU 11008, RMSNorm eps 1e-6, RoPE theta 1e4, batch 4 x seq 2048 prefill, vocab 32000."""
    from morok_amd import decoder, synth, tensor

    B, S, hidden, heads, ffn, vocab = 4, 2048, 4096, 32, 11008, 32000
    T = B * S
    w = decoder.synthetic_weights(hidden, ffn, vocab, seed=5)
    blk = decoder.DecoderBlock(w, B, S, hidden, heads, ffn, eps=1e-6, theta=10000.0)
    tok = tensor.Tensor.from_numpy(synth.randint((T,), 5, 1, vocab))
    plan = blk.forward(tok).prepare()      # schedule + compile once (Tensor::prepare), then execute per step
    steps = max(1, min(steps, 20))
    ms, stats = _launch_stats(m, plan.execute, steps, warmup)
    prof = plan.execute_profiled()
    gemm_ms = sum(t for n, t in prof if n.startswith("gemm_bf16"))
    flash_ms = sum(t for n, t in prof if n.startswith("flash_fwd"))
    flops = 2.0 * T * hidden * (4 * hidden + 3 * ffn) + 0.5 * 4.0 * B * heads * S * S * (hidden // heads)
    tf = flops / (ms * 1e-3) / 1e12
    rec = {
        "metric": "decoder block TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "dtype": "bf16",
        "steps": steps, "tokens_per_s": T / (ms * 1e-3),
        "config": {"workload": "decoder block via tensor API: hidden 4096, 32x128 heads, SwiGLU 11008, batch 4 x seq 2048 "
                               "prefill (configs[4])"},
        "roofline": {"bound": "mfma", "achieved": tf, "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": tf / BF16_PEAK_TFLOPS, "traffic": None,
                     "traffic_source": "per-kernel figures in profiles/" + PROFILE_OF["decoder"],
                     "kernel": f"gemm_bf16_tile256[_residual] ({sum(n.startswith('gemm_bf16') for n, _ in prof)} of the {len(prof)} kernels)",
                     "algorithmic_flops_per_launch": flops},
        "kernels": len(prof), "gemm_ms": gemm_ms, "flash_ms": flash_ms, "other_ms": sum(t for _, t in prof) - gemm_ms - flash_ms,
    }
    rec.update(stats)
    if cpu:
        from tests.oracle_lib import Oracle

        orc = Oracle()
        sb, ss = 1, 512  # one sequence of 512 tokens through the full-width block
        stok = synth.randint((sb * ss,), 5, 1, vocab)
        cos, sin = decoder.rope_tables(ss, hidden // heads)
        t = orc.max_threads
        sec = _cpu_time(lambda: orc.decoder_block_bf16(stok, w, cos, sin, sb, ss, hidden, heads, ffn, 1e-6, threads=t))
        sflops = 2.0 * sb * ss * hidden * (4 * hidden + 3 * ffn) + 0.5 * 4.0 * sb * heads * ss * ss * (hidden // heads)
        rec["cpu_baseline"] = {"value": sflops / sec / 1e12, "unit": "TFLOP/s", "cores": t, "kind": "port",
                               "sample": f"batch {sb} x seq {ss} through the full-width block (same weights), {t} threads, "
                                         "min of 3 after 1 warm-up"}
    return rec


def bench_decoder_decode(m, dev, steps, warmup, cpu):
    """The same block over 16 tokens (16 sequences, one position each), weights held as `nn::Linear` holds them
    ([out, in]): every weight is streamed once per step, so the step is bound by HBM, and the rate counts the
    weights' bytes.  Eight blocks with different weights run in turn so that none is found in the last-level cache."""
    import numpy as np

    from morok_amd import decoder, synth, tensor

    B, S, hidden, heads, ffn, vocab, layers = 16, 1, 4096, 32, 11008, 32000, 8
    plans = []
    for i in range(layers):
        w = decoder.synthetic_weights(hidden, ffn, vocab, seed=20 + i)
        blk = decoder.DecoderBlock(w, B, S, hidden, heads, ffn, eps=1e-6, theta=10000.0, linear_layout=True)
        tok = tensor.Tensor.from_numpy(synth.randint((B * S,), 5, 1, vocab))
        plans.append((blk, blk.forward(tok).prepare()))

    def step():
        for _, p in plans:
            p.execute()

    ms, stats = _launch_stats(m, step, max(1, min(steps, 20)), warmup)
    prof = plans[0][1].execute_profiled()
    weight_bytes = 2 * hidden * (4 * hidden + 3 * ffn)          # per block
    gbs = layers * weight_bytes / (ms * 1e-3) / 1e9
    rec = {"metric": "decoder block decode HBM GB/s", "value": gbs, "unit": "GB/s", "ms_per_step": ms, "dtype": "bf16", **stats,
           "config": {"workload": "decoder block via tensor API over 16 tokens (16 sequences x 1 position), weights [out, in]: "
                                  "hidden 4096, 32x128 heads, SwiGLU 11008; 8 blocks with different weights per step"},
           "blocks_per_step": layers, "us_per_block": ms * 1e3 / layers, "tokens_per_s": B * S * layers / (ms * 1e-3), "kernels": len(prof),
           "gemm_us": 1e3 * sum(t for n, t in prof if n.startswith("gemm_bf16")), "other_us": 1e3 * sum(t for n, t in prof if not n.startswith("gemm_bf16")),
           "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "traffic": None,
                        "traffic_source": "per-kernel figures in profiles/" + PROFILE_OF["decoder_decode"],
                        "kernel": "gemm_nt_rows (4 of the %d kernels)" % len(prof), "algorithmic_bytes_per_launch": weight_bytes}}
    if cpu:
        from tests.oracle_lib import Oracle

        orc = Oracle()
        w = decoder.synthetic_weights(hidden, ffn, vocab, seed=20)
        stok = synth.randint((B * S,), 5, 1, vocab)
        cos, sin = decoder.rope_tables(S, hidden // heads)
        t = orc.max_threads
        sec = _cpu_time(lambda: orc.decoder_block_bf16(stok, w, cos, sin, B, S, hidden, heads, ffn, 1e-6, threads=t))
        rec["cpu_baseline"] = {"value": weight_bytes / sec / 1e9, "unit": "GB/s", "cores": t, "kind": "port",
                               "sample": f"one block over the same 16 tokens, {t} threads, min of 3 after 1 warm-up"}
    return rec


def bench_matmul_f32(m, dev, steps, warmup, cpu):
    """configs[0]: f32 matmul through Tensor::matmul, A[1024x1024] @ B[1024x1024], uniform(-1,1), seed 1
    (plumbing + correctness: lazy graph -> schedule -> render -> hiprtc -> launch)."""
    from morok_amd import synth, tensor

    n = 1024
    a = synth.uniform((n, n), 1, 0)
    b = synth.uniform((n, n), 1, 1)
    ta, tb = tensor.Tensor.from_numpy(a), tensor.Tensor.from_numpy(b)
    c = ta.matmul(tb)
    plan = c.prepare()
    ms, stats = _launch_stats(m, plan.execute, steps, warmup)
    flops = 2.0 * n ** 3
    tf = flops / (ms * 1e-3) / 1e12
    rec = {
        "metric": "f32 matmul TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "dtype": "f32",
        "config": {"workload": "f32 matmul 1024^3 via the lazy tensor API, generated kernel (configs[0])"},
        # a generated kernel of vector-ALU fused multiply-adds (no matrix instructions exist for
        # f32 operands in the vocabulary): priced against the part's published vector fp32 rate
        "roofline": dict(_roofline("matmul_f32", "valu_fp32", tf, 157.3, "TFLOP/s", plan.kernel_name(0)),
                         algorithmic_flops_per_launch=flops),
    }
    rec.update(stats)
    if cpu:
        from tests.oracle_lib import Oracle

        orc = Oracle()
        t = orc.thread_count(n * n * n, n)
        sec = _cpu_time(lambda: orc.matmul_f32(a, b, threads=t))
        got = c.to_numpy()
        ref = orc.matmul_f32(a, b, threads=t)
        rec["max_rel_err_vs_cpu"] = float(np.abs(got - ref).max() / np.abs(ref).max())
        rec["cpu_baseline"] = {"value": flops / sec / 1e12, "unit": "TFLOP/s", "cores": t, "kind": "port",
                               "sample": f"the whole 1024^3 product, {t} threads, min of 3 after 1 warm-up"}
    return rec


def bench_generated_tc(m, dev, steps, warmup, cpu):
    """The bf16 GEMM of configs[2] through the lazy tensor API with the hand-written kernels
    switched off: tensor-core rewrite (WMMA -> MFMA builtin), operands staged through local
    memory, rendered to HIP C and compiled at run time.  Same inputs as the hand-written GEMM."""
    from morok_amd import synth, tensor, uop

    n = 4096
    a = synth.normal_bf16((n, n), 3, 0)
    b = synth.normal_bf16((n, n), 3, 1)
    tensor.set_fusion(False)
    try:
        c = tensor.Tensor.from_numpy(a, uop.BF16).matmul(tensor.Tensor.from_numpy(b, uop.BF16))
        plan = c.prepare()
    finally:
        tensor.set_fusion(True)
    ms, stats = _launch_stats(m, plan.execute, steps, warmup)
    flops = 2.0 * n ** 3
    tf = flops / (ms * 1e-3) / 1e12
    rec = {
        "metric": "generated tensor-core GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": ms, "dtype": "bf16",
        "config": {"workload": "bf16 GEMM M=N=K=4096 via the lazy tensor API, generated tensor-core kernel "
                               "(hand-written kernels off)"},
        "roofline": _roofline("generated_tc", "mfma", tf, BF16_PEAK_TFLOPS, "TFLOP/s", plan.kernel_name(0),
                              algorithmic_flops_per_launch=flops),
    }
    rec.update(stats)
    if cpu:
        rec["cpu_baseline"] = _gemm_cpu_baseline(n, n, n)
    return rec


def bench_mfma_ceiling(m, dev, steps, warmup, cpu):
    """Calibration only: the MFMA-only kernel at the size of the 4096^3 product."""
    tf = _mfma_ceiling_tflops(m, dev)
    smooth = _mfma_ceiling_tflops(m, dev, False)
    return {"metric": "MFMA-only ceiling TFLOP/s", "smooth_operands_value": smooth, "value": tf, "unit": "TFLOP/s", "ms_per_step": 2.0 * 4096 ** 3 / tf / 1e9,
            "dtype": "bf16", "config": {"workload": "calibration: 256 workgroups x 64 K steps of register-only "
                                                    "v_mfma_f32_16x16x32_bf16 (the MFMA stream of the 4096^3 GEMM), hashed operand values"},
            "roofline": {"bound": "mfma", "achieved": tf, "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": tf / BF16_PEAK_TFLOPS, "traffic": 0, "traffic_source": "no memory operands",
                         "kernel": "mfma_ceiling_kernel", "algorithmic_flops_per_launch": 2.0 * 4096 ** 3}}


def bench_group_reduce(m, dev, steps, warmup, cpu):
    """Row sums of f32 [8, 2^24] through the lazy tensor API: few outputs, long rows, i.e. the GROUP
    reduction (waves of a workgroup share an output through local memory) plus a small second
    kernel that folds the per-workgroup partials.  HBM-bound: 512 MiB read per step."""
    from morok_amd import ops, tensor, uop

    rows, cols = 8, 1 << 24
    n = rows * cols
    bx = dev.buffer(n * 4).ensure_allocated()
    ops.fill_normal(bx, n, seed=6, tensor_id=0)
    tensor.set_fusion(False)
    try:
        t = tensor.Tensor.from_buffer(bx, (rows, cols), uop.F32).sum(1)
        plan = t.prepare()
    finally:
        tensor.set_fusion(True)
    names = [plan.kernel_name(i) for i in range(plan.kernel_count)]
    ms, stats = _launch_stats(m, plan.execute, steps, warmup)
    algo_bytes = n * 4 + rows * 4
    gbs = algo_bytes / (ms * 1e-3) / 1e9
    rec = {"metric": "grouped reduce HBM GB/s", "value": gbs, "unit": "GB/s", "ms_per_step": ms, "dtype": "f32", **stats,
           "config": {"workload": "row sums of f32 [8 x 2^24] via the lazy tensor API (generated GROUP reduce + fold)"},
           "kernels": names,
           "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                        "traffic": None, "traffic_source": "profiles/group_reduce_sum_8x16777216_f32.txt", "kernel": names[0],
                        "algorithmic_bytes_per_launch": algo_bytes}}
    if cpu:
        import numpy as np

        x = bx.copyout(np.float32, (rows, cols))
        sec = _cpu_time(lambda: x.sum(axis=1, dtype=np.float32))
        ref = x.astype(np.float64).sum(1)
        rec["max_rel_err_vs_float64"] = float(np.max(np.abs(t.to_numpy() - ref) / np.abs(x.astype(np.float64)).sum(1)))
        rec["cpu_baseline"] = {"value": algo_bytes / sec / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": "the whole [8 x 2^24] matrix, sequential f32 row sums (numpy, one thread), min of 3 "
                                         "after 1 warm-up"}
    return rec


def bench_linear_decode(m, dev, steps, warmup, cpu):
    """One token through eight Linear layers (x [1, 4096] @ W.T, W [12288, 4096] bf16 as `nn::Linear` stores
    it): the streaming kernel for one and two rows.  HBM-bound; the eight weights (96 MiB each) are
    different buffers visited in turn, so no launch finds its weight in the 256 MiB last-level cache.
    A step is the eight launches; the rate counts every byte a launch has to move."""
    return _linear_decode(m, dev, steps, warmup, cpu, 1, "linear_decode", "gemm_nt_skinny<1,2,false>")


def bench_linear_decode_16(m, dev, steps, warmup, cpu):
    """The same with 16 tokens in flight (x [16, 4096]): the streaming kernel for 3 to 64 rows, which feeds the
    matrix pipes from 16-row blocks staged through LDS."""
    return _linear_decode(m, dev, steps, warmup, cpu, 16, "linear_decode_16", "gemm_nt_rows<1,3,8,false>")


def _linear_decode(m, dev, steps, warmup, cpu, M, workload, kernel):
    import numpy as np

    from morok_amd import ops, synth

    layers, N, K = 8, 12288, 4096
    bx = dev.buffer(M * K * 2).ensure_allocated()
    ops.fill_normal(bx, M * K, seed=7, tensor_id=0, bf16=True)
    ws, ys = [], []
    for i in range(layers):
        w = dev.buffer(N * K * 2).ensure_allocated()
        ops.fill_normal(w, N * K, seed=7, tensor_id=1 + i, bf16=True)
        ws.append(w)
        ys.append(dev.buffer(M * N * 2).ensure_allocated())

    def step():
        for w, y in zip(ws, ys):
            ops.gemm_bf16_nt(bx, w, y, M, N, K)

    ms, stats = _launch_stats(m, step, max(1, min(steps, 20)), warmup)
    algo_bytes = 2 * (N * K + M * K + M * N)  # per launch
    gbs = layers * algo_bytes / (ms * 1e-3) / 1e9
    rec = {"metric": "linear decode HBM GB/s", "value": gbs, "unit": "GB/s", "ms_per_step": ms, "dtype": "bf16", **stats,
           "config": {"workload": "%d token%s x 8 Linear layers [12288, 4096] bf16, weights stored [out, in], one streaming launch each" % (M, "" if M == 1 else "s")},
           "launches_per_step": layers, "us_per_launch": ms * 1e3 / layers,
           "roofline": _roofline(workload, "hbm", gbs, HBM_PEAK_GBS, "GB/s", kernel, algorithmic_bytes_per_launch=algo_bytes)}
    if cpu:
        from tests.oracle_lib import Oracle

        orc = Oracle()
        x = bx.copyout(np.uint16, (M, K))
        rows = 2048                                        # a slice of one weight: the oracle's bf16 product, all host threads
        wt = ws[0].copyout(np.uint16, (N, K))[:rows]
        b = np.ascontiguousarray(wt.T)
        sec = _cpu_time(lambda: orc.gemm_bf16(x, b))
        got = synth.from_bf16(ys[0].copyout(np.uint16, (M, N))[:, :rows])
        ref = synth.from_bf16(orc.gemm_bf16(x, b))
        rec["max_rel_err_vs_cpu"] = float(np.abs(got - ref).max() / np.abs(ref).max())
        rec["cpu_baseline"] = {"value": 2 * (rows * K + K + rows) / sec / 1e9, "unit": "GB/s", "cores": orc.thread_count(M * rows * K, M),
                               "kind": "port", "sample": f"{rows} of the 12288 weight rows of one layer, f32-accumulate bf16 product, min of 3 after 1 warm-up"}
    return rec


def bench_flash_decode(m, dev, steps, warmup, cpu):
    """One new token's attention over the key/value caches of 8 layers (a decode step's eight attention calls):
    32 heads, 4096 cached keys, head dim 128, batch 1 (and batch 8 beside it): K and V are streamed once."""
    import numpy as np

    from morok_amd import ops, synth

    layers, H, Sk, D = 8, 32, 4096, 128
    scale = 1.0 / float(np.sqrt(D))

    def run(B):
        n_kv, n_q = B * H * Sk * D, B * H * D
        bq = dev.buffer(n_q * 2).ensure_allocated()
        ops.fill_normal(bq, n_q, seed=11, tensor_id=0, bf16=True)
        ks, vs, os_ = [], [], []
        for i in range(layers):
            k, v = dev.buffer(n_kv * 2).ensure_allocated(), dev.buffer(n_kv * 2).ensure_allocated()
            ops.fill_normal(k, n_kv, seed=11, tensor_id=1 + 2 * i, bf16=True)
            ops.fill_normal(v, n_kv, seed=11, tensor_id=2 + 2 * i, bf16=True)
            ks.append(k), vs.append(v), os_.append(dev.buffer(n_q * 2).ensure_allocated())

        def step():
            for k, v, o in zip(ks, vs, os_):
                ops.flash_attn_fwd_bf16(bq, k, v, o, B, H, 1, Sk, D, scale, False)

        ms, stats = _launch_stats(m, step, max(1, min(steps, 20)), warmup)
        algo = 2 * n_kv * 2 + 2 * n_q * 2  # per launch: K and V once, q and o
        return ms, stats, algo, (bq, ks[0], vs[0], os_[0])

    ms, stats, algo_bytes, (bq, k0, v0, o0) = run(1)
    gbs = layers * algo_bytes / (ms * 1e-3) / 1e9
    rec = {"metric": "attention decode HBM GB/s", "value": gbs, "unit": "GB/s", "ms_per_step": ms, "dtype": "bf16", **stats,
           "config": {"workload": "1 query per head x 8 layers' caches [1, 32, 4096, 128] bf16 (K and V), no causal rule, keys split over workgroups"},
           "launches_per_step": layers, "us_per_launch": ms * 1e3 / layers,
           "roofline": _roofline("flash_decode", "hbm", gbs, HBM_PEAK_GBS, "GB/s", "flash_decode_split<128>", algorithmic_bytes_per_launch=algo_bytes)}
    if cpu:
        from tests.oracle_lib import Oracle

        orc = Oracle()
        q, k, v = bq.copyout(np.uint16, (1, H, 1, D)), k0.copyout(np.uint16, (1, H, Sk, D)), v0.copyout(np.uint16, (1, H, Sk, D))
        sec = _cpu_time(lambda: orc.sdpa_bf16(q, k, v, scale, causal=False))
        got, ref = synth.from_bf16(o0.copyout(np.uint16, (1, H, 1, D))), synth.from_bf16(orc.sdpa_bf16(q, k, v, scale, causal=False))
        rec["max_rel_err_vs_cpu"] = float(np.abs(got - ref).max() / np.abs(ref).max())
        rec["cpu_baseline"] = {"value": algo_bytes / sec / 1e9, "unit": "GB/s", "cores": orc.max_threads, "kind": "port",
                               "sample": "one layer's attention (32 heads x 4096 keys), the oracle's SDPA, min of 3 after 1 warm-up"}
    del bq, k0, v0, o0
    dev.synchronize()
    dev.lru_clear()
    if REFERENCE_LEGS:  # the same step for a batch of 8 sequences (256 pairs: one key range each, one launch)
        ms8, _, algo8, _ = run(8)
        rec["batch_8"] = {"us_per_launch": ms8 * 1e3 / layers, "GB/s": layers * algo8 / (ms8 * 1e-3) / 1e9,
                          "frac": layers * algo8 / (ms8 * 1e-3) / 1e9 / HBM_PEAK_GBS}
        dev.synchronize()
        dev.lru_clear()
        # grouped-query attention: a batch of 16 with 8 key heads and 8 query heads each, K and V with a zero head stride
        # (batch x key heads as batches): one pass over a key head's 4096 keys serves its 8 query heads
        groups, G = 16 * 8, 8
        n_kv, n_q = groups * Sk * D, groups * G * D
        bq, bo = dev.buffer(n_q * 2).ensure_allocated(), dev.buffer(n_q * 2).ensure_allocated()
        ops.fill_normal(bq, n_q, seed=12, tensor_id=0, bf16=True)
        kvs = []
        for i in range(4):
            k, v = dev.buffer(n_kv * 2).ensure_allocated(), dev.buffer(n_kv * 2).ensure_allocated()
            ops.fill_normal(k, n_kv, seed=12, tensor_id=1 + 2 * i, bf16=True)
            ops.fill_normal(v, n_kv, seed=12, tensor_id=2 + 2 * i, bf16=True)
            kvs.append((k, v))
        st = [G * D, D, D, Sk * D, 0, D, Sk * D, 0, D, G * D, D, D]

        def gqa_step():
            for k, v in kvs:
                ops.flash_attn_fwd_bf16_strided(bq, k, v, bo, groups, G, 1, Sk, D, scale, st, (0, 0, 0, 0), False)

        msg, _ = _launch_stats(m, gqa_step, max(1, min(steps, 20)), warmup)
        algo_g = 2 * n_kv * 2 + 2 * n_q * 2
        rec["grouped_query_16x8x8"] = {"us_per_launch": msg * 1e3 / len(kvs), "GB/s": len(kvs) * algo_g / (msg * 1e-3) / 1e9,
                                        "frac": len(kvs) * algo_g / (msg * 1e-3) / 1e9 / HBM_PEAK_GBS}
    return rec


def bench_copy(m, dev, steps, warmup, cpu):
    """Calibration only: 256 MiB streaming copy kernel (known traffic 2 x 256 MiB per launch)."""
    from morok_amd import ops

    nbytes = 256 << 20
    bx = dev.buffer(nbytes).ensure_allocated()
    by = dev.buffer(nbytes).ensure_allocated()
    ops.fill_normal(bx, nbytes // 4, seed=9)
    ms, stats = _launch_stats(m, lambda: ops.copy_kernel(bx, by, nbytes), steps, warmup)
    gbs = 2 * nbytes / (ms * 1e-3) / 1e9
    return {"metric": "copy GB/s", "value": gbs, "unit": "GB/s", "ms_per_step": ms, "dtype": "u8", **stats,
            "config": {"workload": "calibration: 256 MiB streaming copy kernel"},
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": gbs / HBM_PEAK_GBS, "traffic": None, "kernel": "copy_kernel",
                         "algorithmic_bytes_per_launch": 2 * nbytes}}


WORKLOADS = {"softmax": bench_softmax, "gemm": bench_gemm, "flash": bench_flash, "decoder": bench_decoder,
             "matmul_f32": bench_matmul_f32, "generated_tc": bench_generated_tc, "copy": bench_copy, "mfma_ceiling": bench_mfma_ceiling,
             "group_reduce": bench_group_reduce, "gemm_f16": bench_gemm_f16, "flash_options": bench_flash_options,
             "linear_decode": bench_linear_decode, "linear_decode_16": bench_linear_decode_16,
             "decoder_decode": bench_decoder_decode, "flash_decode": bench_flash_decode}
PRIMARY_ORDER = ["gemm", "flash", "softmax", "decoder", "matmul_f32", "generated_tc", "linear_decode", "linear_decode_16", "flash_decode"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all", help="all | " + " | ".join(sorted(WORKLOADS)))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-reference-legs", action="store_true",
                    help="skip the MFMA-only ceiling, the direct C-ABI leg and the vendor reference of the GEMM workload "
                         "(profiler runs: only the measured kernel in the trace)")
    ap.add_argument("--settle-ms", type=float, default=SETTLE_MS,
                    help="untimed launches for this many ms before warm-up (0 for counter-collection runs)")
    args = ap.parse_args()
    globals()["SETTLE_MS"] = args.settle_ms
    globals()["REFERENCE_LEGS"] = not args.no_reference_legs
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
        "dtype": primary["dtype"], "data": "synthetic", "config": primary["config"], "settle_ms": SETTLE_MS,
        "roofline": primary["roofline"],
    }
    cpu_model = _cpu_model()
    for r in recs:
        if "cpu_baseline" in r:
            r["cpu_baseline"]["cpu_model"] = cpu_model
            r["cpu_baseline"]["host_cores"] = os.cpu_count()
    for k in ("median_ms", "min_ms", "plan_item", "direct_abi_ms_per_step", "vendor_reference", "additive_mask_softcap", "batch_8", "grouped_query_16x8x8", "launches_per_step", "us_per_launch"):
        if k in primary:
            line[k] = primary[k]
    if "cpu_baseline" in primary:
        line["cpu_baseline"] = primary["cpu_baseline"]
    if len(recs) > 1:
        line["also"] = recs[1:]
    print(json.dumps(line))


if __name__ == "__main__":
    main()
