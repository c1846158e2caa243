"""Kernel cache, execution plan, benchmark hook and timeline signal on the GPU
(runtime/src/kernel_cache.rs, runtime/src/execution_plan.rs, runtime/src/benchmark.rs,
device/src/sync.rs)."""
import time

import numpy as np
import pytest

import morok_amd
from morok_amd import MorokHipError, ops, synth
from tests import kernels_lib as KL

pytestmark = pytest.mark.gpu


def test_kernel_cache_dedup(dev):
    morok_amd.kernel_cache_clear()
    k = KL.elementwise_unary("exp", 4096)
    a = morok_amd.Kernel.get_or_compile(k, "E_exp", dev.device_id)
    assert not a.was_cached and morok_amd.kernel_cache_size() == 1
    b = morok_amd.Kernel.get_or_compile(KL.elementwise_unary("exp", 4096), "E_exp", dev.device_id)
    assert b.was_cached and a.same_as(b) and morok_amd.kernel_cache_size() == 1
    c = morok_amd.Kernel.get_or_compile(KL.elementwise_unary("exp", 8192), "E_exp", dev.device_id)
    assert not c.was_cached and not c.same_as(a) and morok_amd.kernel_cache_size() == 2
    assert a.entry_point == "E_exp" and "expf(" in a.code
    f1 = morok_amd.Kernel.builtin("softmax_f32", [8, 256], dev.device_id)
    f2 = morok_amd.Kernel.builtin("softmax_f32", [8, 256], dev.device_id)
    assert f1.same_as(f2)
    morok_amd.kernel_cache_clear()
    assert morok_amd.kernel_cache_size() == 0


def test_plan_three_kernel_softmax_vs_fused(dev, oracle):
    rows, cols = 64, 512
    x = synth.normal((rows, cols), 2, 0, sigma=2.0)
    k1, k2, k3 = (morok_amd.Kernel.get_or_compile(k, n, dev.device_id)
                  for k, n in zip(KL.softmax_kernels(rows, cols), ("r_max", "r_expsum", "E_div")))
    plan = morok_amd.ExecutionPlan(dev.device_id)
    bx = plan.add_buffer(morok_amd.Buffer.from_numpy(x, dev.device_id))
    y_buf, m_buf, s_buf = dev.buffer(x.nbytes), dev.buffer(rows * 4), dev.buffer(rows * 4)
    assert not m_buf.is_allocated()  # intermediates are allocated by build()
    by, bm, bs = plan.add_buffer(y_buf), plan.add_buffer(m_buf), plan.add_buffer(s_buf)
    plan.add_kernel(k1, [bm, bx])
    plan.add_kernel(k2, [bs, bx, bm])
    plan.add_kernel(k3, [by, bx, bm, bs])
    plan.build()
    assert m_buf.is_allocated() and plan.kernel_count == 3
    plan.execute()
    y3 = y_buf.copyout(np.float32, (rows, cols))
    ref = oracle.softmax_f32(x)
    assert (np.abs(y3 - ref) / np.maximum(ref, 1e-30))[ref > 1e-30].max() <= 1e-5

    fused = morok_amd.ExecutionPlan(dev.device_id)
    fx = fused.add_buffer(morok_amd.Buffer.from_numpy(x, dev.device_id))
    yf = dev.buffer(x.nbytes)
    fy = fused.add_buffer(yf)
    fused.add_kernel(morok_amd.Kernel.builtin("softmax_f32", [rows, cols], dev.device_id), [fy, fx])
    fused.build().execute()
    y1 = yf.copyout(np.float32, (rows, cols))
    assert (np.abs(y1 - ref) / np.maximum(ref, 1e-30))[ref > 1e-30].max() <= 1e-5

    prof = plan.execute_profiled()
    assert [p[0] for p in prof] == ["r_max", "r_expsum", "E_div"]
    assert all(p[1] > 0 for p in prof)
    # re-execution is idempotent
    plan.execute()
    assert np.array_equal(y_buf.copyout(np.float32, (rows, cols)), y3)


def test_plan_errors(dev):
    k = morok_amd.Kernel.get_or_compile(KL.elementwise_unary("neg", 256), "E_neg", dev.device_id)
    plan = morok_amd.ExecutionPlan(dev.device_id)
    b = plan.add_buffer(dev.buffer(1024))
    with pytest.raises(MorokHipError):
        plan.add_kernel(k, [b, 7])  # buffer index out of range
    with pytest.raises(MorokHipError):
        plan.add_kernel(k, [b, b], vals=[1])  # kernel takes no variables
    plan.add_kernel(k, [b])  # wrong buffer count surfaces at execute
    with pytest.raises(MorokHipError) as e:
        plan.execute()
    assert "Kernel 0 failed" in e.value.message


def test_execute_with_vars_rebinds_by_name(dev):
    from morok_amd import uop as U

    k = U.Kernel()
    out = k.param(0, U.f32, 1024)
    n = k.define_var("n", U.i32, 0, 1024)
    l = k.special("lidx0", 256)
    g = k.special("gidx0", 4)
    idx = k.add(k.mul(g, k.const(256)), l)
    k.if_(k.binary("lt", idx, n))
    k.store(k.index(out, idx), k.const(1.0, U.f32))
    k.endif()
    kern = morok_amd.Kernel.get_or_compile(k, "fill_n", dev.device_id)
    assert kern.var_names == ["n"]
    plan = morok_amd.ExecutionPlan(dev.device_id)
    ob = dev.buffer(4096, zero_init=True)
    plan.add_kernel(kern, [plan.add_buffer(ob)], vals=[10])
    plan.build().execute()
    assert ob.copyout(np.float32).sum() == 10
    plan.execute_with_vars({"n": 600, "unrelated": 3})
    assert ob.copyout(np.float32).sum() == 600


def test_benchmark_kernel_protocol(dev):
    rows = cols = 2048
    bx = dev.buffer(rows * cols * 4).ensure_allocated()
    by = dev.buffer(rows * cols * 4).ensure_allocated()
    ops.fill_normal(bx, rows * cols, seed=5)
    prog = morok_amd.Program.builtin("softmax_f32", [rows, cols], dev.device_id)
    mn, mean = morok_amd.benchmark_kernel(prog, [by, bx], warmup=1, runs=3, device_id=dev.device_id)
    assert 0 < mn <= mean < 50
    with pytest.raises(MorokHipError):
        morok_amd.benchmark_kernel(prog, [by, bx], runs=0, device_id=dev.device_id)


def test_benchmark_kernel_with_cutoff(dev):
    """runtime/src/benchmark.rs:178-197: a kernel within the cutoff is timed in full, one whose
    first run exceeds three times the cutoff is given up."""
    rows = cols = 4096
    bx = dev.buffer(rows * cols * 4).ensure_allocated()
    by = dev.buffer(rows * cols * 4).ensure_allocated()
    ops.fill_normal(bx, rows * cols, seed=5)
    prog = morok_amd.Program.builtin("softmax_f32", [rows, cols], dev.device_id)
    res = morok_amd.benchmark_kernel_with_cutoff(prog, [by, bx], cutoff_ms=50.0, device_id=dev.device_id)
    assert res is not None and 0 < res[0] <= res[1]
    assert morok_amd.benchmark_kernel_with_cutoff(prog, [by, bx], cutoff_ms=res[0] / 100.0, device_id=dev.device_id) is None
    assert morok_amd.benchmark_kernel_with_cutoff(prog, [by, bx], cutoff_ms=0.0, device_id=dev.device_id) is not None


def test_timeline_signal(dev):
    s = morok_amd.TimelineSignal(dev.device_id)
    assert s.value == 0
    t0 = time.time()
    with pytest.raises(MorokHipError) as e:
        s.wait(1, 20)  # nothing recorded: times out (device/src/sync.rs:363-369)
    assert e.value.code == 12 and "timed out" in e.value.message and time.time() - t0 < 2
    bx = dev.buffer(1 << 24).ensure_allocated()
    by = dev.buffer(1 << 24).ensure_allocated()
    for v in range(1, 25):  # more than the 16 kept events
        ops.copy_kernel(bx, by, 1 << 24, dev.device_id)
        s.set(v)
    s.wait(24, 5000)
    assert s.value == 24 and s.is_reached(10) and not s.is_reached(25)


def test_beam_search_matmul_f32(dev, oracle, tmp_path, monkeypatch):
    """Beam search over LOCAL / UPCAST / UNROLL with event-timed candidates: the winner is a
    valid kernel, computes the right product, is at least as fast as the fixed heuristic, and
    the second search is answered by the disk cache."""
    import morok_amd
    from morok_amd import sched, synth

    monkeypatch.setenv("MOROK_CACHE_DIR", str(tmp_path))
    monkeypatch.delenv("IGNORE_BEAM_CACHE", raising=False)
    n = 512
    opts, best_ms, cached, timed = sched.beam_search_matmul_f32(n, n, n, width=2)
    assert not cached and timed >= 9 and best_ms > 0
    a = synth.uniform((n, n), 1, 0)
    b = synth.uniform((n, n), 1, 1)
    ba, bb, bc = morok_amd.Buffer.from_numpy(a), morok_amd.Buffer.from_numpy(b), dev.buffer(n * n * 4)
    k = morok_amd.Kernel.get_or_compile(sched.build_matmul_f32_opts(n, n, n, opts), "beam_winner")
    plan = morok_amd.ExecutionPlan()
    plan.add_kernel(k, [plan.add_buffer(bc), plan.add_buffer(ba), plan.add_buffer(bb)])
    plan.build().execute()
    got = bc.copyout(np.float32, (n, n))
    ref = oracle.matmul_f32(a, b)
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-4 * np.abs(ref).max())
    base_ms = sched.compile_and_time(sched.build_matmul_f32(n, n, n), [bc, ba, bb], warmup=1, runs=5)
    assert best_ms <= base_ms * 1.15
    opts2, _, cached2, timed2 = sched.beam_search_matmul_f32(n, n, n, width=2)
    assert cached2 and timed2 == 0 and opts2 == opts


def test_tensor_matmul_with_beam(dev, oracle, tmp_path, monkeypatch):
    from morok_amd import synth, tensor

    monkeypatch.setenv("MOROK_CACHE_DIR", str(tmp_path))
    monkeypatch.setenv("MOROK_BEAM", "1")
    a = synth.uniform((256, 192), 7, 0)
    b = synth.uniform((192, 128), 7, 1)
    got = tensor.Tensor.from_numpy(a).matmul(tensor.Tensor.from_numpy(b)).to_numpy()
    np.testing.assert_allclose(got, oracle.matmul_f32(a, b), rtol=1e-4, atol=1e-4)


def test_beam_search_wmma_matmul(dev, tmp_path, monkeypatch):
    """The same search over the LDS-staged tensor-core kernel (waves per workgroup, tiles per
    wave, K steps per barrier pair): the winner computes the bits of the default choice (same
    products, same K order), is no slower than it, and the second search comes from the disk
    cache."""
    import morok_amd
    from morok_amd import sched, synth, uop as U

    monkeypatch.setenv("MOROK_CACHE_DIR", str(tmp_path))
    monkeypatch.delenv("IGNORE_BEAM_CACHE", raising=False)
    M, N, K = 1024, 512, 512
    opts, best_ms, cached, timed = sched.beam_search_wmma_matmul(3, M, N, K, width=2)
    assert not cached and timed >= 12 and best_ms > 0
    a = synth.normal_bf16((M, K), 8, 0)
    b = synth.normal_bf16((K, N), 8, 1)
    ba, bb = morok_amd.Buffer.from_numpy(a), morok_amd.Buffer.from_numpy(b)

    def run(kern, name):
        bc = dev.buffer(M * N * 2)
        k = morok_amd.Kernel.get_or_compile(kern, name)
        plan = morok_amd.ExecutionPlan()
        plan.add_kernel(k, [plan.add_buffer(bc), plan.add_buffer(ba), plan.add_buffer(bb)])
        plan.build().execute()
        return bc, bc.copyout(np.uint16, (M, N))

    bc, got = run(sched.build_wmma_matmul_lds_opts(3, M, N, K, U.BF16, opts), "beam_tc_winner")
    _, want = run(sched.build_wmma_matmul_lds(3, M, N, K, U.BF16), "beam_tc_default")
    assert np.array_equal(got, want)
    ref = synth.from_bf16(a).astype(np.float64) @ synth.from_bf16(b).astype(np.float64)
    assert np.abs(synth.from_bf16(got) - ref).max() <= 2e-2 * np.abs(ref).max()
    base_ms = sched.compile_and_time(sched.build_wmma_matmul_lds(3, M, N, K, U.BF16), [bc, ba, bb], warmup=1, runs=5)
    assert best_ms <= base_ms * 1.15
    opts2, _, cached2, timed2 = sched.beam_search_wmma_matmul(3, M, N, K, width=2)
    assert cached2 and timed2 == 0 and opts2 == opts


def test_copy_and_compute_queues_with_signals(dev):
    """A copy queue feeds a compute queue chunk by chunk; timeline signals order producer and
    consumer on the GPU (hipStreamWaitEvent), the host never waits between chunks.  Each chunk
    is staged through the same two buffers, so a missing dependency would corrupt the result."""
    import morok_amd
    from morok_amd import uop as U

    n, chunks = 1 << 20, 8
    k = U.Kernel()
    out = k.param(0, U.f32, n)
    inp = k.param(1, U.f32, n)
    gx, lx = k.special("gidx0", n // 256), k.special("lidx0", 256)
    i = k.add(k.mul(gx, k.const(256)), lx)
    k.store(k.index(out, i), k.add(k.mul(k.load(k.index(inp, i)), k.const(2.0, U.f32)), k.const(1.0, U.f32)))
    kern = morok_amd.Kernel.get_or_compile(k, "scale_add")
    src = [morok_amd.Buffer.from_numpy(np.full(n, float(c), np.float32)) for c in range(chunks)]
    dst = [dev.buffer(n * 4).ensure_allocated() for _ in range(chunks)]
    stage = [dev.buffer(n * 4).ensure_allocated() for _ in range(2)]
    dev.synchronize()
    copied, consumed = morok_amd.TimelineSignal(), morok_amd.TimelineSignal()
    qc, qx = morok_amd.HardwareQueue(copy_queue=True), morok_amd.HardwareQueue()
    for c in range(chunks):
        if c >= 2:
            qc.wait(consumed, c - 1)          # stage[c % 2] was read by chunk c-2, i.e. consumed value c-1
        qc.copy(stage[c % 2], src[c]).signal(copied, c + 1)
        qx.wait(copied, c + 1).exec(kern, [dst[c], stage[c % 2]]).signal(consumed, c + 1)
    # submit the consumer first: its waits refer to values the producer has not recorded yet
    import threading

    t = threading.Thread(target=lambda: qx.submit(wait_timeout_ms=20000))
    t.start()
    qc.submit(wait_timeout_ms=20000)
    t.join()
    qx.synchronize()
    qc.synchronize()
    consumed.wait(chunks, 5000)
    for c in range(chunks):
        got = dst[c].copyout(np.float32, (n,))
        assert np.all(got == 2.0 * c + 1.0), c


def test_concurrent_realize_from_threads(dev, oracle):
    """Entry points are thread-safe (Renderer / Compiler are Send + Sync upstream, kernels are
    shared through the cache): several host threads build, schedule and run graphs at once."""
    import threading

    from morok_amd import synth, tensor

    errors, results = [], {}

    def work(i):
        try:
            a = synth.uniform((128, 96), 50 + i, 0)
            b = synth.uniform((96, 64), 50 + i, 1)
            for _ in range(5):
                t = tensor.Tensor.from_numpy(a).matmul(tensor.Tensor.from_numpy(b)).try_add(float(i)).softmax(-1)
                results[i] = (t.to_numpy(), a, b)
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i, (got, a, b) in results.items():
        ref = oracle.softmax_f32(oracle.matmul_f32(a, b) + np.float32(i))
        np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-6)


def test_plan_graph_replay_matches_eager(dev, oracle):
    """ExecutionPlan::execute_graph: the recorded graph (kernel launches only: generated
    kernels, GEMMs, flash attention) is replayed several times with the program's own eager work
    and synchronisations in between, on fresh inputs each time; every replay must give exactly
    what the eager launches give."""
    from morok_amd import decoder, tensor

    cfg = dict(batch=2, seq=128, hidden=256, heads=2, ffn=512, vocab=1000)
    T = cfg["batch"] * cfg["seq"]
    w = decoder.synthetic_weights(cfg["hidden"], cfg["ffn"], cfg["vocab"], seed=3)
    blk = decoder.DecoderBlock(w, cfg["batch"], cfg["seq"], cfg["hidden"], cfg["heads"], cfg["ffn"])
    tok_host = synth.randint((T,), 3, 1, cfg["vocab"]).astype(np.int32)
    tok = tensor.Tensor.from_numpy(tok_host)
    out = blk.forward(tok)
    plan = out.prepare()
    tok_buf = tok.buffer()

    def result():
        dev.synchronize()
        return out.buffer().copyout(np.uint16, (T, cfg["hidden"])).copy()

    plan.execute()
    eager = result()
    ref = oracle.decoder_block_bf16(tok_host, w, blk.cos_host, blk.sin_host, cfg["batch"], cfg["seq"], cfg["hidden"],
                                    cfg["heads"], cfg["ffn"], 1e-6)
    err = np.abs(synth.from_bf16(eager) - synth.from_bf16(ref)).max() / np.abs(synth.from_bf16(ref)).max()
    assert err <= 2e-2
    for i in range(4):
        # new tokens, eager result first, then the graph on the same inputs
        toks = synth.randint((T,), 30 + i, 1, cfg["vocab"]).astype(np.int32)
        tok_buf.copyin(toks)
        plan.execute()
        want = result()
        out.buffer().copyin(np.zeros(T * cfg["hidden"], np.uint16))   # the replay must rewrite it
        plan.execute_graph()
        got = result()
        assert np.array_equal(got, want), i
        # unrelated eager work between the replays
        x = synth.normal((64, 512), 5, i, sigma=1.0)
        bx = morok_amd.Buffer.from_numpy(x, dev.device_id)
        by = dev.buffer(x.nbytes)
        ops.softmax_f32(bx, by, 64, 512, dev.device_id)
        dev.synchronize()
    assert not np.array_equal(want, eager)    # the inputs did change between rounds
