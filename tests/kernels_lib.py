"""Linearized kernels, written the way morok's pipeline hands them to a renderer
(post gpudims: GLOBAL/LOCAL ranges are SPECIAL gidx/lidx, reductions are RANGE loops with
DEFINE_REG accumulators or REDUCE nodes, late rewrites applied: a*b+c is MULACC)."""
from morok_amd import uop as U


def elementwise_unary(op, n, dt=U.f32, block=256):
    k = U.Kernel()
    out = k.param(0, dt, n)
    inp = k.param(1, dt, n)
    g = k.special("gidx0", (n + block - 1) // block)
    l = k.special("lidx0", block)
    idx = k.add(k.mul(g, k.const(block)), l)
    gate = k.binary("lt", idx, k.const(n))
    x = k.load(k.index(inp, idx, gate=gate))
    y = k.unary(op, x)
    k.if_(gate)
    k.store(k.index(out, idx), y)
    k.endif()
    return k


def elementwise_binary(op, n, dt=U.f32, block=256, out_dt=None):
    k = U.Kernel()
    out = k.param(0, out_dt or dt, n)
    a = k.param(1, dt, n)
    b = k.param(2, dt, n)
    g = k.special("gidx0", (n + block - 1) // block)
    l = k.special("lidx0", block)
    idx = k.add(k.mul(g, k.const(block)), l)
    gate = k.binary("lt", idx, k.const(n))
    x = k.load(k.index(a, idx, gate=gate))
    # second operand defaults to 1 on masked lanes so that integer division stays defined
    one = k.const(1.0 if dt.is_float else 1, dt)
    y = k.load(k.index(b, idx, gate=gate), alt=one)
    z = k.binary(op, x, y)
    if out_dt is not None and out_dt.scalar != k.dtypes[z].scalar:
        z = k.cast(z, out_dt)
    k.if_(gate)
    k.store(k.index(out, idx), z)
    k.endif()
    return k


def row_reduce(op, rows, cols, use_reduce_node):
    """One work-item per row, sequential loop over the columns (the schedule of softmax's
    max / sum kernels when no GROUP opt applies)."""
    k = U.Kernel()
    out = k.param(0, U.f32, rows)
    inp = k.param(1, U.f32, rows * cols)
    block = 64
    g = k.special("gidx0", (rows + block - 1) // block)
    l = k.special("lidx0", block)
    row = k.add(k.mul(g, k.const(block)), l)
    gate = k.binary("lt", row, k.const(rows))
    base = k.mul(row, k.const(cols))
    if use_reduce_node:
        r = k.range(cols, 0, U.AX_REDUCE)
        x = k.load(k.index(inp, k.add(base, r), gate=gate))
        red = k.reduce(op, x, r)
        k.end(r)
        result = red
    else:  # DEFINE_REG accumulator form (schedule/src/devectorize.rs:1814-1861)
        acc = k.define_reg(0, U.f32, 1)
        zero = k.const(0)
        ident = k.const(float("-inf") if op == "max" else 0.0, U.f32)
        k.store(k.index(acc, zero), ident)
        r = k.range(cols, 0, U.AX_REDUCE)
        x = k.load(k.index(inp, k.add(base, r), gate=gate))
        cur = k.load(k.index(acc, zero))
        nxt = k.binary("max" if op == "max" else "add", cur, x)
        k.store(k.index(acc, zero), nxt)
        k.end(r)
        result = k.load(k.index(acc, zero))
    k.if_(gate)
    k.store(k.index(out, row), result)
    k.endif()
    return k


def softmax_kernels(rows, cols):
    """The reference's three-kernel softmax schedule (tensor/src/test/unit/fusion.rs:83-88):
    max-reduce; exp + sum-reduce; exp + div.  Buffers: (m <- x), (s <- x, m), (y <- x, m, s)."""
    k1 = row_reduce("max", rows, cols, use_reduce_node=True)

    k2 = U.Kernel()
    s_out = k2.param(0, U.f32, rows)
    x_in = k2.param(1, U.f32, rows * cols)
    m_in = k2.param(2, U.f32, rows)
    g = k2.special("gidx0", (rows + 63) // 64)
    l = k2.special("lidx0", 64)
    row = k2.add(k2.mul(g, k2.const(64)), l)
    gate = k2.binary("lt", row, k2.const(rows))
    m = k2.load(k2.index(m_in, row, gate=gate))
    base = k2.mul(row, k2.const(cols))
    r = k2.range(cols, 0, U.AX_REDUCE)
    x = k2.load(k2.index(x_in, k2.add(base, r), gate=gate))
    e = k2.unary("exp", k2.binary("sub", x, m))
    red = k2.reduce("add", e, r)
    k2.end(r)
    k2.if_(gate)
    k2.store(k2.index(s_out, row), red)
    k2.endif()

    k3 = U.Kernel()
    n = rows * cols
    y_out = k3.param(0, U.f32, n)
    x_in = k3.param(1, U.f32, n)
    m_in = k3.param(2, U.f32, rows)
    s_in = k3.param(3, U.f32, rows)
    g = k3.special("gidx0", (n + 255) // 256)
    l = k3.special("lidx0", 256)
    idx = k3.add(k3.mul(g, k3.const(256)), l)
    gate = k3.binary("lt", idx, k3.const(n))
    row = k3.binary("idiv", idx, k3.const(cols))
    x = k3.load(k3.index(x_in, idx, gate=gate))
    m = k3.load(k3.index(m_in, row, gate=gate))
    one = k3.const(1.0, U.f32)
    s = k3.load(k3.index(s_in, row, gate=gate), alt=one)
    y = k3.binary("fdiv", k3.unary("exp", k3.binary("sub", x, m)), s)
    k3.if_(gate)
    k3.store(k3.index(y_out, idx), y)
    k3.endif()
    return k1, k2, k3


def matmul_f32_upcast4x4(M, N, K):
    """f32 matmul as one kernel (fusion.rs:28-33): output tiled LOCAL 16x16, UPCAST 4x4 per
    work-item, K as a REDUCE loop with MULACC into 16 register accumulators, B read and C
    written as float4.  Requires M, N % 64 == 0."""
    assert M % 64 == 0 and N % 64 == 0
    k = U.Kernel()
    c = k.param(0, U.f32, M * N)
    a = k.param(1, U.f32, M * K)
    b = k.param(2, U.f32, K * N)
    gx = k.special("gidx0", N // 64)
    gy = k.special("gidx1", M // 64)
    lx = k.special("lidx0", 16)
    ly = k.special("lidx1", 16)
    col0 = k.add(k.mul(gx, k.const(64)), k.mul(lx, k.const(4)))
    row0 = k.add(k.mul(gy, k.const(64)), k.mul(ly, k.const(4)))
    acc = k.define_reg(0, U.f32, 16)
    zero = k.const(0.0, U.f32)
    for i in range(16):
        k.store(k.index(acc, k.const(i)), zero)
    r = k.range(K, 0, U.AX_REDUCE)
    bvec = k.load(k.index(b, k.add(k.mul(r, k.const(N)), col0)), dt=U.f32.vec(4))
    for i in range(4):
        arow = k.add(row0, k.const(i))
        av = k.load(k.index(a, k.add(k.mul(arow, k.const(K)), r)))
        for j in range(4):
            slot = k.index(acc, k.const(i * 4 + j))
            k.store(slot, k.mulacc(av, k.gep(bvec, j), k.load(slot)))
    k.end(r)
    for i in range(4):
        arow = k.add(row0, k.const(i))
        vals = [k.load(k.index(acc, k.const(i * 4 + j))) for j in range(4)]
        k.store(k.index(c, k.add(k.mul(arow, k.const(N)), col0)), k.vectorize(*vals))
    return k


def wmma_gemm_bf16(M, N, K):
    """bf16 matmul through the WMMA UOp for the CDNA 16x16x32 tensor core
    (schedule/src/optimizer/renderer.rs:549-558: 64 lanes, A and B 8 elements per lane, C 4):
    one wave per 16x16 output tile, f32 accumulate, bf16 result.  M, N % 16 == 0, K % 32 == 0."""
    assert M % 16 == 0 and N % 16 == 0 and K % 32 == 0
    k = U.Kernel()
    c = k.param(0, U.bf16, M * N)
    a = k.param(1, U.bf16, M * K)
    b = k.param(2, U.bf16, K * N)
    gx = k.special("gidx0", N // 16)
    gy = k.special("gidx1", M // 16)
    lane = k.special("lidx0", 64)
    l16 = k.binary("and", lane, k.const(15))
    lg = k.binary("shr", lane, k.const(4))
    row = k.add(k.mul(gy, k.const(16)), l16)  # A operand: lane holds row l%16, k = 8*(l/16)..+8
    col = k.add(k.mul(gx, k.const(16)), l16)  # B operand: lane holds column l%16, same k range
    acc = k.define_reg(0, U.f32.vec(4), 1)
    z = k.const(0.0, U.f32)
    k.store(k.index(acc, k.const(0)), k.vectorize(z, z, z, z))
    r = k.range(K // 32, 0, U.AX_REDUCE)
    kbase = k.add(k.mul(r, k.const(32)), k.mul(lg, k.const(8)))
    avec = k.load(k.index(a, k.add(k.mul(row, k.const(K)), kbase)), dt=U.bf16.vec(8))
    bel = [k.load(k.index(b, k.add(k.mul(k.add(kbase, k.const(e)), k.const(N)), col))) for e in range(8)]
    bvec = k.vectorize(*bel)
    slot = k.index(acc, k.const(0))
    k.store(slot, k.wmma(avec, bvec, k.load(slot), "WMMA_16_16_32_bfloat_float"))
    k.end(r)
    res = k.load(k.index(acc, k.const(0)))
    # accumulator element i of lane l is C[row = 4*(l/16) + i][col = l%16]
    for i in range(4):
        orow = k.add(k.mul(gy, k.const(16)), k.add(k.mul(lg, k.const(4)), k.const(i)))
        k.store(k.index(c, k.add(k.mul(orow, k.const(N)), col)), k.cast(k.gep(res, i), U.bf16))
    return k


def wave_row_sum(rows, cols):
    """Row sums with one wave per row: strided partial sums per lane, then the wave64
    cross-lane reduction (extension op WAVE_REDUCE).  cols % 64 == 0."""
    assert cols % 64 == 0
    k = U.Kernel()
    out = k.param(0, U.f32, rows)
    inp = k.param(1, U.f32, rows * cols)
    g = k.special("gidx0", rows)
    lane = k.special("lidx0", 64)
    base = k.add(k.mul(g, k.const(cols)), lane)
    r = k.range(cols // 64, 0, U.AX_REDUCE)
    x = k.load(k.index(inp, k.add(base, k.mul(r, k.const(64)))))
    part = k.reduce("add", x, r)
    k.end(r)
    total = k.wave_reduce("add", part)
    k.if_(k.binary("eq", lane, k.const(0)))
    k.store(k.index(out, g), total)
    k.endif()
    return k


def async_copy_transposing_load():
    """One wave: a 1 KB ASYNC_COPY of a [16][32] matrix of 16-bit elements into local memory (lane i
    fetches elements 8i .. 8i + 7, which land 16 i bytes into the tile: the identity layout), then
    every group of 16 lanes takes a 4 x 16 block (rows 4g .. 4g + 3, columns 0 .. 15) through
    LOAD_TR and writes its four elements to out[lane][0..3] (extension ops ASYNC_COPY, WAIT_ASYNC,
    LOAD_TR)."""
    k = U.Kernel()
    out = k.param(0, U.bf16, 256)
    inp = k.param(1, U.bf16, 512)
    lane = k.special("lidx0", 64)
    tile = k.define_local(0, U.bf16, 512)
    k.async_copy(k.index(inp, k.mul(lane, k.const(8))), k.index(tile, k.const(0)))
    k.wait_async(0)
    k.barrier()
    i16, g = k.binary("mod", lane, k.const(16)), k.binary("idiv", lane, k.const(16))
    row = k.add(k.mul(g, k.const(4)), k.binary("idiv", i16, k.const(4)))
    at = k.add(k.mul(row, k.const(32)), k.mul(k.binary("mod", i16, k.const(4)), k.const(4)))
    v = k.load_tr(k.index(tile, at))
    k.store(k.index(out, k.mul(lane, k.const(4))), v)
    return k


def local_memory_transpose(n):
    """n x n tile transposed through LDS with a barrier (DEFINE_LOCAL + BARRIER)."""
    k = U.Kernel()
    out = k.param(0, U.f32, n * n)
    inp = k.param(1, U.f32, n * n)
    lx = k.special("lidx0", n)
    ly = k.special("lidx1", n)
    tile = k.define_local(0, U.f32, n * n)
    v = k.load(k.index(inp, k.add(k.mul(ly, k.const(n)), lx)))
    st = k.store(k.index(tile, k.add(k.mul(ly, k.const(n)), lx)), v)
    k.barrier(st)
    t = k.load(k.index(tile, k.add(k.mul(lx, k.const(n)), ly)))
    k.store(k.index(out, k.add(k.mul(ly, k.const(n)), lx)), t)
    return k
