// Fused row softmax, f32, last axis.  One pass over HBM for rows of up to 65536 columns: each
// row is read once into registers, reduced (max, then sum of exp) with wave64 DPP reductions,
// and written once; longer rows take a two-sweep kernel.  Rows need no particular alignment.
// The reference schedules the same lazy graph (tensor/src/activation.rs:90-101) as three
// kernels that move the matrix through memory three times
// (tensor/src/test/unit/fusion.rs:83-88); fusing them is what makes the op HBM-bound at
// its algorithmic 2 * rows * cols * 4 bytes.
//
// Numerics: m = max(x); e = expf(x - m) (correctly rounded-to-1ulp device expf, no
// fast-math); s = sum(e); y = e * (1/s).  The CPU backend divides by s; multiplying by the
// reciprocal differs by at most 1 ulp, far inside the 1e-5 elementwise tolerance.
#include <hip/hip_runtime.h>

#include "kernels.h"
#include "wave.h"

namespace mrk::dev {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// How a row splits into an unaligned head (0..3 floats up to the first 16-byte boundary), a
// body of float4 and a tail (0..3 floats).  x and y rows must be misaligned alike, which holds
// when both base pointers are 16-byte aligned (the host checks it).
struct RowSplit {
    int head, nvec, tail;
};
__device__ __forceinline__ RowSplit split_row(const float* xr, long cols) {
    RowSplit r;
    const int mis = (int)((reinterpret_cast<uintptr_t>(xr) >> 2) & 3);
    const int h = (4 - mis) & 3;
    r.head = cols < h ? (int)cols : h;
    r.nvec = (int)((cols - r.head) >> 2);
    r.tail = (int)(cols - r.head - 4L * r.nvec);
    return r;
}

// kThreads work-items cooperate on one row; each holds kVec float4 registers of its body (plus
// at most one head and one tail element).  Requires cols <= kThreads * kVec * 4.  blockDim.x =
// kThreads * kRowsPerBlock, one row per group of kThreads.
template <int kThreads, int kVec, int kRowsPerBlock>
__global__ __launch_bounds__(kThreads* kRowsPerBlock) void softmax_rows_in_regs(const float* __restrict__ x,
                                                                                  float* __restrict__ y, long rows,
                                                                                  int cols) {
    constexpr int kWaves = kThreads / 64;
    __shared__ float red[kRowsPerBlock][2][kWaves > 1 ? kWaves : 1];
    const int sub = threadIdx.x / kThreads;  // which row of this block
    const int t = threadIdx.x % kThreads;
    const long row = (long)blockIdx.x * kRowsPerBlock + sub;
    const bool active = row < rows;
    const float* xrow = x + (active ? row : 0) * (long)cols;
    float* yrow = y + (active ? row : 0) * (long)cols;
    const RowSplit sp = split_row(xrow, cols);
    const int nvec = sp.nvec;
    const f32x4* xr = reinterpret_cast<const f32x4*>(xrow + sp.head);
    f32x4* yr = reinterpret_cast<f32x4*>(yrow + sp.head);
    const float* xtail = xrow + sp.head + 4L * nvec;
    float* ytail = yrow + sp.head + 4L * nvec;

    f32x4 v[kVec];
#pragma unroll
    for (int i = 0; i < kVec; i++) {
        int idx = t + i * kThreads;
        if (active && idx < nvec)
            v[i] = __builtin_nontemporal_load(xr + idx);
        else
            v[i] = f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    }
    float eh = (active && t < sp.head) ? xrow[t] : -INFINITY;
    float et = (active && t < sp.tail) ? xtail[t] : -INFINITY;
    float m = fmaxf(eh, et);
#pragma unroll
    for (int i = 0; i < kVec; i++) m = fmaxf(m, fmaxf(fmaxf(v[i].x, v[i].y), fmaxf(v[i].z, v[i].w)));
    m = wave_reduce<MaxOp>(m);
    if constexpr (kWaves > 1) {
        const int w = t / 64;
        if ((t & 63) == 0) red[sub][0][w] = m;
        __syncthreads();
        m = red[sub][0][0];
#pragma unroll
        for (int i = 1; i < kWaves; i++) m = fmaxf(m, red[sub][0][i]);
    }
    // padded lanes hold -inf: expf(-inf - m) = 0 contributes nothing
    eh = expf(eh - m);
    et = expf(et - m);
    float s = eh + et;
#pragma unroll
    for (int i = 0; i < kVec; i++) {
        v[i].x = expf(v[i].x - m);
        v[i].y = expf(v[i].y - m);
        v[i].z = expf(v[i].z - m);
        v[i].w = expf(v[i].w - m);
        s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    }
    s = wave_reduce<SumOp>(s);
    if constexpr (kWaves > 1) {
        const int w = t / 64;
        if ((t & 63) == 0) red[sub][1][w] = s;
        __syncthreads();
        s = red[sub][1][0];
#pragma unroll
        for (int i = 1; i < kWaves; i++) s += red[sub][1][i];
    }
    const float inv = 1.0f / s;
#pragma unroll
    for (int i = 0; i < kVec; i++) {
        int idx = t + i * kThreads;
        if (active && idx < nvec) __builtin_nontemporal_store(v[i] * inv, yr + idx);
    }
    if (active && t < sp.head) yrow[t] = eh * inv;
    if (active && t < sp.tail) ytail[t] = et * inv;
}

// Rows too long for registers: one workgroup of 1024 per row, two sweeps.  The first keeps a
// running maximum and a sum relative to it per work-item (one rescale of the sum per float4
// instead of a sweep of its own for the maximum), the second re-reads the row (from L2 or the
// memory-side cache when it fits) and writes the result: 3 x the row through memory instead
// of the 2 x of the in-register kernel.
__device__ __forceinline__ void online_add4(float& m, float& s, f32x4 v) {
    const float mx = fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w));
    const float mn = fmaxf(m, mx);
    const float ref = mn == -INFINITY ? 0.0f : mn;  // all -inf so far: every term below is 0
    s = s * expf(m - ref) + ((expf(v.x - ref) + expf(v.y - ref)) + (expf(v.z - ref) + expf(v.w - ref)));
    m = mn;
}
__global__ __launch_bounds__(1024) void softmax_rows_streaming(const float* __restrict__ x, float* __restrict__ y,
                                                               long rows, long cols) {
    constexpr int kThreads = 1024, kWaves = kThreads / 64;
    __shared__ float red[2][kWaves];
    const long row = blockIdx.x;
    if (row >= rows) return;
    const float* xrow = x + row * cols;
    float* yrow = y + row * cols;
    const int t = threadIdx.x;
    // rows misaligned differently in x and y (bases not both 16-byte aligned): all scalar
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(xrow) ^ reinterpret_cast<uintptr_t>(yrow)) & 15) == 0;
    RowSplit sp = split_row(xrow, cols);
    if (!vec_ok) sp = RowSplit{0, 0, 0};
    const long scalar_from = sp.head + 4L * sp.nvec;  // [scalar_from, cols) is handled element-wise
    const f32x4* xv = reinterpret_cast<const f32x4*>(xrow + sp.head);
    f32x4* yv = reinterpret_cast<f32x4*>(yrow + sp.head);
    const f32x4 ninf = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};

    float m = -INFINITY, s = 0.0f;
    for (int i = t; i < sp.nvec; i += kThreads) online_add4(m, s, xv[i]);
    {
        f32x4 e = ninf;
        if (t < sp.head) e.x = xrow[t];
        long c = scalar_from + t;
        if (c < cols) e.y = xrow[c];
        online_add4(m, s, e);
        for (c += kThreads; c < cols; c += kThreads) {
            e = ninf;
            e.x = xrow[c];
            online_add4(m, s, e);
        }
    }
    // combine the (maximum, sum) pairs: first the maxima, then the sums rescaled to the common one
    float M = wave_reduce<MaxOp>(m);
    if ((t & 63) == 0) red[0][t / 64] = M;
    __syncthreads();
    M = red[0][0];
#pragma unroll
    for (int i = 1; i < kWaves; i++) M = fmaxf(M, red[0][i]);
    const float Mref = M == -INFINITY ? 0.0f : M;
    float S = wave_reduce<SumOp>(s * expf(m - Mref));
    if ((t & 63) == 0) red[1][t / 64] = S;
    __syncthreads();
    S = red[1][0];
#pragma unroll
    for (int i = 1; i < kWaves; i++) S += red[1][i];
    const float inv = 1.0f / S;

    for (int i = t; i < sp.nvec; i += kThreads) {
        f32x4 v = xv[i];
        v.x = expf(v.x - M) * inv;
        v.y = expf(v.y - M) * inv;
        v.z = expf(v.z - M) * inv;
        v.w = expf(v.w - M) * inv;
        __builtin_nontemporal_store(v, yv + i);
    }
    if (t < sp.head) yrow[t] = expf(xrow[t] - M) * inv;
    for (long c = scalar_from + t; c < cols; c += kThreads) yrow[c] = expf(xrow[c] - M) * inv;
}

template <int kThreads, int kVec, int kRowsPerBlock>
static void launch_regs(hipStream_t s, const float* x, float* y, long rows, int cols) {
    unsigned grid = (unsigned)((rows + kRowsPerBlock - 1) / kRowsPerBlock);
    softmax_rows_in_regs<kThreads, kVec, kRowsPerBlock><<<grid, kThreads * kRowsPerBlock, 0, s>>>(x, y, rows, cols);
}

}  // namespace mrk::dev

namespace mrk {

int launch_softmax_f32(void* stream, const void* x, void* y, long rows, long cols, int variant) {
    using namespace mrk::dev;
    if (rows <= 0 || cols <= 0) return 0;
    if (rows > 0x7fffffffL || cols > 0x7fffffffL) return (int)hipErrorInvalidValue;  // grid extent, 32-bit row split
    hipStream_t s = static_cast<hipStream_t>(stream);
    (void)hipGetLastError();  // launch status below must be this launch's own
    const float* xi = static_cast<const float*>(x);
    float* yo = static_cast<float*>(y);
    // rows of x and y start equally far from a 16-byte boundary when both bases are aligned
    const bool aligned = (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) % 16 == 0;
    // the float4 body of a row has at most cols / 4 elements; up to 3 + 3 floats go to head and tail
    if (aligned && cols <= 65536) {
        int c = (int)cols;
        if (variant == 1 && c <= 8192) {  // one wave per row, 4 rows per workgroup
            if (c <= 256 * 1) launch_regs<64, 1, 4>(s, xi, yo, rows, c);
            else if (c <= 256 * 4) launch_regs<64, 4, 4>(s, xi, yo, rows, c);
            else if (c <= 256 * 8) launch_regs<64, 8, 4>(s, xi, yo, rows, c);
            else if (c <= 256 * 16) launch_regs<64, 16, 4>(s, xi, yo, rows, c);
            else launch_regs<64, 32, 4>(s, xi, yo, rows, c);
        } else {  // default: one wave for short rows, 256 to 1024 work-items per row for long ones
            if (c <= 256 * 1) launch_regs<64, 1, 4>(s, xi, yo, rows, c);
            else if (c <= 256 * 4) launch_regs<64, 4, 4>(s, xi, yo, rows, c);
            else if (c <= 1024 * 2) launch_regs<256, 2, 1>(s, xi, yo, rows, c);
            else if (c <= 1024 * 4) launch_regs<256, 4, 1>(s, xi, yo, rows, c);
            else if (c <= 1024 * 8) launch_regs<256, 8, 1>(s, xi, yo, rows, c);
            else if (c <= 1024 * 16) launch_regs<512, 8, 1>(s, xi, yo, rows, c);
            else if (c <= 1024 * 32) launch_regs<1024, 8, 1>(s, xi, yo, rows, c);
            else launch_regs<1024, 16, 1>(s, xi, yo, rows, c);
        }
    } else {
        softmax_rows_streaming<<<(unsigned)rows, 1024, 0, s>>>(xi, yo, rows, cols);
    }
    return (int)hipGetLastError();
}

}  // namespace mrk
