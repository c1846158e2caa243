// Fused row softmax, f32, last axis.  One pass over HBM: each row is read once into
// registers, reduced (max, then sum of exp) with wave64 DPP reductions, and written once.
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

// kThreads work-items cooperate on one row; each holds kVec float4 registers of it.
// Requires cols % 4 == 0 and cols <= kThreads * kVec * 4.  blockDim.x = kThreads *
// kRowsPerBlock, one row per group of kThreads.
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
    const int nvec = cols >> 2;
    const f32x4* xr = reinterpret_cast<const f32x4*>(x + (active ? row : 0) * (long)cols);
    f32x4* yr = reinterpret_cast<f32x4*>(y + (active ? row : 0) * (long)cols);

    f32x4 v[kVec];
#pragma unroll
    for (int i = 0; i < kVec; i++) {
        int idx = t + i * kThreads;
        if (active && idx < nvec)
            v[i] = __builtin_nontemporal_load(xr + idx);
        else
            v[i] = f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    }
    float m = -INFINITY;
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
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < kVec; i++) {
        // padded lanes hold -inf: expf(-inf - m) = 0 contributes nothing
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
}

// Any cols: one workgroup per row, three sweeps over the row (the later sweeps hit L2).
__global__ __launch_bounds__(256) void softmax_rows_streaming(const float* __restrict__ x, float* __restrict__ y,
                                                              long rows, long cols) {
    __shared__ float red[2][4];
    const long row = blockIdx.x;
    if (row >= rows) return;
    const float* xr = x + row * cols;
    float* yr = y + row * cols;
    const int t = threadIdx.x;
    float m = -INFINITY;
    for (long c = t; c < cols; c += 256) m = fmaxf(m, xr[c]);
    m = wave_reduce<MaxOp>(m);
    if ((t & 63) == 0) red[0][t / 64] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
    float s = 0.0f;
    for (long c = t; c < cols; c += 256) s += expf(xr[c] - m);
    s = wave_reduce<SumOp>(s);
    if ((t & 63) == 0) red[1][t / 64] = s;
    __syncthreads();
    s = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
    const float inv = 1.0f / s;
    for (long c = t; c < cols; c += 256) yr[c] = expf(xr[c] - m) * inv;
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
    if (rows > 0x7fffffffL) return -1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    (void)hipGetLastError();  // launch status below must be this launch's own
    const float* xi = static_cast<const float*>(x);
    float* yo = static_cast<float*>(y);
    const bool aligned = (cols % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) % 16 == 0);
    if (aligned && cols <= 8192) {
        int c = (int)cols;
        if (variant == 1) {  // one wave per row, 4 rows per workgroup
            if (c <= 256 * 1) launch_regs<64, 1, 4>(s, xi, yo, rows, c);
            else if (c <= 256 * 4) launch_regs<64, 4, 4>(s, xi, yo, rows, c);
            else if (c <= 256 * 8) launch_regs<64, 8, 4>(s, xi, yo, rows, c);
            else if (c <= 256 * 16) launch_regs<64, 16, 4>(s, xi, yo, rows, c);
            else launch_regs<64, 32, 4>(s, xi, yo, rows, c);
        } else {  // default: 256 work-items per row for long rows, one wave for short ones
            if (c <= 256 * 1) launch_regs<64, 1, 4>(s, xi, yo, rows, c);
            else if (c <= 256 * 4) launch_regs<64, 4, 4>(s, xi, yo, rows, c);
            else if (c <= 1024 * 2) launch_regs<256, 2, 1>(s, xi, yo, rows, c);
            else if (c <= 1024 * 4) launch_regs<256, 4, 1>(s, xi, yo, rows, c);
            else launch_regs<256, 8, 1>(s, xi, yo, rows, c);
        }
    } else {
        softmax_rows_streaming<<<(unsigned)rows, 256, 0, s>>>(xi, yo, rows, cols);
    }
    return (int)hipGetLastError();
}

}  // namespace mrk
