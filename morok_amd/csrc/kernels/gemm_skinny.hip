// C[M, N] = A[M, K] @ Bt[N, K]^T for a handful of rows (M <= 16) against a weight stored as a Linear
// layer keeps it ([out_features, in_features], tensor/src/nn/linear.rs:9-14,39-41): the decode step
// of a language model.  The product is a stream over the weight: 2 * N * K bytes against 2 * M * N * K
// flops, HBM-bound for these M, so nothing is tiled for the matrix pipes.  A workgroup of four waves
// owns two to eight weight rows; the waves take the 512-element chunks of K in turn, a lane loads
// 16 bytes of each of the rows (a wave reads 1 KB of one row per instruction) and of each row of A
// (cache hits: every workgroup reads the same few KB, each starting at another chunk so that they
// do not all queue on the same L2 channel), and multiplies with packed two-element dot products
// (v_dot2c_f32_bf16 / _f16: exact products, f32 accumulation).  The lanes' partial sums are folded
// with a transposing butterfly (after step s a lane keeps half of the values it held, summed with
// its partner's: V values take V - 1 exchanges in all, not 6 each), the four waves' results meet in
// LDS, wave 0 adds them in a fixed order and writes the outputs.  One launch, no scratch memory, no
// atomics: results do not depend on scheduling.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace mrk::dev {

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

namespace {
constexpr int kChunk = 512;       // elements of K one wave covers per step (64 lanes x 8)

template <bool kF16>
__device__ __forceinline__ float dot2(unsigned a, unsigned b, float c) {
    if constexpr (kF16) return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
    else return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
}

__device__ __forceinline__ unsigned short round_bf16(float f) {
    unsigned u = __builtin_bit_cast(unsigned, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);  // NaN stays NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}
// Transposing butterfly over the 64 lanes: with kCount values left, the lane whose bit kMask is
// clear keeps the lower half and receives its partner's lower half, the other lane the upper
// halves; with one value left the remaining steps are plain exchanges.  Afterwards acc[0] holds
// the sum over all lanes of the value whose index the lane's upper bits spell.
template <int kCount, int kMask>
__device__ __forceinline__ void fold_lanes(float* acc, int lane) {
    if constexpr (kMask >= 1) {
        if constexpr (kCount > 1) {
            constexpr int kHalf = kCount / 2;
            const bool upper = (lane & kMask) != 0;
#pragma unroll
            for (int i = 0; i < kHalf; i++) {
                const float send = upper ? acc[i] : acc[i + kHalf];
                const float keep = upper ? acc[i + kHalf] : acc[i];
                acc[i] = keep + __shfl_xor(send, kMask, 64);
            }
            fold_lanes<kHalf, kMask / 2>(acc, lane);
        } else {
            acc[0] += __shfl_xor(acc[0], kMask, 64);
            fold_lanes<1, kMask / 2>(acc, lane);
        }
    }
}
}  // namespace

// kM: rows of A the kernel holds accumulators for (M <= kM; rows beyond M repeat row M - 1 and are
// not written); kRowsPerGroup: weight rows of a workgroup.  grid = (ceil(N / kRowsPerGroup), batch).
template <int kM, int kRowsPerGroup, bool kF16>
__global__ __launch_bounds__(256) void gemm_nt_skinny(const unsigned short* __restrict__ A, const unsigned short* __restrict__ Bt,
                                                       unsigned short* __restrict__ C, int M, int N, int K) {
    constexpr int kV = kM * kRowsPerGroup;  // values a lane accumulates
    __shared__ float partial[4][kV];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long n0 = (long)blockIdx.x * kRowsPerGroup;
    A += (size_t)blockIdx.y * M * K;
    Bt += (size_t)blockIdx.y * N * K;
    C += (size_t)blockIdx.y * M * N;
    const u32x4* w_row[kRowsPerGroup];
#pragma unroll
    for (int r = 0; r < kRowsPerGroup; r++) {
        const long n = n0 + r < N ? n0 + r : N - 1;  // a row past the end repeats the last one (not written)
        w_row[r] = reinterpret_cast<const u32x4*>(Bt + (size_t)n * K);
    }
    const u32x4* a_row[kM];
#pragma unroll
    for (int m = 0; m < kM; m++) a_row[m] = reinterpret_cast<const u32x4*>(A + (size_t)(m < M ? m : M - 1) * K);

    float acc[kV];
#pragma unroll
    for (int v = 0; v < kV; v++) acc[v] = 0.0f;
    // The waves take the chunks in turn, every workgroup starting at another one: at any moment the
    // workgroups then read different parts of A (rows of A lie a multiple of 4 KB apart for the usual K,
    // i.e. in the same L2 channel, and workgroups in step would all queue on that one channel).
    const int chunks = (K + kChunk - 1) / kChunk;
    const int first = (int)(blockIdx.x % (unsigned)chunks);
    for (int c = wave; c < chunks; c += 4) {
        int cc = c + first;
        if (cc >= chunks) cc -= chunks;
        const int g = cc * 64 + lane;  // 16-byte group of the row
        if (g >= (K >> 3)) continue;
        u32x4 w[kRowsPerGroup], x[kM];
#pragma unroll
        for (int r = 0; r < kRowsPerGroup; r++) w[r] = __builtin_nontemporal_load(w_row[r] + g);
#pragma unroll
        for (int m = 0; m < kM; m++) x[m] = a_row[m][g];
#pragma unroll
        for (int m = 0; m < kM; m++)
#pragma unroll
            for (int r = 0; r < kRowsPerGroup; r++) {
                float s = acc[m * kRowsPerGroup + r];
                s = dot2<kF16>(x[m].x, w[r].x, s);
                s = dot2<kF16>(x[m].y, w[r].y, s);
                s = dot2<kF16>(x[m].z, w[r].z, s);
                s = dot2<kF16>(x[m].w, w[r].w, s);
                acc[m * kRowsPerGroup + r] = s;
            }
    }
    // transposing butterfly (fold_lanes): all 64 lanes' sums, one value left per lane
    fold_lanes<kV, 32>(acc, lane);
    // value index of this lane: bit (5 - s) of the lane chose the half at step s
    int v = 0;
    {
        int c = kV, mask = 32;
        while (c > 1) {
            c >>= 1;
            if (lane & mask) v += c;
            mask >>= 1;
        }
    }
    constexpr int kSteps = kV >= 64 ? 6 : kV == 32 ? 5 : kV == 16 ? 4 : kV == 8 ? 3 : kV == 4 ? 2 : kV == 2 ? 1 : 0;
    static_assert((kV & (kV - 1)) == 0 && kV <= 64, "a power of two of values, one per lane at most");
    const bool owner = (lane & ((1 << (6 - kSteps)) - 1)) == 0;  // one lane of each group that ended up with the same value
    if (owner) partial[wave][v] = acc[0];
    __syncthreads();
    if (wave == 0 && lane < kV) {
        const float s = ((partial[0][lane] + partial[1][lane]) + partial[2][lane]) + partial[3][lane];
        const int m = lane / kRowsPerGroup, r = lane % kRowsPerGroup;
        if (m < M && n0 + r < N) {
            unsigned short out;
            if constexpr (kF16) out = __builtin_bit_cast(unsigned short, (_Float16)s);
            else out = round_bf16(s);
            C[(size_t)m * N + n0 + r] = out;
        }
    }
}

}  // namespace mrk::dev

namespace mrk {

bool gemm_nt_skinny_supported(long M, long N, long K, long batch) {
    return M >= 1 && M <= 16 && N >= 1 && K >= 8 && K % 8 == 0 && K <= 0x7fffffffL && N <= 0x7fffffffL && batch >= 1 && batch <= 65535 &&
           true;
}

int launch_gemm_nt_skinny(void* stream, const void* A, const void* Bt, void* C, long M, long N, long K, long batch, bool f16) {
    using namespace mrk::dev;
    if (!gemm_nt_skinny_supported(M, N, K, batch)) return (int)hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(Bt)) % 16 || reinterpret_cast<uintptr_t>(C) % 2) return (int)hipErrorInvalidValue;
    (void)hipGetLastError();
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned short* a = static_cast<const unsigned short*>(A);
    const unsigned short* b = static_cast<const unsigned short*>(Bt);
    unsigned short* c = static_cast<unsigned short*>(C);
    // more weight rows per workgroup where the accumulators allow it: every workgroup reads all of A,
    // so A's share of the traffic is M / rows
#define MRK_SKINNY(KM, KR)                                                                                  \
    do {                                                                                                    \
        const dim3 grid((unsigned)((N + KR - 1) / KR), (unsigned)batch);                                    \
        if (f16) gemm_nt_skinny<KM, KR, true><<<grid, 256, 0, s>>>(a, b, c, (int)M, (int)N, (int)K);        \
        else gemm_nt_skinny<KM, KR, false><<<grid, 256, 0, s>>>(a, b, c, (int)M, (int)N, (int)K);           \
    } while (0)
    if (M == 1) MRK_SKINNY(1, 2);  // (one row: two weight rows per workgroup stream fastest, 6.2 against 6.0 TB/s with four)
    else if (M == 2) MRK_SKINNY(2, 4);
    else if (M <= 4) MRK_SKINNY(4, 8);
    else if (M <= 8) MRK_SKINNY(8, 8);
    else MRK_SKINNY(16, 4);
#undef MRK_SKINNY
    return (int)hipGetLastError();
}

}  // namespace mrk
