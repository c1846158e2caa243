// bf16 GEMM for gfx950: C[M,N] = A[M,K] * B[K,N], row-major bf16 in, f32 accumulate on
// MFMA, one round-to-nearest-even to bf16 at the end.
//
// Stands for the lazy graph of Tensor::matmul on bf16 operands
// (tensor/src/matmul.rs:82-110: broadcast multiply then sum(-1) with the accumulator
// promoted to f32, tensor/src/reduce.rs:101-117, cast back 665-691) after the tensor-core
// rewrite (schedule/src/optimizer/tc.rs:36-94 strips the CAST around the product, so
// exact bf16*bf16 products are accumulated in f32).  The reference names the instruction
// shape in its CDNA table (schedule/src/optimizer/renderer.rs:549-558,724-733); this
// hand-written kernel uses the 32x32x16 shape of the same family for more flops per LDS
// byte.
//
// Main kernel: 256x256 output tile per workgroup of 4 waves (2x2), each wave 128x128 =
// 4x4 MFMA tiles (256 accumulator registers), K step 64.  Global -> registers -> LDS
// with two LDS stages, one barrier per K step.  A is kept in LDS row-major with an XOR
// swizzle of its 16-byte chunks, B row-major (n contiguous) with a 32-byte row skew and
// read through the transposing LDS load, which hands each lane the 4 consecutive-k
// values of its column.  The MFMA is issued with swapped operands (D' = B^T A^T) so each
// lane ends up with 4 consecutive n of one row, which makes the epilogue 8-byte LDS
// writes and 16-byte coalesced global stores.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace mrk::dev {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

constexpr int kBM = 256, kBN = 256, kBK = 64;
constexpr int kAStage = kBM * kBK * 2;         // 32768 B, row pitch 128 B, chunk-swizzled
constexpr int kBPitch = kBN * 2 + 32;          // 544 B: rows skewed by 32 B across banks
constexpr int kBStage = kBK * kBPitch;         // 34816 B
constexpr int kCPitch = 128 * 2 + 16;          // epilogue staging pitch per wave
constexpr int kCWave = 128 * kCPitch;          // 34816 B
constexpr int kSmemMain = 2 * kAStage + 2 * kBStage;  // 135168
constexpr int kSmemEpi = 4 * kCWave;                  // 139264
constexpr int kSmem = kSmemEpi > kSmemMain ? kSmemEpi : kSmemMain;

// Maps the linear workgroup id to an output tile so that the workgroups that land on one
// XCD (ids congruent mod 8 share an L2) cover a compact block of tiles: first regroup
// ids by XCD, then walk tiles in column groups of 4 tile-rows.
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int* tm, int* tn) {
    const int total = tiles_m * tiles_n;
    const int per = total >> 3, rem = total & 7;
    const int xcd = bid & 7, idx = bid >> 3;
    int id = xcd * per + (xcd < rem ? xcd : rem) + idx;
    if (total < 8) id = bid;
    constexpr int kGroup = 4;
    const int group_sz = kGroup * tiles_n;
    const int g = id / group_sz;
    const int first_m = g * kGroup;
    const int gm = (tiles_m - first_m) < kGroup ? (tiles_m - first_m) : kGroup;
    const int in = id - g * group_sz;
    *tm = first_m + in % gm;
    *tn = in / gm;
}

__global__ __launch_bounds__(256) void gemm_bf16_tile256(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                         __bf16* __restrict__ C, int M, int N, int K, int tiles_m,
                                                         int tiles_n) {
    __shared__ __attribute__((aligned(16))) char smem[kSmem];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    int tile_m, tile_n;
    tile_of_block(blockIdx.x, tiles_m, tiles_n, &tile_m, &tile_n);
    const size_t m0 = (size_t)tile_m * kBM, n0 = (size_t)tile_n * kBN;
    const __bf16* Ag = A + m0 * K;
    const __bf16* Bg = B + n0;
    char* sA0 = smem;
    char* sB0 = smem + 2 * kAStage;

    u32x4 ra[8], rb[8];
    // per-thread chunk coordinates (fixed over the K loop)
    // A: 2048 chunks of 16 B per stage, chunk c = i*256 + tid -> row c>>3, k-chunk c&7
    // B: 2048 chunks, c -> k row c>>5, n-chunk c&31
    auto gload = [&](int kt) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int c = i * 256 + tid;
            ra[i] = *reinterpret_cast<const u32x4*>(Ag + (size_t)(c >> 3) * K + (size_t)kt * kBK + (c & 7) * 8);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int c = i * 256 + tid;
            rb[i] = *reinterpret_cast<const u32x4*>(Bg + ((size_t)kt * kBK + (c >> 5)) * N + (c & 31) * 8);
        }
    };
    auto swrite = [&](int buf) {
        char* sA = sA0 + buf * kAStage;
        char* sB = sB0 + buf * kBStage;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int c = i * 256 + tid;
            const int row = c >> 3, kc = c & 7;
            *LDS_PTR(u32x4, sA + row * 128 + ((kc ^ (row & 7)) << 4)) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int c = i * 256 + tid;
            *LDS_PTR(u32x4, sB + (c >> 5) * kBPitch + ((c & 31) << 4)) = rb[i];
        }
    };

    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // lane-constant parts of the fragment addresses
    const int a_row_l = wm * 128 + (lane & 31);  // + i*32
    const int a_kch_l = lane >> 5;               // + ks*2
    const int b_krow_l = 8 * (lane >> 5) + ((lane & 15) >> 2);                    // + ks*16 + 4*r
    const int b_ncol_l = wn * 128 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);      // + j*32

    const int KT = K / kBK;
    gload(0);
    swrite(0);
    __syncthreads();
    int cur = 0;
    for (int kt = 0; kt < KT; kt++) {
        if (kt + 1 < KT) gload(kt + 1);
        const char* sA = sA0 + cur * kAStage;
        const char* sB = sB0 + cur * kBStage;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            bf16x8 af[4], bfr[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = a_row_l + i * 32;
                const int kch = ks * 2 + a_kch_l;
                af[i] = *LDS_PTR(bf16x8, sA + row * 128 + ((kch ^ (row & 7)) << 4));
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int off = (ks * 16 + b_krow_l) * kBPitch + (b_ncol_l + j * 32) * 2;
                bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sB + off));
                bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sB + off + 4 * kBPitch));
                bfr[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[j], af[i], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < KT) swrite(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }

    // Epilogue.  With swapped operands lane l of tile (i, j) holds, in registers 4g..4g+3,
    // C[m = i*32 + l%32][n = j*32 + 8g + 4*(l/32) + 0..3].
    char* sC = smem + wave * kCWave;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                f32x4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                bf16x4 h = __builtin_convertvector(v, bf16x4);
                const int ml = i * 32 + (lane & 31);
                const int nl = j * 32 + 8 * g + 4 * (lane >> 5);
                *LDS_PTR(bf16x4, sC + ml * kCPitch + nl * 2) = h;
            }
    __syncthreads();
    __bf16* Cg = C + (m0 + wm * 128) * N + n0 + wn * 128;
#pragma unroll 4
    for (int it = 0; it < 32; it++) {
        const int r = it * 4 + (lane >> 4);
        const int ch = lane & 15;
        u32x4 v = *LDS_PTR(u32x4, sC + r * kCPitch + ch * 16);
        *reinterpret_cast<u32x4*>(Cg + (size_t)r * N + ch * 8) = v;
    }
}

// Any shape: one wave per 32x32 output tile, operands fetched straight from global memory
// with bounds checks (zero fill), no LDS.  Correct for every M, N, K; used when the shape
// does not fit the tiled kernel.
__global__ __launch_bounds__(256) void gemm_bf16_generic(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                         __bf16* __restrict__ C, int M, int N, int K, int tiles_n,
                                                         long total_tiles) {
    const int lane = threadIdx.x & 63;
    const long tile = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tile >= total_tiles) return;
    const long m0 = (tile / tiles_n) * 32, n0 = (tile % tiles_n) * 32;
    const long m = m0 + (lane & 31), n = n0 + (lane & 31);
    const int kg = 8 * (lane >> 5);
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.0f;
    for (int k0 = 0; k0 < K; k0 += 16) {
        bf16x8 a, b;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int k = k0 + kg + e;
            a[e] = (m < M && k < K) ? A[m * K + k] : (__bf16)0.0f;
            b[e] = (n < N && k < K) ? B[(long)k * N + n] : (__bf16)0.0f;
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
    }
    // lane l register e: row 8*(e/4) + 4*(l/32) + e%4, column l%32
#pragma unroll
    for (int e = 0; e < 16; e++) {
        const long r = m0 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
        if (r < M && n < N) C[r * N + n] = (__bf16)acc[e];
    }
}

}  // namespace mrk::dev

namespace mrk {

int launch_gemm_bf16(void* stream, const void* A, const void* B, void* C, long M, long N, long K, int variant) {
    using namespace mrk::dev;
    if (M <= 0 || N <= 0) return 0;
    if (M > 0x7fffffffL || N > 0x7fffffffL || K > 0x7fffffffL || K < 0) return (int)hipErrorInvalidValue;
    hipStream_t s = static_cast<hipStream_t>(stream);
    (void)hipGetLastError();
    const bool aligned = ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(C)) % 16) == 0;
    if (variant != 2 && aligned && K > 0 && M % kBM == 0 && N % kBN == 0 && K % kBK == 0) {
        const int tm = (int)(M / kBM), tn = (int)(N / kBN);
        gemm_bf16_tile256<<<tm * tn, 256, 0, s>>>(static_cast<const __bf16*>(A), static_cast<const __bf16*>(B),
                                                  static_cast<__bf16*>(C), (int)M, (int)N, (int)K, tm, tn);
    } else {
        const long tm = (M + 31) / 32, tn = (N + 31) / 32;
        const long total = tm * tn;
        const long blocks = (total + 3) / 4;
        if (blocks > 0x7fffffffL) return (int)hipErrorInvalidValue;
        gemm_bf16_generic<<<(unsigned)blocks, 256, 0, s>>>(static_cast<const __bf16*>(A), static_cast<const __bf16*>(B),
                                                           static_cast<__bf16*>(C), (int)M, (int)N, (int)K, (int)tn,
                                                           total);
    }
    return (int)hipGetLastError();
}

}  // namespace mrk
