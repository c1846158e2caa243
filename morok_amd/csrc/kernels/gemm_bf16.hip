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

#include <type_traits>

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
    const int a_base_l = (wm * 128 + (lane & 31)) * 128;                                  // + i*4096
    const int b_base_l = (8 * (lane >> 5) + ((lane & 15) >> 2)) * kBPitch +
                         (wn * 128 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;        // + ks*16*pitch + j*64
    int a_xo[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) a_xo[ks] = ((ks * 2 + (lane >> 5)) ^ (lane & 7)) << 4;

    bf16x8 fa[2][4], fb[2][4];
    auto load_frags = [&](int buf, int ks, int slot) {
        const char* sA = sA0 + buf * kAStage + a_base_l + a_xo[ks];
        const char* sB = sB0 + buf * kBStage + b_base_l + ks * 16 * kBPitch;
#pragma unroll
        for (int i = 0; i < 4; i++) fa[slot][i] = *LDS_PTR(bf16x8, sA + i * 4096);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sB + j * 64));
            bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sB + j * 64 + 4 * kBPitch));
            fb[slot][j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
    };
    auto mma = [&](int slot) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[slot][j], fa[slot][i], acc[i][j], 0, 0, 0);
    };
    // LDS writes of this wave are complete and every wave has arrived: the only
    // synchronisation the K loop needs (global loads stay in flight across it).
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // Software pipeline.  While tile kt is consumed from LDS stage `cur`, tile kt+1 sits
    // in registers (loaded one iteration earlier) and is written to the other stage
    // during k-step 0; tile kt+2 is requested from global memory during k-step 1.
    // Fragments are double-buffered in registers: the LDS reads for k-step ks+1 are
    // issued among the MFMAs of k-step ks.  The sched_group_barrier sequences spell out
    // that interleaving (one memory instruction between consecutive MFMAs) so that LDS
    // and global traffic proceed while the matrix pipe is busy.
    const int KT = K / kBK;
    gload(0);
    swrite(0);
    gload(KT > 1 ? 1 : 0);
    lds_barrier();
    load_frags(0, 0, 0);

    // No branches inside an iteration, so that every k-step stays one basic block the
    // scheduler can interleave: near the end of K the prefetches simply re-request the
    // last tile (a cache hit) and fill an LDS stage nobody reads.
    auto iteration = [&](auto cur_c, int kt) {
        constexpr int cur = decltype(cur_c)::value;
        // k-step 0: MFMAs on slot 0 | LDS reads of k-step 1 | LDS writes of tile kt+1
        swrite(cur ^ 1);
        load_frags(cur, 1, 1);
        mma(0);
#pragma unroll
        for (int n = 0; n < 16; n++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
            if (n < 12) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // DS write
        }
        __builtin_amdgcn_sched_barrier(0);
        // k-step 1: MFMAs on slot 1 | LDS reads of k-step 2 | global loads of tile kt+2
        gload(kt + 2 < KT ? kt + 2 : KT - 1);
        load_frags(cur, 2, 0);
        mma(1);
#pragma unroll
        for (int n = 0; n < 16; n++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (n < 12) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 1, 0);  // VALU (address)
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // VMEM read
        }
        __builtin_amdgcn_sched_barrier(0);
        // k-step 2: MFMAs on slot 0 | LDS reads of k-step 3
        load_frags(cur, 3, 1);
        mma(0);
#pragma unroll
        for (int n = 0; n < 16; n++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (n < 12) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        // every wave has finished reading stage `cur` and writing the other stage
        lds_barrier();
        // k-step 3: MFMAs on slot 1 | LDS reads of k-step 0 of the next tile
        load_frags(cur ^ 1, 0, 0);
        mma(1);
#pragma unroll
        for (int n = 0; n < 16; n++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (n < 12) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
        iteration(I0{}, kt);
        iteration(I1{}, kt + 1);
    }
    if (kt < KT) iteration(I0{}, kt);
    lds_barrier();

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
