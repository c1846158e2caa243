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
// 4x4 MFMA tiles (256 accumulator registers), K step 64.  Tiles travel global -> LDS
// directly (global_load_lds, 16 B per lane, no register staging) into two LDS stages,
// one barrier per K step; the copy of tile kt+2 is issued among the MFMAs of the last
// k-step of tile kt, a full tile of work ahead of its first use.  A is kept in LDS
// row-major with an XOR swizzle of its 16-byte chunks, B row-major (n contiguous) with
// an XOR swizzle of its 32-byte granules and read through the transposing LDS load,
// which hands each lane the 4 consecutive-k values of its column.  Fragments are
// double-buffered in registers so LDS reads of k-step ks+1 run under the MFMAs of ks.  The MFMA is issued with swapped operands (D' = B^T A^T) so each
// lane ends up with 4 consecutive n of one row, which makes the epilogue 8-byte LDS
// writes and 16-byte coalesced global stores.
#include <hip/hip_runtime.h>

#include <cstdint>
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
constexpr int kBStageSw = kBK * kBN * 2;       // 32768 B, row pitch 512 B, granule-swizzled
constexpr int kCPitch = 128 * 2 + 16;          // epilogue staging pitch per wave
constexpr int kCWave = 128 * kCPitch;          // 34816 B
constexpr int kSmemMain = 2 * kAStage + 2 * kBStageSw;  // 131072
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
    // two stages; A stage: 256 rows x 128 B, 16 B chunks XOR-swizzled by ((row >> 1) & 7);
    // B stage: 64 k-rows x 512 B, 32 B granules XOR-swizzled by (k & 3).
    __shared__ __attribute__((aligned(1024))) char smem[kSmem];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    int tile_m, tile_n;
    tile_of_block(blockIdx.x, tiles_m, tiles_n, &tile_m, &tile_n);
    const size_t m0 = (size_t)tile_m * kBM, n0 = (size_t)tile_n * kBN;
    char* sA0 = smem;
    char* sB0 = smem + 2 * kAStage;

    // ---- direct global -> LDS copies: each wave moves 8 KB of A and 8 KB of B per tile,
    // one instruction = 64 lanes x 16 B = 1 KB of contiguous LDS.
    // A chunk q (1 KB = 8 rows): lane -> row q*8 + lane/8, LDS chunk lane%8 holds logical
    // chunk (lane%8) ^ ((row >> 1) & 7).  The LDS serves 16 lanes x 16 B per cycle over 64
    // banks; with 128 B rows this swizzle puts 16 consecutive rows of one logical chunk
    // into 16 different 16 B slots.
    // (two variants: (row >> 1) & 7 depends on the parity of q)
    const unsigned a_voff0 = (unsigned)(((size_t)(wave * 64 + (lane >> 3)) * K + (((lane & 7) ^ (lane >> 4)) << 3)) * 2);
    const unsigned a_voff1 = (unsigned)(((size_t)(wave * 64 + (lane >> 3)) * K + (((lane & 7) ^ (4 + (lane >> 4))) << 3)) * 2);
    // B chunk q (1 KB = 2 k-rows): lane -> k-row q*2 + lane/32, LDS 16 B chunk lane%32 ->
    // granule (lane%32)/2 ^ (krow & 3).
    const int b_h = lane & 1, b_g = (lane & 31) >> 1, b_r = lane >> 5;
    const unsigned b_voff0 = (unsigned)(((size_t)(wave * 16 + b_r) * N + ((((b_g ^ (0 + b_r)) << 1) | b_h) << 3)) * 2);
    const unsigned b_voff1 = (unsigned)(((size_t)(wave * 16 + b_r) * N + ((((b_g ^ (2 + b_r)) << 1) | b_h) << 3)) * 2);
    const char* a_tile = reinterpret_cast<const char*>(A + m0 * K);
    const char* b_tile = reinterpret_cast<const char*>(B + n0);
    const unsigned lds_a = (unsigned)(uintptr_t)LDS_PTR(char, sA0) + wave * 8192;
    const unsigned lds_b = (unsigned)(uintptr_t)LDS_PTR(char, sB0) + wave * 8192;
    // One direct copy: 64 lanes x 16 B land at LDS [m0, m0 + 1 KB); the compiler is not told
    // about it (it would otherwise wait for the copy before every later LDS read), so the
    // waits are explicit: tile_barrier() drains vmcnt before the tile is consumed.
    auto dma = [&](unsigned lds_addr, unsigned voff, const char* sbase) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(sbase)
                     : "m0");
    };
    // n = 0..7: A chunks, n = 8..15: B chunks of tile kt into `stage`
    auto dma_one = [&](int n, int kt, int stage) {
        if (n < 8) {
            dma(lds_a + stage * kAStage + n * 1024, (n & 1) ? a_voff1 : a_voff0, a_tile + ((size_t)kt * kBK + (size_t)n * 8 * K) * 2);
        } else {
            const int q = n - 8;
            dma(lds_b + stage * kBStageSw + q * 1024, (q & 1) ? b_voff1 : b_voff0,
                b_tile + ((size_t)kt * kBK + q * 2) * N * 2);
        }
    };
    auto dma_tile = [&](int kt, int stage) {
#pragma unroll
        for (int n = 0; n < 16; n++) dma_one(n, kt, stage);
    };

    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // lane-constant parts of the fragment addresses
    const int a_base_l = (wm * 128 + (lane & 31)) * 128;  // + i*4096
    int a_xo[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) a_xo[ks] = ((ks * 2 + (lane >> 5)) ^ ((lane >> 1) & 7)) << 4;
    const int b_rr = (lane & 15) >> 2;
    const int b_g0 = wn * 8 + ((lane >> 4) & 1);
    const int b_row_l = (8 * (lane >> 5) + b_rr) * 512 + 8 * (lane & 3);  // + ks*16*512 + r*4*512
    const int b_p0 = b_row_l + ((b_g0 ^ b_rr) << 5);                      // j = 0 (+128: j = 2)
    const int b_p1 = b_row_l + (((b_g0 ^ b_rr) ^ 2) << 5);                // j = 1 (+128: j = 3)

    bf16x8 fa[2][4], fb[2][4];
    auto load_frags = [&](int buf, int ks, int slot) {
        const char* sA = sA0 + buf * kAStage + a_base_l + a_xo[ks];
        const char* sB = sB0 + buf * kBStageSw + ks * 16 * 512;
#pragma unroll
        for (int i = 0; i < 4; i++) fa[slot][i] = *LDS_PTR(bf16x8, sA + i * 4096);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int off = ((j & 1) ? b_p1 : b_p0) + (j >> 1) * 128;
            bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sB + off));
            bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sB + off + 4 * 512));
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
    // this wave's LDS reads and its direct-to-LDS copies are complete, then all waves meet
    auto tile_barrier = [&]() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    const int KT = K / kBK;
    dma_tile(0, 0);
    dma_tile(KT > 1 ? 1 : 0, 1);
    tile_barrier();
    load_frags(0, 0, 0);

    auto iteration = [&](auto cur_c, int kt) {
        constexpr int cur = decltype(cur_c)::value;
        load_frags(cur, 1, 1);
        mma(0);
#pragma unroll
        for (int n = 0; n < 16; n++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (n < 12) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        load_frags(cur, 2, 0);
        mma(1);
#pragma unroll
        for (int n = 0; n < 16; n++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (n < 12) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        load_frags(cur, 3, 1);
        mma(0);
#pragma unroll
        for (int n = 0; n < 16; n++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (n < 12) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        // tile kt+1 has landed in the other stage; nobody reads stage `cur` any more
        tile_barrier();
        {
            const int ktn = kt + 2 < KT ? kt + 2 : KT - 1;
            const char* sAn = sA0 + (cur ^ 1) * kAStage + a_base_l + a_xo[0];
            const char* sBn = sB0 + (cur ^ 1) * kBStageSw;
            bf16x4 lo[4], hi[4];
#pragma unroll
            for (int n = 0; n < 16; n++) {
                acc[n >> 2][n & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[1][n & 3], fa[1][n >> 2], acc[n >> 2][n & 3], 0, 0, 0);
                if (n < 4) fa[0][n] = *LDS_PTR(bf16x8, sAn + n * 4096);
                else if (n < 12) {
                    const int j = (n - 4) >> 1;
                    const int off = ((j & 1) ? b_p1 : b_p0) + (j >> 1) * 128;
                    if ((n & 1) == 0) lo[j] = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sBn + off));
                    else hi[j] = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sBn + off + 4 * 512));
                }
                dma_one(n, ktn, cur);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int j = 0; j < 4; j++) fb[0][j] = __builtin_shufflevector(lo[j], hi[j], 0, 1, 2, 3, 4, 5, 6, 7);
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
    tile_barrier();

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
    // the tiled kernel addresses a tile's rows with 32-bit byte offsets from the tile origin:
    // 255 rows of A (K elements each) and 49 rows of B (N elements each) must stay below 4 GiB
    const bool offsets_fit = K <= (1L << 23) && N <= (1L << 25);
    if (variant != 2 && aligned && offsets_fit && K > 0 && M % kBM == 0 && N % kBN == 0 && K % kBK == 0) {
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

