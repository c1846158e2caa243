// bf16 GEMM for gfx950: C[M,N] = A[M,K] * B[K,N], row-major bf16 in, f32 accumulate on
// MFMA, one round-to-nearest-even to bf16 at the end.
//
// Stands for the lazy graph of Tensor::matmul on bf16 operands
// (tensor/src/matmul.rs:82-110: broadcast multiply then sum(-1) with the accumulator
// promoted to f32, tensor/src/reduce.rs:101-117, cast back 665-691) after the tensor-core
// rewrite (schedule/src/optimizer/tc.rs:36-94 strips the CAST around the product, so
// exact bf16*bf16 products are accumulated in f32).  The instruction is the 16x16x32 shape the
// reference names in its CDNA table (schedule/src/optimizer/renderer.rs:549-558,724-733): of
// the two bf16 shapes of gfx950 it is the one the part sustains the higher clock on (it moves
// less accumulator data per product than 32x32x16; 1.96 against 1.72 PFLOP/s from registers).
//
// Main kernel: 256x256 output tile per workgroup of 4 waves (2x2), each wave 128x128 =
// 8x8 MFMA tiles (256 accumulator registers), K step 64 = two 32-deep sub-steps.  Tiles travel
// global -> LDS directly (global_load_lds, 16 B per lane, no register staging).  A is kept in LDS
// row-major with an XOR swizzle of its 16-byte chunks, B row-major (n contiguous) with
// an XOR swizzle of its 32-byte granules and read through the transposing LDS load,
// which hands each lane the 4 consecutive-k values of its column.  The MFMA is issued with
// swapped operands (D' = B^T A^T) so each lane ends up with 4 consecutive n of one row,
// which makes the epilogue 8-byte LDS writes and 16-byte coalesced global stores.  A second
// operand stored as B^T [N, K] (k contiguous: a Linear layer's weight) is staged and read
// exactly like A instead.
//
// Pipeline.  The vector-memory path takes a 1 KB copy every ~16 cycles, so the 64 copies a
// workgroup issues per K step need about half of the step's MFMA time; issued in one burst
// they stall the waves' instruction streams behind them.  They are therefore spread evenly,
// four per 32-MFMA phase and wave: the LDS holds two A stages and three B stages (160 KB, all
// of it), the copies of B tile kt+2 go out during the first two phases of tile kt into the
// stage tile kt-1 left, the one barrier of the step sits in the middle of it, and the copies
// of A tile kt+2 follow in the last two phases into the stage tile kt has just left.  For the
// barrier to sit there every fragment of tile kt must have been read by then: fragments are
// read a sub-step ahead of their MFMAs into two register slots (one per 32-deep sub-step).
//
// Shapes.  M is arbitrary, N and K multiples of 8: edge tiles redirect out-of-range rows and
// column chunks to the last valid one and mask their stores; a partial last K step is copied
// from zeros beyond K.  A second instance of the same body with a 128x256 workgroup tile serves
// shapes that would otherwise leave most compute units idle; a leading batch dimension runs as
// grid.y.  Everything else takes the any-shape kernel at the end of this file.
#include <hip/hip_runtime.h>
#include <atomic>

#include <cstdint>
#include <type_traits>

#include "kernels.h"

namespace mrk::dev {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

constexpr int kBM = 256, kBN = 256, kBK = 64;
constexpr int kBStageSw = kBK * kBN * 2;       // 32768 B per B stage, row pitch 512 B, granule-swizzled
// (an A stage is rows x 128 B, chunk-swizzled: 32768 B for the 256-row tile, which with two A
// and three B stages fills all 160 KB of the LDS)

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

// Sixteen zero bytes in device memory: where the copies of a partial last K step point the
// lanes whose k lies beyond K.
__device__ __attribute__((aligned(16))) const unsigned g_zero16[4] = {0u, 0u, 0u, 0u};

// kRaggedK: K is not a multiple of 64 (but of 8).  The copies of the last, partial K step use
// per-lane 64-bit addresses so that chunks beyond K can be redirected to g_zero16: zero
// operands on both sides contribute nothing.  Every other step is copied as in the full case.
//
// kJ: 32-column blocks (two MFMA tile columns each) per wave.  kJ = 4: 256x256 workgroup tile, waves 2x2, each 128x128.
// kJ = 2: 128x256 workgroup tile, waves 1x4, each 128x64 (half the accumulators, an A stage of
// half the size, the same B stages and pipeline) for shapes whose 256x256 tiles would leave
// most compute units without work.
//
// kSplitK: blockIdx.z selects a range of `kt_per_split` K steps; the workgroup writes its f32
// partial tile to W[z][batch][M][N] instead of C and gemm_splitk_reduce adds the partials up in
// a fixed order.  For shapes with so few tiles that the K loop itself has to be spread over
// the chip (a handful of rows against a large weight matrix).
//
// kResidual: the epilogue adds a bf16 matrix R of C's shape to the rounded product,
// C = bf16(float(bf16(A B)) + float(R)): the bits of the product kernel followed by an
// elementwise add, without writing and re-reading the product.
//
// kBT: the second operand is stored as B^T [N, K] (k contiguous).  Its stage holds 256 n-rows of
// 128 B, chunk-swizzled, copied and read like an A stage: one 16-byte read per fragment instead of
// two transposing 8-byte reads.  Same products in the same order: the same bits as the [K, N] form.
//
// kSwiGLU (256-row tile only): B is [K, 2F] holding a gate matrix in its columns [0, F) and an up
// matrix in [F, 2F) (N = 2F is B's row pitch); the workgroup's 256 tile columns are 128 gate
// columns followed by the 128 up columns at the same offset, and the epilogue writes
// C[M, F] = bf16(silu(float(bf16(A gate))) * float(bf16(A up))): the two products rounded to bf16
// as separate kernels would leave them, then x * sigmoid(x) * y in f32 with one rounding, without
// the 2F-wide product ever reaching memory.
//
// kF16: the operands and the result are IEEE half precision instead of bf16
// (v_mfma_f32_16x16x32_f16: the f16 entry of the reference's CDNA4 table,
// schedule/src/optimizer/renderer.rs:724-733).  Both are 16-bit elements, so copies, LDS layout,
// fragment reads and stores are the same bytes; only the matrix instruction and the conversion of
// the f32 accumulators differ.  The element pointers stay typed as 16-bit carriers.
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
template <bool kF16>
__device__ __forceinline__ bf16x4 round_to_elem(const f32x4& v) {
    if constexpr (kF16) return __builtin_bit_cast(bf16x4, __builtin_convertvector(v, f16x4));
    else return __builtin_convertvector(v, bf16x4);
}
//
// kRope (256-row tile only): the product of a packed projection whose first `split` columns are
// attention heads of 128 columns each (q | k of a fused QKV product).  The epilogue applies the
// rotary embedding (non-interleaved form, tensor/src/transformer.rs:32-69) to those heads on the
// bf16-rounded product, as the separate kernel would: with x1 = columns 0..63 and x2 = columns
// 64..127 of a head, out = [x1 cos - x2 sin | x1 sin + x2 cos] in f32 and one rounding, cos / sin
// [seq, 64] f32 indexed by the row's position (row % seq).  A wave's 128 columns are exactly one
// head, so both halves of a pair sit in the tile row the wave has just staged.  The rotated
// columns go to C with a row pitch of `split`; the columns behind them (v) go, unrotated, to a
// second matrix of their own with a row pitch of N - split.
struct RopeEpilogue {
    const float* cos;
    const float* sin;
    __bf16* rest;  // [M, N - split]: the columns from `split` on
    int seq, split;
};
template <bool kRaggedK, int kJ, bool kSplitK = false, bool kResidual = false, bool kSwiGLU = false, bool kBT = false, bool kF16 = false,
          bool kRope = false>
__device__ __forceinline__ void gemm_tile_body(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                               __bf16* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n,
                                               float* __restrict__ W = nullptr, int kt_per_split = 0,
                                               const __bf16* __restrict__ R = nullptr, const RopeEpilogue& rope = RopeEpilogue{},
                                               int ldr = -1) {
    static_assert(!kF16 || (!kResidual && !kSwiGLU && !kRope), "the fused epilogues exist for bf16 only");
    static_assert(!kRope || (kJ == 4 && !kSplitK && !kResidual && !kSwiGLU), "the rotary epilogue exists for the plain 256-row tile only");
    constexpr int kTM = kJ == 4 ? 256 : 128;      // rows of the workgroup tile
    constexpr int kAq = kTM / 32;                 // 1 KB A chunks (8 rows) each wave copies per K step
    constexpr int kAStageT = kTM * kBK * 2;       // bytes of an A stage
    constexpr int kCPitchT = kJ * 64 + 16;        // epilogue staging pitch per wave
    constexpr int kCWaveT = 128 * kCPitchT;
    constexpr int kSmemMainT = 2 * kAStageT + 3 * kBStageSw;
    constexpr int kSmemT = 4 * kCWaveT > kSmemMainT ? 4 * kCWaveT : kSmemMainT;
    constexpr int kI16 = 8, kJ16 = 2 * kJ;        // 16x16 MFMA tiles per wave: rows, columns
    constexpr int kSlots = 4 * kJ16;              // MFMAs per phase (four tile rows x all tile columns)
    // A stage: kTM rows x 128 B, 16 B chunks XOR-swizzled by ((row >> 1) & 7);
    // B stage: 64 k-rows x 512 B, 32 B granules XOR-swizzled by (k & 3).
    __shared__ __attribute__((aligned(1024))) char smem[kSmemT];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = kJ == 4 ? wave >> 1 : 0, wn = kJ == 4 ? (wave & 1) : wave;
    // blockIdx.y: which of the back-to-back stored products
    A += (size_t)blockIdx.y * M * K;
    B += (size_t)blockIdx.y * K * N;
    if (!kSplitK) C += (size_t)blockIdx.y * M * N;
    // row pitch of R in elements: N for a matrix of C's shape, 0 for one row added to every row of C (a bias)
    const size_t r_pitch = ldr < 0 ? (size_t)N : (size_t)ldr;
    if (kResidual) R += (size_t)blockIdx.y * M * r_pitch;
    int tile_m, tile_n;
    tile_of_block(blockIdx.x, tiles_m, tiles_n, &tile_m, &tile_n);
    static_assert(!kSwiGLU || (kJ == 4 && !kSplitK && !kResidual), "the gated epilogue exists for the 256-row tile only");
    const size_t m0 = (size_t)tile_m * kTM, n0 = (size_t)tile_n * (kSwiGLU ? kBN / 2 : kBN);
    char* sA0 = smem;                 // two A stages
    char* sB0 = smem + 2 * kAStageT;  // three B stages

    // ---- direct global -> LDS copies: each wave moves kAq KB of A and 8 KB of B per tile,
    // one instruction = 64 lanes x 16 B = 1 KB of contiguous LDS.
    // A chunk q (1 KB = 8 rows): lane -> row q*8 + lane/8, LDS chunk lane%8 holds logical
    // chunk (lane%8) ^ ((row >> 1) & 7).  The LDS serves 16 lanes x 16 B per cycle over 64
    // banks; with 128 B rows this swizzle puts 16 consecutive rows of one logical chunk
    // into 16 different 16 B slots.  ((row >> 1) & 7 depends on the parity of q: two variants.)
    // B chunk q (1 KB = 2 k-rows): lane -> k-row q*2 + lane/32, LDS 16 B chunk lane%32 ->
    // granule (lane%32)/2 ^ (krow & 3).
    // Ragged edges: a tile may reach past row M or column N.  Source rows / column chunks
    // beyond the edge are redirected to the last valid one (the duplicates only feed outputs
    // the epilogue does not store), which costs nothing per K step: the redirected offsets do
    // not depend on it.  N % 8 == 0 keeps the redirected chunk 16-byte aligned.
    unsigned a_voff[kAq];
#pragma unroll
    for (int q = 0; q < kAq; q++) {
        size_t row = m0 + wave * (kAq * 8) + q * 8 + (lane >> 3);
        row = row < (size_t)M ? row : (size_t)M - 1;
        const int chunk = (lane & 7) ^ ((q & 1) * 4 + (lane >> 4));
        a_voff[q] = (unsigned)(((row - m0) * K + (chunk << 3)) * 2);
    }
    const int b_h = lane & 1, b_g = (lane & 31) >> 1, b_r = lane >> 5;
    // kBT: B^T chunk q (1 KB = 8 n-rows of 128 B), copied and swizzled exactly like an A chunk;
    // each wave moves the 64 rows wave*64 .. wave*64+63 of the stage.
    unsigned bt_voff[kBT ? 8 : 1];
    if constexpr (kBT) {
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const size_t lr = wave * 64 + q * 8 + (lane >> 3);  // row inside the 256-row stage
            size_t row;
            if (kSwiGLU) {
                // stage rows 0..127 are gate rows of B^T, 128..255 the up rows at the same offset
                const size_t F = (size_t)N / 2, half = lr >> 7;
                row = n0 + (lr & 127);
                row = (row < F ? row : F - 1) + half * F;
            } else {
                row = n0 + lr;
                row = row < (size_t)N ? row : (size_t)N - 1;
            }
            const int chunk = (lane & 7) ^ ((q & 1) * 4 + (lane >> 4));
            bt_voff[q] = (unsigned)(((row - n0) * K + (chunk << 3)) * 2);
        }
    }
    unsigned b_voff[2];
#pragma unroll
    for (int par = 0; par < 2; par++) {
        size_t col = n0 + ((((b_g ^ (par * 2 + b_r)) << 1) | b_h) << 3);
        if (kSwiGLU) {
            // tile columns 0..127 come from the gate half of B, 128..255 from the up half
            const size_t F = (size_t)N / 2, lc = col - n0, half = lc >> 7;
            col = n0 + (lc & 127);
            col = (col + 8 <= F ? col : F - 8) + half * F;
        } else {
            col = col + 8 <= (size_t)N ? col : (size_t)N - 8;
        }
        b_voff[par] = (unsigned)(((size_t)(wave * 16 + b_r) * N + (col - n0)) * 2);
    }
    const int KT_all = (K + kBK - 1) / kBK;
    const int kt0 = kSplitK ? (int)blockIdx.z * kt_per_split : 0;  // first K step of this workgroup
    const int KT = kSplitK ? (KT_all - kt0 < kt_per_split ? KT_all - kt0 : kt_per_split) : KT_all;
    const bool has_last = kt0 + KT == KT_all;  // the (possibly partial) last K step is in this range
    const char* a_tile = reinterpret_cast<const char*>(A + m0 * K) + (size_t)kt0 * kBK * 2;
    const char* b_tile = kBT ? reinterpret_cast<const char*>(B + n0 * K) + (size_t)kt0 * kBK * 2
                             : reinterpret_cast<const char*>(B + n0) + (size_t)kt0 * kBK * N * 2;
    const unsigned lds_a = (unsigned)(uintptr_t)LDS_PTR(char, sA0) + wave * (kAq * 1024);
    const unsigned lds_b = (unsigned)(uintptr_t)LDS_PTR(char, sB0) + wave * 8192;
    // One direct copy: 64 lanes x 16 B land at LDS [m0, m0 + 1 KB); the compiler is not told
    // about it (it would otherwise wait for the copy before every later LDS read), so the
    // waits are explicit in the barriers below.
    auto dma = [&](unsigned lds_addr, unsigned voff, const char* sbase) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(sbase)
                     : "m0");
    };
    auto dma_from = [&](unsigned lds_addr, const char* addr) {  // per-lane 64-bit source address
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_addr), "v"(addr) : "m0");
    };
    const int k_last = K - (KT_all - 1) * kBK;  // depth of the last K step: 64, or 8..56 when ragged
    const char* zero16 = reinterpret_cast<const char*>(g_zero16);
    // (stage_off: byte offset of the stage inside the A or B part of the LDS)
    auto dma_a = [&](int q, int kt, unsigned stage_off) {
        if (kRaggedK && has_last && kt == KT - 1) {
            const int chunk = (lane & 7) ^ ((q & 1) * 4 + (lane >> 4));  // logical 8-deep k chunk of this lane
            dma_from(lds_a + stage_off + q * 1024,
                     chunk * 8 < k_last ? a_tile + (size_t)kt * kBK * 2 + a_voff[q] : zero16);
        } else {
            dma(lds_a + stage_off + q * 1024, a_voff[q], a_tile + (size_t)kt * kBK * 2);
        }
    };
    auto dma_b = [&](int q, int kt, unsigned stage_off) {
        if constexpr (kBT) {
            if (kRaggedK && has_last && kt == KT - 1) {
                const int chunk = (lane & 7) ^ ((q & 1) * 4 + (lane >> 4));
                dma_from(lds_b + stage_off + q * 1024,
                         chunk * 8 < k_last ? b_tile + (size_t)kt * kBK * 2 + bt_voff[q] : zero16);
            } else {
                dma(lds_b + stage_off + q * 1024, bt_voff[q], b_tile + (size_t)kt * kBK * 2);
            }
            return;
        }
        if (kRaggedK && has_last && kt == KT - 1) {
            dma_from(lds_b + stage_off + q * 1024,
                     wave * 16 + q * 2 + b_r < k_last ? b_tile + ((size_t)kt * kBK + q * 2) * N * 2 + b_voff[q & 1] : zero16);
            return;
        }
        dma(lds_b + stage_off + q * 1024, b_voff[q & 1], b_tile + ((size_t)kt * kBK + q * 2) * N * 2);
    };

    f32x4 acc[kI16][kJ16];
#pragma unroll
    for (int i = 0; i < kI16; i++)
#pragma unroll
        for (int j = 0; j < kJ16; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[i][j][e] = 0.0f;

    // lane-constant parts of the fragment addresses.  An operand fragment of the 16x16x32 MFMA is
    // row (lane % 16) of a 16-row tile, k = 8 * (lane / 16) .. +7 of the 32-deep sub-step.
    const int a_base_l = (wm * 128 + (lane & 15)) * 128;  // + i*2048
    int a_xo[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) a_xo[ks] = ((ks * 4 + (lane >> 4)) ^ ((lane >> 1) & 7)) << 4;
    // B through the transposing read: 16-lane block b = lane / 16 covers k-rows 8b .. 8b+7 (two
    // reads of four rows), lane j' of the block points at k-row j'/4, 8-byte unit j'%4 of the
    // 32-byte granule (16 columns) of its tile column
    const int b_rr = (lane & 15) >> 2;
    const int b_row_l = (8 * (lane >> 4) + b_rr) * 512 + 8 * (lane & 3) + ((wn * kJ16) << 5);  // + ks*32*512 (+ 4*512: second read)
    int b_p[4];  // tile column j: b_p[j & 3] + (j >> 2) * 128
#pragma unroll
    for (int q = 0; q < 4; q++) b_p[q] = b_row_l + ((q ^ b_rr) << 5);
    const int bt_base_l = (wn * (kJ * 32) + (lane & 15)) * 128;  // kBT: + j*2048, chunk offset a_xo[ks]

    bf16x8 fa[2][kI16], fb[2][kJ16];  // fragment slot = 32-deep sub-step
    // all but this wave's newest 8 copies (the B chunks issued since the last barrier) have
    // landed, its LDS reads are complete; then all waves meet
    auto tile_barrier = [&]() { asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    auto full_barrier = [&]() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

#pragma unroll
    for (int q = 0; q < kAq; q++) dma_a(q, 0, 0);
#pragma unroll
    for (int q = 0; q < 8; q++) dma_b(q, 0, 0);
#pragma unroll
    for (int q = 0; q < kAq; q++) dma_a(q, KT > 1 ? 1 : 0, kAStageT);
#pragma unroll
    for (int q = 0; q < 8; q++) dma_b(q, KT > 1 ? 1 : 0, kBStageSw);
    // tile 0 has landed (the kAq + 8 copies of tile 1 may still be in flight; the first
    // tile_barrier() covers them)
    if (kAq == 8) asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    // B fragment of tile column j, sub-step base sB (a stage plus ks * 32 rows)
    auto read_b = [&](const char* sB, int j, bf16x4* lo, bf16x4* hi) {
        const int off = b_p[j & 3] + (j >> 2) * 128;
        *lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sB + off));
        *hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sB + off + 4 * 512));
    };
    {  // the fragments of sub-step 0 of tile 0
        const char* sA = sA0 + a_base_l + a_xo[0];
#pragma unroll
        for (int i = 0; i < kI16; i++) fa[0][i] = *LDS_PTR(bf16x8, sA + i * 2048);
#pragma unroll
        for (int j = 0; j < kJ16; j++) {
            if constexpr (kBT) {
                fb[0][j] = *LDS_PTR(bf16x8, sB0 + bt_base_l + a_xo[0] + j * 2048);
            } else {
                bf16x4 lo, hi;
                read_b(sB0, j, &lo, &hi);
                fb[0][j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
        }
    }

    // The accumulators as the matrix instructions below see them: initialised, and the writes of
    // the initial zeros a few wait states back.
    auto touch_acc = [&]() {
#pragma unroll
        for (int i = 0; i < kI16; i++)
#pragma unroll
            for (int j = 0; j < kJ16; j++) asm volatile("" : "+a"(acc[i][j]));
    };
    touch_acc();
    asm volatile("s_nop 7" ::: "memory");

    // Scalars carried from one K step to the next: the tile the copies of this step fetch
    // (kt2 = min(kt + 2, KT - 1)), its source addresses, and the three B stages' byte offsets
    // (tile kt, tile kt + 1, the stage being filled).  They are advanced at the end of a step, in
    // issue slots nothing else uses, instead of being recomputed from kt at the top of the next.
    struct Carried {
        int kt2;
        const char* a_src;  // A tile kt2 (row 0 of the workgroup tile)
        const char* b_src;  // B tile kt2: k-row 0 of it ([K, N] form) or n-row 0 (B^T form)
        unsigned sb_cur, sb_nxt, sb_fill;
    } ls;
    const unsigned b_step32 = kBT ? (unsigned)(kBK * 2) : (unsigned)kBK * (unsigned)N * 2u;  // bytes from one B tile to the next (N < 2^25)
    unsigned adv = 0;
    const size_t b_row2 = (size_t)N * 4;                                // [K, N] form: bytes from one 1 KB chunk (2 k-rows) to the next
    ls.kt2 = KT > 2 ? 2 : KT - 1;
    ls.a_src = a_tile + (size_t)ls.kt2 * kBK * 2;
    ls.b_src = b_tile + (size_t)ls.kt2 * b_step32;
    ls.sb_cur = 0, ls.sb_nxt = kBStageSw, ls.sb_fill = 2 * kBStageSw;

    // The matrix instruction, written out so that the accumulator stays in place in the
    // accumulation registers (through the builtin the compiler leaves this shape untied and copies
    // tiles around) ...
    auto mfma = [&](f32x4& c, const bf16x8& a, const bf16x8& b) {
        if constexpr (kF16) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
        else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    };
    // One direct copy with the LDS address formed in the instruction that writes M0 ...
    auto dma_at = [&](unsigned lds_base, auto q_c, unsigned voff, const char* sbase) {
        asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
                     :
                     : "s"(lds_base), "n"(decltype(q_c)::value * 1024), "v"(voff), "s"(sbase)
                     : "m0", "scc");
    };
    // ... and the matrix instruction with one such copy behind it in one statement (the LDS address is formed
    // in the instruction that writes M0), so that nothing else lands between them.
    auto mfma_dma = [&](f32x4& c, const bf16x8& a, const bf16x8& b, unsigned lds_base, auto q_c, unsigned voff, const char* sbase) {
        if constexpr (kF16)
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0\n\ts_add_u32 m0, %3, %4\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %5, %6"
                         : "+a"(c)
                         : "v"(a), "v"(b), "s"(lds_base), "n"(decltype(q_c)::value * 1024), "v"(voff), "s"(sbase)
                         : "m0", "scc");
        else
            asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\ts_add_u32 m0, %3, %4\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %5, %6"
                         : "+a"(c)
                         : "v"(a), "v"(b), "s"(lds_base), "n"(decltype(q_c)::value * 1024), "v"(voff), "s"(sbase)
                         : "m0", "scc");
    };

    // One phase = half of a 32-deep sub-step: phase p covers sub-step p / 2 (fragment slot p / 2)
    // and tile rows 4 * (p % 2) .. +3 against every tile column, 4 * kJ16 MFMAs, with the other
    // pipes' work slotted between them: the LDS reads of the other slot's fragments (the next
    // sub-step; from sAn / sBn) for the same four tile rows and half of the tile columns, and
    // chunk copies of tile kt2: phases 0-1 four of its B chunks each into the B stage being
    // filled, phases 2-3 (after the barrier) kAq / 2 of its A chunks each into A stage `cur`.
    // The columns loaded during the second phase of a sub-step are the ones the next sub-step
    // multiplies last.  A wave issues one instruction every four cycles and an MFMA of this shape
    // occupies the pipe for sixteen, so at most three other instructions fit behind an MFMA
    // without delaying the next one: the reads take the first slots of a phase one by one, every
    // copy (M0, the wait state, the load) a later slot of its own, its source address the slot
    // before, and the carried scalars the tail of the last phase.
    auto phase = [&](auto p_c, auto cur_c, const char* sAn, const char* sBn) {
        constexpr int p = decltype(p_c)::value, cur = decltype(cur_c)::value;
        constexpr int slot = p >> 1, nslot = slot ^ 1, h = p & 1;
        constexpr int kHalfJ = kJ16 / 2;  // tile columns per half
        bf16x4 lo[kHalfJ], hi[kHalfJ];
        constexpr int kCopies = p < 2 ? 4 : kAq / 2;                 // copies of this phase
        constexpr int kFirst = 4 + kJ16;                             // first slot without a fragment read
        constexpr int kTail = p == 3 ? 3 : p == 2 ? 1 : 0;           // last slots, kept for the carried scalars
        constexpr int kEvery = (kSlots - kFirst - kTail) / kCopies;  // slots per copy (address, then copy)
        static_assert(kEvery >= 2, "a copy needs two slots");
        const unsigned lds_dst = p < 2 ? lds_b + ls.sb_fill : lds_a + cur * kAStageT;
        const bool ragged_now = kRaggedK && has_last && ls.kt2 == KT - 1;  // this step copies the partial last tile
        const char* src = p < 2 ? ls.b_src : ls.a_src;
        if (p == 1 && !kBT) src += 4 * b_row2;
#pragma unroll
        for (int n = 0; n < kSlots; n++) {
            // first the columns whose fragments arrived a sub-step ago, then the other half; back
            // and forth over the columns and the rows, so that consecutive instructions share one
            // operand register set (fewer operand bits toggle: about 1 % on the clock the part
            // sustains)
            const int jh = n / (kSlots / 2), r = n % (kSlots / 2), rr = r / kHalfJ, jj = r % kHalfJ;
            const int mi = 4 * h + (jh ? 3 - rr : rr);
            const int mj = jh * kHalfJ + ((rr & 1) ? kHalfJ - 1 - jj : jj);
            const bool copy_range = n >= kFirst && (n - kFirst) / kEvery < kCopies;
            const int c = copy_range ? (n - kFirst) / kEvery : 0, part = copy_range ? (n - kFirst) % kEvery : -1;
            const int q = (p & 1) * kCopies + c;  // chunk of the tile
            // a copy slot: the MFMA and the copy as one statement; where a step may have to copy
            // the partial last tile instead (kRaggedK) the choice is made at run time, and the MFMA
            // stays outside that branch: an accumulator that flows through a branch would be moved
            // by the compiler, which does not know that it has to wait for the matrix pipe first
            auto with_q = [&](auto&& f) {
                switch (q) {  // q is a constant of the unrolled loop
                    case 0: f(std::integral_constant<int, 0>{}); break;
                    case 1: f(std::integral_constant<int, 1>{}); break;
                    case 2: f(std::integral_constant<int, 2>{}); break;
                    case 3: f(std::integral_constant<int, 3>{}); break;
                    case 4: f(std::integral_constant<int, 4>{}); break;
                    case 5: f(std::integral_constant<int, 5>{}); break;
                    case 6: f(std::integral_constant<int, 6>{}); break;
                    default: f(std::integral_constant<int, 7>{}); break;
                }
            };
            auto voff_of = [&](auto q_c) {
                constexpr int qq = decltype(q_c)::value;
                return p >= 2 ? a_voff[qq < kAq ? qq : 0] : kBT ? bt_voff[kBT ? qq : 0] : b_voff[qq & 1];
            };
            if (part == 1 && !kRaggedK) {
                with_q([&](auto q_c) { mfma_dma(acc[mi][mj], fb[slot][mj], fa[slot][mi], lds_dst, q_c, voff_of(q_c), src); });
            } else {
                mfma(acc[mi][mj], fb[slot][mj], fa[slot][mi]);
                if (part == 1) {
                    if (ragged_now) {
                        if (p < 2) dma_b(q, ls.kt2, ls.sb_fill);
                        else dma_a(q, ls.kt2, cur * kAStageT);
                    } else {
                        with_q([&](auto q_c) { dma_at(lds_dst, q_c, voff_of(q_c), src); });
                    }
                }
            }
            if (n < 4) fa[nslot][4 * h + n] = *LDS_PTR(bf16x8, sAn + (4 * h + n) * 2048);
            else if constexpr (kBT) {
                if (n < 4 + kHalfJ) fb[nslot][h * kHalfJ + n - 4] = *LDS_PTR(bf16x8, sBn + (h * kHalfJ + n - 4) * 2048);
            } else if (n < 4 + 2 * kHalfJ) {
                const int jl = (n - 4) >> 1, j = h * kHalfJ + jl;
                const int off = b_p[j & 3] + (j >> 2) * 128;
                if ((n & 1) == 0) lo[jl] = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sBn + off));
                else hi[jl] = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sBn + off + 4 * 512));
            }
            if (part == 0) {
                // the chunk's source address, one slot ahead of the copy
                if (p < 2 && !kBT && c > 0) src += b_row2;
                asm volatile("" : "+s"(src));
            }
            // the scalars of the next K step, in the slots left over at the end
            if (p == 2 && n == kSlots - 1) {
                // (the copies of this step into the stage being filled went out in phases 0-1)
                const unsigned t = ls.sb_cur;
                ls.sb_cur = ls.sb_nxt;
                ls.sb_nxt = ls.sb_fill;
                ls.sb_fill = t;
            }
            if (p == 3 && n == kSlots - 3) {
                // 1 while the copies have not reached the last tile (as a minimum: a comparison's
                // result would take a detour through the vector unit to become a number)
                adv = (unsigned)__builtin_elementwise_min(KT - 1 - ls.kt2, 1);
                ls.kt2 += (int)adv;
                asm volatile("" : "+s"(adv));
            }
            if (p == 3 && n == kSlots - 2) {
                ls.a_src += adv * (unsigned)(kBK * 2);
                asm volatile("" : "+s"(ls.a_src));
            }
            if (p == 3 && n == kSlots - 1) {
                ls.b_src += adv * b_step32;  // (32-bit product: a tile-to-tile step stays below 4 GiB)
                asm volatile("" : "+s"(ls.b_src));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (!kBT) {
#pragma unroll
            for (int jl = 0; jl < kHalfJ; jl++)
                fb[nslot][h * kHalfJ + jl] = __builtin_shufflevector(lo[jl], hi[jl], 0, 1, 2, 3, 4, 5, 6, 7);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;
    using C2 = std::integral_constant<int, 2>;
    using C3 = std::integral_constant<int, 3>;
    // tile kt: A in stage cur = kt & 1, B in the stage at ls.sb_cur (next tile's B at ls.sb_nxt, the one after goes to ls.sb_fill)
    auto iteration = [&](auto cur_c) {
        constexpr int cur = decltype(cur_c)::value;
        using C = std::integral_constant<int, cur>;
        const char* sAc = sA0 + cur * kAStageT + a_base_l;
        const char* sBc = sB0 + ls.sb_cur + (kBT ? bt_base_l : 0);
        const char* sAx = sA0 + (cur ^ 1) * kAStageT + a_base_l;
        const char* sBx = sB0 + ls.sb_nxt + (kBT ? bt_base_l : 0);
        // sub-step ks of a B stage: 32 k-rows of 512 B further, or (kBT) the same chunk offset as A's
        auto b_ks = [&](int ks) { return kBT ? a_xo[ks] : ks * 32 * 512; };
        phase(C0{}, C{}, sAc + a_xo[1], sBc + b_ks(1));
        phase(C1{}, C{}, sAc + a_xo[1], sBc + b_ks(1));
        // tile kt+1 has landed; nobody reads A stage cur any more
        tile_barrier();
        phase(C2{}, C{}, sAx + a_xo[0], sBx + b_ks(0));
        phase(C3{}, C{}, sAx + a_xo[0], sBx + b_ks(0));
    };
    // What the epilogue of the plain and the residual product needs, ahead of the loop's end: lane l
    // stores (and fetches from R) 16-byte chunk l % kChunks of row it * kRowsPerIt + l / kChunks of
    // the wave's 128-row tile, for it = 0 .. kIts-1.
    const size_t row0 = m0 + wm * 128, col0 = n0 + wn * (kJ * 32);
    constexpr int kChunks = kJ * 4;          // 16-byte chunks per row of the wave's tile
    constexpr int kRowsPerIt = 64 / kChunks;  // rows one store instruction covers
    constexpr int kIts = 128 / kRowsPerIt;
    const int lr = lane / kChunks, lc = lane % kChunks;
    const int rows_here = row0 >= (size_t)M ? 0 : (size_t)M - row0 < 128 ? (int)((size_t)M - row0) : 128;  // rows of the wave's tile inside C
    const bool col_ok = col0 + lc * 8 + 8 <= (size_t)N;
    u32x4 res[kResidual ? kIts : 1];
    auto fetch_residual = [&](int first, int last) {
        const __bf16* Rl = R + (row0 + lr) * r_pitch + col0 + lc * 8;
#pragma unroll
        for (int it = first; it < last; it++) {
            res[it] = u32x4{0u, 0u, 0u, 0u};
            if (col_ok && it * kRowsPerIt + lr < rows_here) res[it] = *reinterpret_cast<const u32x4*>(Rl + (size_t)(it * kRowsPerIt) * r_pitch);
        }
    };
    {
        int kt = 0;
        for (; kt + 1 < KT; kt += 2) {
            iteration(C0{});
            iteration(C1{});
        }
        if (kt < KT) iteration(C0{});
    }
    // The residual rows are on their way while the accumulators are converted and staged: the
    // fragment registers of the loop are free from here on.  (Fetching half of them before the
    // last two K steps instead measured the same: the loop's waits on its own copies count
    // vector-memory operations in order, so they wait for the residual rows as well.)
    if constexpr (kResidual) fetch_residual(0, kIts);
    full_barrier();
    // the last MFMAs' results must have left the matrix pipe before the vector ALUs read them (the
    // compiler does not see the instructions above as matrix operations); the empty statements
    // behind the wait keep every later use of an accumulator behind it
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    touch_acc();

    // Epilogue.  With swapped operands lane l of tile (i, j) holds, in its four registers,
    // C[m = i*16 + l%16][n = j*16 + 4*(l/16) + 0..3].
    if (kSplitK) {
        // f32 partials straight from the registers: 16 bytes per lane, rows and columns masked
        float* Wt = W + ((size_t)blockIdx.z * gridDim.y + blockIdx.y) * (size_t)M * N;
#pragma unroll
        for (int i = 0; i < kI16; i++)
#pragma unroll
            for (int j = 0; j < kJ16; j++) {
                const size_t row = row0 + i * 16 + (lane & 15), col = col0 + j * 16 + 4 * (lane >> 4);
                if (row < (size_t)M && col + 4 <= (size_t)N) *reinterpret_cast<f32x4*>(Wt + row * N + col) = acc[i][j];
            }
        return;
    }
    char* sC = smem + wave * kCWaveT;
    if constexpr (!kSwiGLU) {
        // The plain and the residual product: 16 rows at a time.  A wave reads back only what it
        // staged itself, and the LDS serves a wave's requests in order, so the rows of tile row i
        // are read back and stored while tile row i + 1 is being converted and staged: the stores
        // start one tile row after the loop ends instead of after the whole staging.
        constexpr int kPerRow = 16 / kRowsPerIt;  // store instructions per tile row
        // (rotary epilogue: the tile's columns lie either all in front of `split` or all behind it)
        const bool rotate = kRope && n0 < (size_t)rope.split;
        const size_t ldc = !kRope ? (size_t)N : rotate ? (size_t)rope.split : (size_t)(N - rope.split);
        __bf16* Cl = (!kRope || rotate ? C + col0 : rope.rest + (col0 - rope.split)) + (row0 + lr) * ldc + lc * 8;
        const char* sCl = sC + lr * kCPitchT + lc * 16;
        auto stage_row = [&](int i) {
#pragma unroll
            for (int j = 0; j < kJ16; j++) {
                bf16x4 h = round_to_elem<kF16>(acc[i][j]);
                *LDS_PTR(bf16x4, sC + (i * 16 + (lane & 15)) * kCPitchT + (j * 16 + 4 * (lane >> 4)) * 2) = h;
            }
        };
        // Rotary epilogue: the angles of a tile row (four store steps: eight cos and eight sin values each)
        // are requested one tile row ahead; the row's position advances by the rows of a store step,
        // wrapping at seq, so the only division is the one that finds the first position.
        f32x8 cs_nxt[kRope ? kPerRow : 1], sn_nxt[kRope ? kPerRow : 1], cs_cur[kRope ? kPerRow : 1], sn_cur[kRope ? kPerRow : 1];
        unsigned rope_pos = 0;
        auto fetch_angles = [&]() {
            if constexpr (kRope) {
                const unsigned seq = (unsigned)rope.seq;
#pragma unroll
                for (int t = 0; t < kPerRow; t++) {
                    cs_nxt[t] = *reinterpret_cast<const f32x8*>(rope.cos + (size_t)rope_pos * 64 + (lc & 7) * 8);
                    sn_nxt[t] = *reinterpret_cast<const f32x8*>(rope.sin + (size_t)rope_pos * 64 + (lc & 7) * 8);
                    rope_pos += kRowsPerIt;
                    if (seq < (unsigned)kRowsPerIt) rope_pos %= seq;
                    else if (rope_pos >= seq) rope_pos -= seq;
                }
            }
        };
        if constexpr (kRope) {
            if (rotate) {
                rope_pos = (unsigned)((row0 + lr) % (size_t)rope.seq);
                fetch_angles();
            }
        }
        stage_row(0);
#pragma unroll
        for (int i = 0; i < kI16; i++) {
            u32x4 v[kPerRow], pv[kRope ? kPerRow : 1];
#pragma unroll
            for (int t = 0; t < kPerRow; t++) v[t] = *LDS_PTR(u32x4, sCl + (i * 16 + t * kRowsPerIt) * kCPitchT);
            if constexpr (kRope) {
                if (rotate) {
                    // the partners 64 columns away: chunk lc ^ 8 of the same staged rows
#pragma unroll
                    for (int t = 0; t < kPerRow; t++) {
                        pv[t] = *LDS_PTR(u32x4, sC + (i * 16 + t * kRowsPerIt + lr) * kCPitchT + (lc ^ 8) * 16);
                        cs_cur[t] = cs_nxt[t];
                        sn_cur[t] = sn_nxt[t];
                    }
                    if (i + 1 < kI16) fetch_angles();
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (i + 1 < kI16) stage_row(i + 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < kPerRow; t++) {
                const int r = i * 16 + t * kRowsPerIt;
                if constexpr (kResidual) {
                    const f32x8 sum = __builtin_convertvector(__builtin_bit_cast(bf16x8, v[t]), f32x8) +
                                      __builtin_convertvector(__builtin_bit_cast(bf16x8, res[i * kPerRow + t]), f32x8);
                    v[t] = __builtin_bit_cast(u32x4, __builtin_convertvector(sum, bf16x8));
                }
                if constexpr (kRope) {
                    if (rotate) {
                        // this lane's 8 columns of a head, their partners, and the 8 angles of the row's position
                        const f32x8 x = __builtin_convertvector(__builtin_bit_cast(bf16x8, v[t]), f32x8);
                        const f32x8 y = __builtin_convertvector(__builtin_bit_cast(bf16x8, pv[t]), f32x8);
                        const f32x8 sn = lc < 8 ? -sn_cur[t] : sn_cur[t];  // first half: x1 cos - x2 sin; second half: x2 cos + x1 sin
                        const f32x8 o = x * cs_cur[t] + y * sn;
                        v[t] = __builtin_bit_cast(u32x4, __builtin_convertvector(o, bf16x8));
                    }
                }
                if (col_ok && r + lr < rows_here) *reinterpret_cast<u32x4*>(Cl + (size_t)r * ldc) = v[t];
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < kI16; i++)
#pragma unroll
        for (int j = 0; j < kJ16; j++) {
            bf16x4 h = __builtin_convertvector(acc[i][j], bf16x4);
            const int ml = i * 16 + (lane & 15);
            const int nl = j * 16 + 4 * (lane >> 4);
            *LDS_PTR(bf16x4, sC + ml * kCPitchT + nl * 2) = h;
        }
    // The gated epilogue: waves (wm, 0) and (wm, 1) staged the gate and the up block of the same
    // 128 rows x 128 columns; each of the two now combines 64 of those rows: 16 chunks of 8 columns
    // per row.
    if constexpr (kSwiGLU) {
        __syncthreads();
        const size_t F = (size_t)N / 2;
        const char* sG = smem + (wm * 2 + 0) * kCWaveT;
        const char* sU = smem + (wm * 2 + 1) * kCWaveT;
#pragma unroll 4
        for (int it = 0; it < 16; it++) {
            const int r = wn * 64 + it * 4 + (lane >> 4);
            const int ch = lane & 15;
            const f32x8 gf = __builtin_convertvector(__builtin_bit_cast(bf16x8, *LDS_PTR(u32x4, sG + r * kCPitchT + ch * 16)), f32x8);
            const f32x8 uf = __builtin_convertvector(__builtin_bit_cast(bf16x8, *LDS_PTR(u32x4, sU + r * kCPitchT + ch * 16)), f32x8);
            f32x8 y;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                // x * sigmoid(x) * y with sigmoid(x) = 1 / (1 + exp2(x * (-1 / ln 2)))
                const float sg = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(gf[e] * -1.4426950408889634f));
                y[e] = gf[e] * sg * uf[e];
            }
            const u32x4 v = __builtin_bit_cast(u32x4, __builtin_convertvector(y, bf16x8));
            if (row0 + r < (size_t)M && n0 + ch * 8 + 8 <= F) *reinterpret_cast<u32x4*>(C + (row0 + r) * F + n0 + ch * 8) = v;
        }
    }
}

__global__ __launch_bounds__(256) void gemm_bf16_tile256(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                         __bf16* __restrict__ C, int M, int N, int K, int tiles_m,
                                                         int tiles_n) {
    gemm_tile_body<false, 4>(A, B, C, M, N, K, tiles_m, tiles_n);
}
// B^T variants: the second operand is Bt[N, K] row-major (k contiguous, the layout of a Linear
// layer's weight), C = A Bt^T; for the gated epilogue Bt is [2F, K], gate rows first.
#define MRK_GEMM_NT_KERNEL(name, ...)                                                                                      \
    __global__ __launch_bounds__(256) void name(const __bf16* __restrict__ A, const __bf16* __restrict__ Bt,              \
                                                __bf16* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n) { \
        gemm_tile_body<__VA_ARGS__>(A, Bt, C, M, N, K, tiles_m, tiles_n);                                                  \
    }
#define MRK_GEMM_NT_RESIDUAL_KERNEL(name, ...)                                                                          \
    __global__ __launch_bounds__(256) void name(const __bf16* __restrict__ A, const __bf16* __restrict__ Bt,           \
                                                const __bf16* __restrict__ R, __bf16* __restrict__ C, int M, int N,    \
                                                int K, int tiles_m, int tiles_n, int ldr) {                            \
        gemm_tile_body<__VA_ARGS__>(A, Bt, C, M, N, K, tiles_m, tiles_n, nullptr, 0, R, RopeEpilogue{}, ldr);           \
    }
MRK_GEMM_NT_KERNEL(gemm_bf16_nt_tile256, false, 4, false, false, false, true)
MRK_GEMM_NT_KERNEL(gemm_bf16_nt_tile256_ragged_k, true, 4, false, false, false, true)
MRK_GEMM_NT_KERNEL(gemm_bf16_nt_tile128, false, 2, false, false, false, true)
MRK_GEMM_NT_KERNEL(gemm_bf16_nt_tile128_ragged_k, true, 2, false, false, false, true)
MRK_GEMM_NT_KERNEL(gemm_bf16_nt_tile256_swiglu, false, 4, false, false, true, true)
MRK_GEMM_NT_KERNEL(gemm_bf16_nt_tile256_swiglu_ragged_k, true, 4, false, false, true, true)
MRK_GEMM_NT_RESIDUAL_KERNEL(gemm_bf16_nt_tile256_residual, false, 4, false, true, false, true)
MRK_GEMM_NT_RESIDUAL_KERNEL(gemm_bf16_nt_tile256_residual_ragged_k, true, 4, false, true, false, true)
MRK_GEMM_NT_RESIDUAL_KERNEL(gemm_bf16_nt_tile128_residual, false, 2, false, true, false, true)
MRK_GEMM_NT_RESIDUAL_KERNEL(gemm_bf16_nt_tile128_residual_ragged_k, true, 2, false, true, false, true)
// half-precision instantiations (plain product; [K, N] and [N, K] second operand)
MRK_GEMM_NT_KERNEL(gemm_f16_tile256, false, 4, false, false, false, false, true)
MRK_GEMM_NT_KERNEL(gemm_f16_tile256_ragged_k, true, 4, false, false, false, false, true)
MRK_GEMM_NT_KERNEL(gemm_f16_tile128, false, 2, false, false, false, false, true)
MRK_GEMM_NT_KERNEL(gemm_f16_tile128_ragged_k, true, 2, false, false, false, false, true)
MRK_GEMM_NT_KERNEL(gemm_f16_nt_tile256, false, 4, false, false, false, true, true)
MRK_GEMM_NT_KERNEL(gemm_f16_nt_tile256_ragged_k, true, 4, false, false, false, true, true)
MRK_GEMM_NT_KERNEL(gemm_f16_nt_tile128, false, 2, false, false, false, true, true)
MRK_GEMM_NT_KERNEL(gemm_f16_nt_tile128_ragged_k, true, 2, false, false, false, true, true)
#undef MRK_GEMM_NT_KERNEL
#undef MRK_GEMM_NT_RESIDUAL_KERNEL
__global__ __launch_bounds__(256) void gemm_f16_tile128_splitk(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                               float* __restrict__ W, int M, int N, int K, int tiles_m,
                                                               int tiles_n, int kt_per_split) {
    gemm_tile_body<false, 2, true, false, false, false, true>(A, B, nullptr, M, N, K, tiles_m, tiles_n, W, kt_per_split);
}
__global__ __launch_bounds__(256) void gemm_f16_tile128_splitk_ragged_k(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                                        float* __restrict__ W, int M, int N, int K, int tiles_m,
                                                                        int tiles_n, int kt_per_split) {
    gemm_tile_body<true, 2, true, false, false, false, true>(A, B, nullptr, M, N, K, tiles_m, tiles_n, W, kt_per_split);
}
// split-K over a second operand stored [N, K]
#define MRK_GEMM_NT_SPLITK_KERNEL(name, ragged, f16)                                                                                   \
    __global__ __launch_bounds__(256) void name(const __bf16* __restrict__ A, const __bf16* __restrict__ B, float* __restrict__ W, int M, \
                                                int N, int K, int tiles_m, int tiles_n, int kt_per_split) {                             \
        gemm_tile_body<ragged, 2, true, false, false, true, f16>(A, B, nullptr, M, N, K, tiles_m, tiles_n, W, kt_per_split);            \
    }
MRK_GEMM_NT_SPLITK_KERNEL(gemm_bf16_nt_tile128_splitk, false, false)
MRK_GEMM_NT_SPLITK_KERNEL(gemm_bf16_nt_tile128_splitk_ragged_k, true, false)
MRK_GEMM_NT_SPLITK_KERNEL(gemm_f16_nt_tile128_splitk, false, true)
MRK_GEMM_NT_SPLITK_KERNEL(gemm_f16_nt_tile128_splitk_ragged_k, true, true)
#undef MRK_GEMM_NT_SPLITK_KERNEL
__global__ __launch_bounds__(256) void gemm_bf16_tile256_rope(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                              __bf16* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n,
                                                              RopeEpilogue rope) {
    gemm_tile_body<false, 4, false, false, false, false, false, true>(A, B, C, M, N, K, tiles_m, tiles_n, nullptr, 0, nullptr, rope);
}
__global__ __launch_bounds__(256) void gemm_bf16_nt_tile256_rope(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                              __bf16* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n,
                                                              RopeEpilogue rope) {
    gemm_tile_body<false, 4, false, false, false, true, false, true>(A, B, C, M, N, K, tiles_m, tiles_n, nullptr, 0, nullptr, rope);
}
__global__ __launch_bounds__(256) void gemm_bf16_tile256_ragged_k(const __bf16* __restrict__ A,
                                                                  const __bf16* __restrict__ B, __bf16* __restrict__ C,
                                                                  int M, int N, int K, int tiles_m, int tiles_n) {
    gemm_tile_body<true, 4>(A, B, C, M, N, K, tiles_m, tiles_n);
}
__global__ __launch_bounds__(256) void gemm_bf16_tile256_residual(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                                  const __bf16* __restrict__ R, __bf16* __restrict__ C, int M,
                                                                  int N, int K, int tiles_m, int tiles_n, int ldr) {
    gemm_tile_body<false, 4, false, true>(A, B, C, M, N, K, tiles_m, tiles_n, nullptr, 0, R, RopeEpilogue{}, ldr);
}
__global__ __launch_bounds__(256) void gemm_bf16_tile256_residual_ragged_k(const __bf16* __restrict__ A,
                                                                           const __bf16* __restrict__ B,
                                                                           const __bf16* __restrict__ R, __bf16* __restrict__ C,
                                                                           int M, int N, int K, int tiles_m, int tiles_n, int ldr) {
    gemm_tile_body<true, 4, false, true>(A, B, C, M, N, K, tiles_m, tiles_n, nullptr, 0, R, RopeEpilogue{}, ldr);
}
__global__ __launch_bounds__(256) void gemm_bf16_tile256_swiglu(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                                __bf16* __restrict__ C, int M, int N2, int K, int tiles_m,
                                                                int tiles_n) {
    gemm_tile_body<false, 4, false, false, true>(A, B, C, M, N2, K, tiles_m, tiles_n);
}
__global__ __launch_bounds__(256) void gemm_bf16_tile256_swiglu_ragged_k(const __bf16* __restrict__ A,
                                                                         const __bf16* __restrict__ B, __bf16* __restrict__ C,
                                                                         int M, int N2, int K, int tiles_m, int tiles_n) {
    gemm_tile_body<true, 4, false, false, true>(A, B, C, M, N2, K, tiles_m, tiles_n);
}
__global__ __launch_bounds__(256) void gemm_bf16_tile128_residual(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                                  const __bf16* __restrict__ R, __bf16* __restrict__ C, int M,
                                                                  int N, int K, int tiles_m, int tiles_n, int ldr) {
    gemm_tile_body<false, 2, false, true>(A, B, C, M, N, K, tiles_m, tiles_n, nullptr, 0, R, RopeEpilogue{}, ldr);
}
__global__ __launch_bounds__(256) void gemm_bf16_tile128_residual_ragged_k(const __bf16* __restrict__ A,
                                                                           const __bf16* __restrict__ B,
                                                                           const __bf16* __restrict__ R, __bf16* __restrict__ C,
                                                                           int M, int N, int K, int tiles_m, int tiles_n, int ldr) {
    gemm_tile_body<true, 2, false, true>(A, B, C, M, N, K, tiles_m, tiles_n, nullptr, 0, R, RopeEpilogue{}, ldr);
}
__global__ __launch_bounds__(256) void gemm_bf16_tile128(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                         __bf16* __restrict__ C, int M, int N, int K, int tiles_m,
                                                         int tiles_n) {
    gemm_tile_body<false, 2>(A, B, C, M, N, K, tiles_m, tiles_n);
}
__global__ __launch_bounds__(256) void gemm_bf16_tile128_ragged_k(const __bf16* __restrict__ A,
                                                                  const __bf16* __restrict__ B, __bf16* __restrict__ C,
                                                                  int M, int N, int K, int tiles_m, int tiles_n) {
    gemm_tile_body<true, 2>(A, B, C, M, N, K, tiles_m, tiles_n);
}
__global__ __launch_bounds__(256) void gemm_bf16_tile128_splitk(const __bf16* __restrict__ A,
                                                                const __bf16* __restrict__ B, float* __restrict__ W,
                                                                int M, int N, int K, int tiles_m, int tiles_n,
                                                                int kt_per_split) {
    gemm_tile_body<false, 2, true>(A, B, nullptr, M, N, K, tiles_m, tiles_n, W, kt_per_split);
}
__global__ __launch_bounds__(256) void gemm_bf16_tile128_splitk_ragged_k(const __bf16* __restrict__ A,
                                                                         const __bf16* __restrict__ B,
                                                                         float* __restrict__ W, int M, int N, int K,
                                                                         int tiles_m, int tiles_n, int kt_per_split) {
    gemm_tile_body<true, 2, true>(A, B, nullptr, M, N, K, tiles_m, tiles_n, W, kt_per_split);
}
// C[i] = bf16(W[0][i] + W[1][i] + ... + W[splits-1][i]), 8 elements per work-item, partials added
// in the order of their K ranges so the result does not depend on timing.  R, when given, is added to the rounded
// sum and the result rounded again (the bits of the product followed by an elementwise add): a matrix of C's shape
// (r_period 0) or one row repeated every r_period elements (a bias).
template <bool kF16>
__global__ __launch_bounds__(256) void gemm_splitk_reduce(const float* __restrict__ W, __bf16* __restrict__ C, long total,
                                                          int splits, const __bf16* __restrict__ R, long r_period) {
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i >= total) return;
    f32x4 lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = lo;
    for (int s = 0; s < splits; s++) {
        const f32x4* p = reinterpret_cast<const f32x4*>(W + (size_t)s * total + i);
        lo += p[0];
        hi += p[1];
    }
    bf16x4 l = round_to_elem<kF16>(lo), h = round_to_elem<kF16>(hi);
    if (R) {
        const bf16x8 r = *reinterpret_cast<const bf16x8*>(R + (r_period ? i % r_period : i));
        auto widen = [](const bf16x4& v) {
            if constexpr (kF16) return __builtin_convertvector(__builtin_bit_cast(f16x4, v), f32x4);
            else return __builtin_convertvector(v, f32x4);
        };
        l = round_to_elem<kF16>(widen(l) + widen(__builtin_shufflevector(r, r, 0, 1, 2, 3)));
        h = round_to_elem<kF16>(widen(h) + widen(__builtin_shufflevector(r, r, 4, 5, 6, 7)));
    }
    *reinterpret_cast<bf16x8*>(C + i) = __builtin_shufflevector(l, h, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Any shape: one wave per 32x32 output tile, operands fetched straight from global memory
// with bounds checks (zero fill), no LDS.  Correct for every M, N, K; used when the shape
// does not fit the tiled kernel.
template <bool kF16>
__global__ __launch_bounds__(256) void gemm_bf16_generic(const __bf16* __restrict__ A, const __bf16* __restrict__ B,
                                                         __bf16* __restrict__ C, int M, int N, int K, int tiles_n,
                                                         long total_tiles) {
    const int lane = threadIdx.x & 63;
    const long tile = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tile >= total_tiles) return;
    A += (size_t)blockIdx.y * M * K;
    B += (size_t)blockIdx.y * K * N;
    C += (size_t)blockIdx.y * M * N;
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
        if constexpr (kF16) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
        else acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
    }
    // lane l register e: row 8*(e/4) + 4*(l/32) + e%4, column l%32
#pragma unroll
    for (int e = 0; e < 16; e++) {
        const long r = m0 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
        if (r < M && n < N) {
            if constexpr (kF16) C[r * N + n] = __builtin_bit_cast(__bf16, (_Float16)acc[e]);
            else C[r * N + n] = (__bf16)acc[e];
        }
    }
}

}  // namespace mrk::dev

// Split-K partials for callers that cannot allocate: 32 MiB per device, held until the process
// ends.  That is the most plan_split_k ever asks for (at most 256 workgroups in flight, each
// with one 128 x 256 f32 partial tile).  In host code the name is only a handle for
// hipGetSymbolAddress; kernels receive the resolved per-device address as an argument.
static constexpr size_t kStaticWsBytes = size_t(32) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticWsBytes];

namespace mrk {

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_static_ws[kMaxDevices];  // resolved address of `scratch` on each device

// Split-K plan for a shape: how many K ranges and how many 64-deep steps each, or splits = 1
// when the plain tiled kernel already has enough workgroups (or the K loop is too short).
struct SplitPlan {
    long splits = 1, kt_per_split = 0;
};
SplitPlan plan_split_k(long M, long N, long K, long batch) {
    SplitPlan p;
    const long tiles = ((M + 127) / 128) * ((N + 255) / 256) * batch;
    const long kt_all = (K + 63) / 64;
    // at most a quarter of the CUs busy; with up to 64 rows (the weight is streamed once, the partial results are
    // small) up to half of them, and then two or three ranges already pay (16 x 22016 x 4096: 86 tiles)
    const bool few_rows = M <= 64;
    if (K % 8 != 0 || N % 8 != 0 || tiles > (few_rows ? 128 : 64) || kt_all < 8) return p;
    long want = 256 / tiles;                 // ranges that would put one workgroup on every CU
    if (want > kt_all / 2) want = kt_all / 2;  // at least two K steps per range
    // the partial results are written and read back once per range: worth it only while that
    // traffic stays below what the operands themselves move
    const double operand_bytes = 2.0 * batch * ((double)M * K + (double)K * N);
    const long least = few_rows ? 2 : 4;
    while (want >= least && 2.0 * want * batch * M * N * 4.0 > operand_bytes) want--;
    if (want < least) return p;
    p.kt_per_split = (kt_all + want - 1) / want;
    p.splits = (kt_all + p.kt_per_split - 1) / p.kt_per_split;
    if (p.splits < 2) p.splits = 1;
    return p;
}
}  // namespace

size_t gemm_bf16_workspace_bytes(long M, long N, long K, long batch) {
    if (M <= 0 || N <= 0 || K <= 0 || batch <= 0) return 0;
    long ks = 0, kr = 0;
    // a handful of rows: streamed (one row on the vector ALUs where that kernel's plan takes the shape, more on the matrix pipes)
    if (gemm_kn_skinny_plan(M, N, K, batch, &ks, &kr)) return (size_t)ks * M * N * sizeof(float);
    if (gemm_kn_rows_plan(M, N, K, batch, &ks, &kr)) return ks > 1 ? (size_t)ks * M * N * sizeof(float) : 0;
    const SplitPlan p = plan_split_k(M, N, K, batch);
    return p.splits > 1 ? (size_t)p.splits * batch * M * N * sizeof(float) : 0;
}

int gemm_bf16_static_workspace_init(int device_id) {
    if (device_id < 0 || device_id >= kMaxDevices) return (int)hipErrorInvalidDevice;
    if (g_static_ws[device_id].load(std::memory_order_acquire)) return 0;
    void* p = nullptr;  // the array's address on the current device (every device has its own copy)
    hipError_t rc = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (rc != hipSuccess) return (int)rc;
    if (!p || reinterpret_cast<uintptr_t>(p) % 256) return (int)hipErrorInvalidSymbol;
    g_static_ws[device_id].store(p, std::memory_order_release);
    return 0;
}

size_t gemm_bf16_static_workspace_capacity() { return kStaticWsBytes; }

int launch_gemm_bf16_static_ws(void* stream, int device_id, const void* A, const void* B, void* C, long M, long N, long K) {
    if (device_id < 0 || device_id >= kMaxDevices) return (int)hipErrorInvalidDevice;
    const size_t need = gemm_bf16_workspace_bytes(M, N, K, 1);
    if (need > kStaticWsBytes) return (int)hipErrorInvalidValue;
    void* ws = g_static_ws[device_id].load(std::memory_order_acquire);
    if (!ws) return (int)hipErrorNotInitialized;
    // every element of a partial tile that the reduce kernel reads is written by the split
    // kernel of the same call, so nothing has to be cleared between calls
    return launch_gemm_bf16(stream, A, B, C, M, N, K, 0, 1, need ? ws : nullptr, need);
}

bool gemm_bf16_residual_supported(long M, long N, long K, long batch);  // (defined behind tiled_shape)

namespace {
// shapes the tiled kernels address (any M; N and K in whole 16-byte chunks; 32-bit offsets inside a tile)
bool tiled_shape(long M, long N, long K, long batch) {
    if (M <= 0 || N <= 0 || K <= 0 || batch <= 0 || batch > 65535) return false;
    if (M > 0x7fffffffL || N > 0x7fffffffL || N % 8 || K % 8 || K > (1L << 23) || N >= (1L << 25)) return false;
    const long tn = (N + mrk::dev::kBN - 1) / mrk::dev::kBN, tm128 = (M + 127) / 128;
    return tm128 * tn <= 0x7fffffffL;
}
}  // namespace

bool gemm_bf16_residual_supported(long M, long N, long K, long batch) { return tiled_shape(M, N, K, batch); }

bool gemm_bf16_nt_supported(long M, long N, long K, long batch) {
    // the tiled kernels (no any-shape kernel for this operand layout), or the streaming kernels for a
    // handful of rows
    return tiled_shape(M, N, K, batch) || gemm_nt_skinny_supported(M, N, K, batch) || gemm_nt_rows_supported(M, N, K, batch);
}

size_t gemm_bf16_nt_workspace_bytes(long M, long N, long K, long batch) {
    if (M <= 0 || N <= 0 || K <= 0 || batch <= 0) return 0;
    if (gemm_nt_skinny_supported(M, N, K, batch) || gemm_nt_rows_supported(M, N, K, batch)) return 0;  // streamed in one launch
    const SplitPlan p = plan_split_k(M, N, K, batch);
    return p.splits > 1 ? (size_t)p.splits * batch * M * N * sizeof(float) : 0;
}

int launch_gemm_16bit(void* stream, const void* A, const void* B, void* C, long M, long N, long K, int variant, long batch, void* workspace,
                      size_t workspace_bytes, bool b_transposed, bool f16, const void* add, bool add_is_row);

namespace {
// the tiled kernels with the residual epilogue (one pass of output tiles; variant 3 / 4 force the tile)
int launch_tiled_residual(void* stream, const void* A, const void* B, const void* R, void* C, long M, long N, long K, long batch,
                          bool b_transposed, bool r_is_row, int variant) {
    using namespace mrk::dev;
    if (M <= 0 || N <= 0 || batch <= 0) return 0;
    if (!tiled_shape(M, N, K, batch)) return (int)hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(R)) % 16)
        return (int)hipErrorInvalidValue;
    hipStream_t s = static_cast<hipStream_t>(stream);
    (void)hipGetLastError();
    const long tn = (N + kBN - 1) / kBN, tm128 = (M + 127) / 128;
    const bool small = variant == 4 || (variant != 3 && tm128 * tn * batch <= 256);
    const long tm = small ? tm128 : (M + kBM - 1) / kBM;
    const dim3 grid((unsigned)(tm * tn), (unsigned)batch);
    const __bf16* a = static_cast<const __bf16*>(A);
    const __bf16* b = static_cast<const __bf16*>(B);
    const __bf16* r = static_cast<const __bf16*>(R);
    __bf16* c = static_cast<__bf16*>(C);
    const bool ragged_k = K % kBK != 0;
    auto kernel = b_transposed ? (small ? (ragged_k ? gemm_bf16_nt_tile128_residual_ragged_k : gemm_bf16_nt_tile128_residual)
                                        : (ragged_k ? gemm_bf16_nt_tile256_residual_ragged_k : gemm_bf16_nt_tile256_residual))
                               : (small ? (ragged_k ? gemm_bf16_tile128_residual_ragged_k : gemm_bf16_tile128_residual)
                                        : (ragged_k ? gemm_bf16_tile256_residual_ragged_k : gemm_bf16_tile256_residual));
    kernel<<<grid, 256, 0, s>>>(a, b, r, c, (int)M, (int)N, (int)K, (int)tm, (int)tn, r_is_row ? 0 : -1);
    return (int)hipGetLastError();
}
}  // namespace

int launch_gemm_bf16_residual(void* stream, const void* A, const void* B, const void* R, void* C, long M, long N, long K, long batch,
                              bool b_transposed, bool r_is_row, void* workspace, size_t workspace_bytes) {
    if (!R) return (int)hipErrorInvalidValue;
    return launch_gemm_16bit(stream, A, B, C, M, N, K, 0, batch, workspace, workspace_bytes, b_transposed, false, R, r_is_row);
}

bool gemm_bf16_bias_supported(long M, long N, long K, long batch, bool b_transposed) {
    if (M <= 0 || N <= 0 || K <= 0 || batch <= 0) return false;
    return (b_transposed && gemm_nt_bias_streamed(M, N, K, batch)) || tiled_shape(M, N, K, batch);
}

bool gemm_bf16_bias_launchable(long M, long N, long K, long batch, bool b_transposed) { return gemm_bf16_bias_supported(M, N, K, batch, b_transposed); }

int launch_gemm_bf16_bias(void* stream, const void* a, const void* b, const void* bias, void* c, long M, long N, long K, long batch,
                          bool b_transposed, void* workspace, size_t workspace_bytes) {
    return launch_gemm_bf16_residual(stream, a, b, bias, c, M, N, K, batch, b_transposed, true, workspace, workspace_bytes);
}

bool gemm_bf16_swiglu_supported(long M, long F, long K, bool b_transposed) {
    if (M <= 0 || F <= 0 || K <= 0) return false;
    // [2F, K] form: the up rows are addressed F rows behind the gate rows with 32-bit byte offsets
    if (b_transposed && (F + 256) * K * 2 >= (1L << 32)) return false;
    if (M > 0x7fffffffL || F % 8 || K % 8 || K > (1L << 23) || 2 * F >= (1L << 25)) return false;
    const long tn = (F + 127) / 128, tm = (M + mrk::dev::kBM - 1) / mrk::dev::kBM;
    return tm * tn <= 0x7fffffffL;
}

int launch_gemm_bf16_swiglu(void* stream, const void* A, const void* B, void* C, long M, long F, long K, bool b_transposed) {
    using namespace mrk::dev;
    if (M <= 0 || F <= 0) return 0;
    if (!gemm_bf16_swiglu_supported(M, F, K, b_transposed)) return (int)hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(C)) % 16) return (int)hipErrorInvalidValue;
    // a handful of rows against a [2F, K] weight: the gated form of the streaming kernel
    if (b_transposed && gemm_nt_swiglu_streamed(M, F, K)) return launch_gemm_nt_swiglu_streamed(stream, A, B, C, M, F, K);
    hipStream_t s = static_cast<hipStream_t>(stream);
    (void)hipGetLastError();
    const long tn = (F + 127) / 128, tm = (M + kBM - 1) / kBM;
    const dim3 grid((unsigned)(tm * tn), 1);
    const __bf16* a = static_cast<const __bf16*>(A);
    const __bf16* b = static_cast<const __bf16*>(B);
    __bf16* c = static_cast<__bf16*>(C);
    const bool ragged_k = K % kBK != 0;
    auto kernel = b_transposed ? (ragged_k ? gemm_bf16_nt_tile256_swiglu_ragged_k : gemm_bf16_nt_tile256_swiglu)
                               : (ragged_k ? gemm_bf16_tile256_swiglu_ragged_k : gemm_bf16_tile256_swiglu);
    kernel<<<grid, 256, 0, s>>>(a, b, c, (int)M, (int)(2 * F), (int)K, (int)tm, (int)tn);
    return (int)hipGetLastError();
}

bool gemm_bf16_rope_supported(long M, long N, long K, long split, long seq) {
    using namespace mrk::dev;
    return M > 0 && N > 0 && K > 0 && seq > 0 && K % kBK == 0 && N % 8 == 0 && split > 0 && split <= N && split % kBN == 0 &&
           M <= 0x7fffffffL && N < (1L << 25) && K <= (1L << 23) && ((M + kBM - 1) / kBM) * ((N + kBN - 1) / kBN) <= 0x7fffffffL;
}

int launch_gemm_bf16_rope(void* stream, const void* A, const void* B, void* C_rot, void* C_rest, long M, long N, long K, long split,
                          const void* cos, const void* sin, long seq, bool b_transposed) {
    using namespace mrk::dev;
    if (!gemm_bf16_rope_supported(M, N, K, split, seq) || !A || !B || !C_rot || !cos || !sin || (split < N && !C_rest))
        return (int)hipErrorInvalidValue;
    const uintptr_t all = reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(C_rot) |
                          reinterpret_cast<uintptr_t>(C_rest) | reinterpret_cast<uintptr_t>(cos) | reinterpret_cast<uintptr_t>(sin);
    if (all % 16 || reinterpret_cast<uintptr_t>(cos) % 32 || reinterpret_cast<uintptr_t>(sin) % 32) return (int)hipErrorInvalidValue;
    (void)hipGetLastError();
    const long tm = (M + kBM - 1) / kBM, tn = (N + kBN - 1) / kBN;
    RopeEpilogue rope{static_cast<const float*>(cos), static_cast<const float*>(sin), static_cast<__bf16*>(C_rest), (int)seq, (int)split};
    auto kernel = b_transposed ? gemm_bf16_nt_tile256_rope : gemm_bf16_tile256_rope;
    kernel<<<dim3((unsigned)(tm * tn)), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const __bf16*>(A), static_cast<const __bf16*>(B), static_cast<__bf16*>(C_rot), (int)M, (int)N, (int)K, (int)tm, (int)tn, rope);
    return (int)hipGetLastError();
}

namespace {
int launch_tiled_residual(void* stream, const void* A, const void* B, const void* R, void* C, long M, long N, long K, long batch,
                          bool b_transposed, bool r_is_row, int variant);
}

// The product, with `add` (a matrix of C's shape or, add_is_row, one row [N]; bf16) added to the rounded result by
// whichever kernel writes it: the streaming kernels, the split-K reduction or the tiled kernels' residual epilogue.
int launch_gemm_16bit(void* stream, const void* A, const void* B, void* C, long M, long N, long K, int variant, long batch, void* workspace,
                      size_t workspace_bytes, bool b_transposed, bool f16, const void* add, bool add_is_row) {
    using namespace mrk::dev;
    if (M <= 0 || N <= 0 || batch <= 0) return 0;
    if (add && reinterpret_cast<uintptr_t>(add) % 16) return (int)hipErrorInvalidValue;
    const __bf16* addp = static_cast<const __bf16*>(add);
    const long add_period = add_is_row ? N : 0;
    if (batch > 65535) return (int)hipErrorInvalidValue;  // grid y extent
    if (M > 0x7fffffffL || N > 0x7fffffffL || K > 0x7fffffffL || K < 0) return (int)hipErrorInvalidValue;
    hipStream_t s = static_cast<hipStream_t>(stream);
    (void)hipGetLastError();
    const bool aligned = ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(C)) % 16) == 0;
    // the tiled kernel addresses a tile's rows with 32-bit byte offsets from the tile origin:
    // 255 rows of A (K elements each) and 49 rows of B (N elements each) must stay below 4 GiB
    const bool offsets_fit = K <= (1L << 23) && N < (1L << 25);
    if (b_transposed) {
        // B given as Bt[N, K]: the tiled kernels, or nothing (variant 3 / 4 force a tile size)
        if (!aligned || !gemm_bf16_nt_supported(M, N, K, batch)) return (int)hipErrorInvalidValue;
        const bool choose = variant == 0 || variant == 5;  // 3 / 4 force a tile where the shape has one
        const bool tiled = tiled_shape(M, N, K, batch);
        // up to 64 rows: one pass over the weight streams it faster than any tile (one or two rows on the
        // vector ALUs, more on the matrix pipes with 16-row blocks staged through LDS)
        if (choose || !tiled) {
            if (add) {
                if (gemm_nt_bias_streamed(M, N, K, batch)) return launch_gemm_nt_bias_streamed(stream, A, B, add, C, M, N, K, f16, add_is_row);
            } else {
                if (gemm_nt_skinny_supported(M, N, K, batch)) return launch_gemm_nt_skinny(stream, A, B, C, M, N, K, batch, f16);
                if (gemm_nt_rows_supported(M, N, K, batch)) return launch_gemm_nt_rows(stream, A, B, C, M, N, K, batch, f16);
            }
        }
        if (!tiled) return (int)hipErrorInvalidValue;
        const long tn = (N + kBN - 1) / kBN, tm128 = (M + 127) / 128;
        const SplitPlan sp = choose ? plan_split_k(M, N, K, batch) : SplitPlan();
        if (sp.splits > 1) {
            // few output tiles against a long K: the K loop spread over the chip when the caller
            // brought the workspace for the partial results
            // (without one the plain tiled kernel runs on the few workgroups it has)
            if (workspace && workspace_bytes >= (size_t)sp.splits * batch * M * N * sizeof(float) &&
                reinterpret_cast<uintptr_t>(workspace) % 16 == 0 && batch * sp.splits <= 65535) {
                const dim3 grid((unsigned)(tm128 * tn), (unsigned)batch, (unsigned)sp.splits);
                float* w = static_cast<float*>(workspace);
                auto split_kernel = f16 ? (K % kBK == 0 ? gemm_f16_nt_tile128_splitk : gemm_f16_nt_tile128_splitk_ragged_k)
                                        : (K % kBK == 0 ? gemm_bf16_nt_tile128_splitk : gemm_bf16_nt_tile128_splitk_ragged_k);
                split_kernel<<<grid, 256, 0, s>>>(static_cast<const __bf16*>(A), static_cast<const __bf16*>(B), w, (int)M, (int)N, (int)K,
                                                  (int)tm128, (int)tn, (int)sp.kt_per_split);
                const long total = batch * M * N;
                auto reduce_kernel = f16 ? gemm_splitk_reduce<true> : gemm_splitk_reduce<false>;
                reduce_kernel<<<(unsigned)((total / 8 + 255) / 256), 256, 0, s>>>(w, static_cast<__bf16*>(C), total, (int)sp.splits, addp, add_period);
                return (int)hipGetLastError();
            }
        }
        if (add) return f16 ? (int)hipErrorInvalidValue : launch_tiled_residual(stream, A, B, add, C, M, N, K, batch, true, add_is_row, variant);
        const bool small = variant == 4 || (variant != 3 && tm128 * tn * batch <= 256);
        const long tm = small ? tm128 : (M + kBM - 1) / kBM;
        const bool ragged_k = K % kBK != 0;
        auto kernel = f16 ? (small ? (ragged_k ? gemm_f16_nt_tile128_ragged_k : gemm_f16_nt_tile128)
                                   : (ragged_k ? gemm_f16_nt_tile256_ragged_k : gemm_f16_nt_tile256))
                          : (small ? (ragged_k ? gemm_bf16_nt_tile128_ragged_k : gemm_bf16_nt_tile128)
                                   : (ragged_k ? gemm_bf16_nt_tile256_ragged_k : gemm_bf16_nt_tile256));
        kernel<<<dim3((unsigned)(tm * tn), (unsigned)batch), 256, 0, s>>>(static_cast<const __bf16*>(A), static_cast<const __bf16*>(B),
                                                                          static_cast<__bf16*>(C), (int)M, (int)N, (int)K, (int)tm, (int)tn);
        return (int)hipGetLastError();
    }
    // up to 16 rows: one streaming pass over the weight into f32 partial sums, then their sum
    {
        long ks = 0, kr = 0;
        if ((variant == 0 || variant == 5) && aligned && gemm_kn_skinny_plan(M, N, K, batch, &ks, &kr) && workspace &&
            workspace_bytes >= (size_t)ks * M * N * sizeof(float) && reinterpret_cast<uintptr_t>(workspace) % 16 == 0) {
            return launch_gemm_kn_skinny(stream, A, B, C, workspace, M, N, K, ks, kr, f16, add, add_is_row);
        }
        if ((variant == 0 || variant == 5) && aligned && gemm_kn_rows_plan(M, N, K, batch, &ks, &kr) &&
            (ks == 1 || (workspace && workspace_bytes >= (size_t)ks * M * N * sizeof(float) && reinterpret_cast<uintptr_t>(workspace) % 16 == 0))) {
            return launch_gemm_kn_rows(stream, A, B, C, workspace, M, N, K, ks, kr, f16, add, add_is_row);
        }
    }
    // any M; N and K in whole 16-byte chunks
    if (variant != 2 && aligned && offsets_fit && K > 0 && N % 8 == 0 && K % 8 == 0) {
        const long tn = (N + kBN - 1) / kBN;
        const long tm128 = (M + 127) / 128;
        // a handful of rows against a large weight matrix: spread the K loop over the chip when
        // the caller brought the workspace for the partial results
        const SplitPlan sp = variant == 0 || variant == 5 ? plan_split_k(M, N, K, batch) : SplitPlan();
        if (sp.splits > 1 && workspace && workspace_bytes >= (size_t)sp.splits * batch * M * N * sizeof(float) &&
            reinterpret_cast<uintptr_t>(workspace) % 16 == 0 && batch * sp.splits <= 65535) {
            const dim3 grid((unsigned)(tm128 * tn), (unsigned)batch, (unsigned)sp.splits);
            float* w = static_cast<float*>(workspace);
            const __bf16* a = static_cast<const __bf16*>(A);
            const __bf16* b = static_cast<const __bf16*>(B);
            auto split_kernel = f16 ? (K % kBK == 0 ? gemm_f16_tile128_splitk : gemm_f16_tile128_splitk_ragged_k)
                                    : (K % kBK == 0 ? gemm_bf16_tile128_splitk : gemm_bf16_tile128_splitk_ragged_k);
            split_kernel<<<grid, 256, 0, s>>>(a, b, w, (int)M, (int)N, (int)K, (int)tm128, (int)tn, (int)sp.kt_per_split);
            const long total = batch * M * N;
            auto reduce_kernel = f16 ? gemm_splitk_reduce<true> : gemm_splitk_reduce<false>;
            reduce_kernel<<<(unsigned)((total / 8 + 255) / 256), 256, 0, s>>>(w, static_cast<__bf16*>(C), total, (int)sp.splits, addp, add_period);
            return (int)hipGetLastError();
        }
        // variant 0: the 128-row tile when all its workgroups are resident at once (at most one per
        // compute unit): twice the workgroups of the 256-row tile for the same work.  3 / 4 force one.
        if (add) return f16 ? (int)hipErrorInvalidValue : launch_tiled_residual(stream, A, B, add, C, M, N, K, batch, false, add_is_row, variant);
        const bool small = variant == 4 || (variant != 3 && tm128 * tn * batch <= 256);
        const long tm = small ? tm128 : (M + kBM - 1) / kBM;
        if (tm * tn > 0x7fffffffL) return (int)hipErrorInvalidValue;
        const dim3 grid((unsigned)(tm * tn), (unsigned)batch);
        const __bf16* a = static_cast<const __bf16*>(A);
        const __bf16* b = static_cast<const __bf16*>(B);
        __bf16* c = static_cast<__bf16*>(C);
        const bool ragged_k = K % kBK != 0;
        auto kernel = f16 ? (small ? (ragged_k ? gemm_f16_tile128_ragged_k : gemm_f16_tile128)
                                   : (ragged_k ? gemm_f16_tile256_ragged_k : gemm_f16_tile256))
                          : (small ? (ragged_k ? gemm_bf16_tile128_ragged_k : gemm_bf16_tile128)
                                   : (ragged_k ? gemm_bf16_tile256_ragged_k : gemm_bf16_tile256));
        kernel<<<grid, 256, 0, s>>>(a, b, c, (int)M, (int)N, (int)K, (int)tm, (int)tn);
    } else {
        if (add) return (int)hipErrorInvalidValue;  // (the any-shape kernel has no epilogue)
        const long tm = (M + 31) / 32, tn = (N + 31) / 32;
        const long total = tm * tn;
        const long blocks = (total + 3) / 4;
        if (blocks > 0x7fffffffL) return (int)hipErrorInvalidValue;
        auto generic = f16 ? gemm_bf16_generic<true> : gemm_bf16_generic<false>;
        generic<<<dim3((unsigned)blocks, (unsigned)batch), 256, 0, s>>>(static_cast<const __bf16*>(A), static_cast<const __bf16*>(B),
                                                           static_cast<__bf16*>(C), (int)M, (int)N, (int)K, (int)tn,
                                                           total);
    }
    return (int)hipGetLastError();
}

int launch_gemm_bf16(void* stream, const void* A, const void* B, void* C, long M, long N, long K, int variant, long batch, void* workspace,
                     size_t workspace_bytes, bool b_transposed, bool f16) {
    return launch_gemm_16bit(stream, A, B, C, M, N, K, variant, batch, workspace, workspace_bytes, b_transposed, f16, nullptr, false);
}

}  // namespace mrk

