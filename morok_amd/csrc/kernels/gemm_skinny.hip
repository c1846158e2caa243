// C[M, N] = A[M, K] @ Bt[N, K]^T for a handful of rows (M <= 64) against a weight stored as a Linear
// layer keeps it ([out_features, in_features], tensor/src/nn/linear.rs:9-14,39-41): the decode step
// of a language model.  The product is a stream over the weight: 2 * N * K bytes against 2 * M * N * K
// flops, HBM-bound for these M.  Two kernels: gemm_nt_skinny for one and two rows on the vector ALUs,
// gemm_nt_rows for 3 to 64 rows on the matrix pipes (further down, with the [K, N] form for one and two rows).
// gemm_nt_skinny: a workgroup of four waves
// owns two or four weight rows; the waves take the 512-element chunks of K in turn, a lane loads
// 16 bytes of each of the rows (a wave reads 1 KB of one row per instruction) and of each row of A
// (cache hits: every workgroup reads the same few KB, each starting at another chunk so that they
// do not all queue on the same L2 channel), and multiplies with packed two-element dot products
// (v_dot2c_f32_bf16 / _f16: exact products, f32 accumulation).  The lanes' partial sums are folded
// with a transposing butterfly (after step s a lane keeps half of the values it held, summed with
// its partner's: V values take V - 1 exchanges in all, not 6 each), the four waves' results meet in
// LDS, wave 0 adds them in a fixed order and writes the outputs.  One launch, no scratch memory, no
// atomics: results do not depend on scheduling.  (A lane needs its own 16 bytes of every row of A per
// 16 bytes of a weight row, so the cache traffic grows with M: 6.2 TB/s of weight for one row, 5.9 for
// two, 4.5 for eight, which is where the matrix-pipe kernel takes over.)
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
// The element a kernel writes: the sum rounded to the result's type; with an addend (a bias row or a matrix of the
// result's shape, of the result's type) that rounded value plus the addend, rounded again (the bits of the product
// followed by the add).  `add` points at the addend's row, or is null.
template <bool kF16>
__device__ __forceinline__ unsigned short round_out(float s, const unsigned short* add, long n) {
    if constexpr (kF16) {
        _Float16 h = (_Float16)s;
        if (add) h = (_Float16)((float)h + (float)__builtin_bit_cast(_Float16, add[n]));
        return __builtin_bit_cast(unsigned short, h);
    } else {
        unsigned short h = round_bf16(s);
        if (add) h = round_bf16(__builtin_bit_cast(float, (unsigned)h << 16) + __builtin_bit_cast(float, (unsigned)add[n] << 16));
        return h;
    }
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
                                                       unsigned short* __restrict__ C, int M, int N, int K,
                                                       const unsigned short* __restrict__ add, long add_pitch) {
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
            C[(size_t)m * N + n0 + r] = round_out<kF16>(s, add ? add + (size_t)m * add_pitch : nullptr, n0 + r);
        }
    }
}


// The same product for 3 to 64 rows of A, on the matrix pipes.  v_mfma_f32_16x16x32 takes, per lane, eight
// consecutive k of one row of each operand (lane l: row l % 16, k 8 * (l / 16) ...), i.e. 16 rows with 64 bytes
// each per instruction if it were loaded straight from memory; the vector-memory path serves such row gathers at
// a fraction of its rate for consecutive bytes.  So both operands go through LDS: a wave copies its chunk (64
// elements of K) of 16-row blocks with direct global -> LDS loads, 1 KB per instruction = eight rows of 128
// bytes, the weight's with the non-temporal hint (it is read once; A stays in L2), and reads the fragments back
// with ds_read_b128.  The 16-byte pieces of a row are stored swizzled by the row (piece p of row r at position
// p ^ ((r >> 1) & 7): the 16 rows a fragment read touches then fall into 16 different bank groups).  The region
// is private to the wave, so the loop has no barrier; the waves of a workgroup take the chunks of K in turn
// (every workgroup starting at another one, as above), each holds kRT x kMT accumulator blocks for the
// workgroup's 16 * kRT weight rows, and their sums meet in LDS at the end and are added in a fixed order.
// What bounds the rate is the number of weight bytes in flight per CU, which is what the LDS holds: with one
// chunk per wave in flight, 8 or 16 waves per workgroup and enough workgroups resident the weight streams at
// 5.6-6.5 TB/s for up to 32 rows of A.  kMT: 16-row blocks of A (M <= 16 * kMT; rows beyond M repeat row M - 1
// and are not written); kRT: 16-row blocks of the weight per workgroup.  grid = (ceil(N / (16 kRT)), batch).
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

#define MRK_LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

template <int kMT, int kRT, int kWaves, bool kF16, bool kGate = false>
__global__ __launch_bounds__(kWaves * 64) void gemm_nt_rows(const unsigned short* __restrict__ A, const unsigned short* __restrict__ Bt,
                                                             unsigned short* __restrict__ C, int M, int N, int K,
                                                             const unsigned short* __restrict__ add, long add_pitch) {
    constexpr int kSteps = 2;                      // 32-deep matrix steps per chunk
    constexpr int kPieces = 4 * kSteps;            // 16-byte pieces of a row per chunk
    constexpr int kRowsPerCopy = 64 / kPieces;     // rows one copy instruction covers
    constexpr int kCopies = 16 / kRowsPerCopy;     // copy instructions per 16-row block
    constexpr int kBlockBytes = 16 * kPieces * 16; // one block's chunk in LDS
    // kGate: the weight is [2 N, K], gate rows first; the workgroup owns kRT blocks of gate rows and the kRT blocks of up
    // rows N rows further down, and writes C[M, N] = silu(a gate) * (a up) (see the end of the kernel)
    constexpr int kWB = kGate ? 2 * kRT : kRT;     // weight blocks per workgroup
    constexpr int kWaveBytes = (kWB + kMT) * kBlockBytes;
    constexpr int kTiles = kWB * kMT;
    constexpr int kSumBytes = kWaves * kTiles * 1024;
    constexpr int kLds = kWaves * kWaveBytes > kSumBytes ? kWaves * kWaveBytes : kSumBytes;
    static_assert(kLds <= 160 * 1024, "LDS");
    __shared__ __attribute__((aligned(1024))) char smem[kLds];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 15, g = lane >> 4;
    const long n0 = (long)blockIdx.x * (16 * kRT);
    A += (size_t)blockIdx.y * M * K;
    Bt += (size_t)blockIdx.y * (kGate ? 2 : 1) * N * K;
    C += (size_t)blockIdx.y * M * N;
    const char* w_base = reinterpret_cast<const char*>(Bt + (size_t)n0 * K);
    const char* a_base = reinterpret_cast<const char*>(A);
    const unsigned lds_wave = (unsigned)(uintptr_t)MRK_LDS_PTR(char, smem) + wave * kWaveBytes;
    // copy side: lane -> (row of the copy, position in the row); byte offsets of its rows from the bases
    const int pos = lane % kPieces, rsub = lane / kPieces;
    unsigned w_off[kWB][kCopies], a_off[kMT][kCopies], piece_of[kCopies];
#pragma unroll
    for (int i = 0; i < kCopies; i++) {
        const int r = i * kRowsPerCopy + rsub;
        piece_of[i] = (unsigned)(pos ^ ((r >> 1) & 7));
#pragma unroll
        for (int t = 0; t < kWB; t++) {
            long n = n0 + (t % kRT) * 16 + r;
            n = n < N ? n : N - 1;  // a row past the end repeats the last one (not written)
            w_off[t][i] = (unsigned)(n - n0 + (t >= kRT ? N : 0)) * (unsigned)K * 2u;
        }
#pragma unroll
        for (int t = 0; t < kMT; t++) {
            int m = t * 16 + r;
            m = m < M ? m : M - 1;
            a_off[t][i] = (unsigned)m * (unsigned)K * 2u;
        }
    }
    f32x4 acc[kWB][kMT];
#pragma unroll
    for (int r = 0; r < kWB; r++)
#pragma unroll
        for (int m = 0; m < kMT; m++) acc[r][m] = f32x4{0.f, 0.f, 0.f, 0.f};
    // read side: row li of a block, piece 4 s + g of the chunk at position (4 s + g) ^ key(li)
    const unsigned rd_row = lds_wave + li * (kPieces * 16);
    const unsigned gx = (unsigned)(g ^ ((li >> 1) & 7));
    const int pieces = K >> 3;
    const int chunks = (pieces + kPieces - 1) / kPieces;
    const int first = (int)(blockIdx.x % (unsigned)chunks);
    for (int c = wave; c < chunks; c += kWaves) {
        int cc = c + first;
        if (cc >= chunks) cc -= chunks;
        const int p0 = cc * kPieces;
        const bool full = p0 + kPieces <= pieces;  // else the last chunk of a K that is no multiple of 64
        // (the previous chunk's fragment reads have all been consumed by matrix instructions; the wait makes that
        // explicit before the copies may overwrite them)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < kCopies; i++) {
            unsigned piece = (unsigned)p0 + piece_of[i];
            if (!full) piece = piece < (unsigned)pieces ? piece : (unsigned)pieces - 1u;  // any valid piece: zeroed below
#pragma unroll
            for (int t = 0; t < kWB; t++)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                             :
                             : "s"(lds_wave + t * kBlockBytes + i * 1024), "v"(w_off[t][i] + piece * 16u), "s"(w_base)
                             : "m0", "memory");
#pragma unroll
            for (int t = 0; t < kMT; t++)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             :
                             : "s"(lds_wave + (kWB + t) * kBlockBytes + i * 1024), "v"(a_off[t][i] + piece * 16u), "s"(a_base)
                             : "m0", "memory");
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            const unsigned po = (((unsigned)(4 * s)) ^ gx) * 16u;
            const bool in = full || p0 + 4 * s + g < pieces;
            u32x4 x[kMT];
#pragma unroll
            for (int t = 0; t < kMT; t++) {
                x[t] = *MRK_LDS_PTR(u32x4, rd_row + (kWB + t) * kBlockBytes + po);
                if (!full) x[t] = in ? x[t] : u32x4{0u, 0u, 0u, 0u};
            }
#pragma unroll
            for (int r = 0; r < kWB; r++) {
                u32x4 w = *MRK_LDS_PTR(u32x4, rd_row + r * kBlockBytes + po);
                if (!full) w = in ? w : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
                for (int t = 0; t < kMT; t++) {
                    if constexpr (kF16)
                        acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, w), __builtin_bit_cast(f16x8, x[t]), acc[r][t], 0, 0, 0);
                    else
                        acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, x[t]), acc[r][t], 0, 0, 0);
                }
            }
        }
    }
    // the waves' partial blocks meet in LDS (over the copy regions, hence the first barrier); a lane of the matrix
    // result holds four consecutive weight rows for one row of A, i.e. four consecutive elements of a row of C
    __syncthreads();
    f32x4* partial = reinterpret_cast<f32x4*>(smem);  // [kWaves][kTiles][64]
#pragma unroll
    for (int r = 0; r < kWB; r++)
#pragma unroll
        for (int m = 0; m < kMT; m++) partial[(wave * kTiles + r * kMT + m) * 64 + lane] = acc[r][m];
    __syncthreads();
    const bool vec = (N & 3) == 0;
    for (int e = threadIdx.x; e < kRT * kMT * 64; e += kWaves * 64) {
        const int tile = e >> 6, l = e & 63;
        f32x4 s = partial[tile * 64 + l];
#pragma unroll
        for (int w = 1; w < kWaves; w++) s += partial[(w * kTiles + tile) * 64 + l];
        const int r = tile / kMT, m = (tile % kMT) * 16 + (l & 15);
        const long n = n0 + r * 16 + 4 * (l >> 4);
        if (m >= M || n >= N) continue;
        unsigned short o[4];
        if constexpr (kGate) {
            // the up block's sums, then x * sigmoid(x) * y on the two products rounded as separate kernels would leave them,
            // in f32 with one rounding: the arithmetic of the generated elementwise kernel this replaces
            f32x4 u = partial[(tile + kRT * kMT) * 64 + l];
#pragma unroll
            for (int w = 1; w < kWaves; w++) u += partial[(w * kTiles + tile + kRT * kMT) * 64 + l];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float g = __builtin_bit_cast(float, (unsigned)round_bf16(s[i]) << 16);
                const float y = __builtin_bit_cast(float, (unsigned)round_bf16(u[i]) << 16);
                o[i] = round_bf16((g * (1.0f / (1.0f + exp2f(g * -1.44269502f)))) * y);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] = round_out<kF16>(s[i], add && n + i < N ? add + (size_t)m * add_pitch : nullptr, n + i);
        }
        unsigned short* dst = C + (size_t)m * N + n;
        if (vec) {
            *reinterpret_cast<u32x2*>(dst) = u32x2{(unsigned)o[0] | ((unsigned)o[1] << 16), (unsigned)o[2] | ((unsigned)o[3] << 16)};
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (n + i < N) dst[i] = o[i];
        }
    }
}


// C[M, N] = A[M, K] @ B[K, N] for one row (the template takes up to eight) with the weight stored [K, N]: the first of two
// kernels, which streams the weight once and leaves f32 partial sums (the tiled kernels' split-K
// reduction adds them up and rounds).  A lane owns eight consecutive columns, a wave 512; the
// workgroups split K (blockIdx.y: rows_per_group consecutive k-rows each, a multiple of 32) and a
// workgroup's four waves split its rows into four consecutive runs.  A wave reads 1 KB of one
// k-row per instruction, eight rows per step; two rows' columns are interleaved into (k, k + 1)
// pairs (v_perm_b32) and multiplied with the matching pair of A, which is wave-uniform and comes
// through scalar loads, by the packed dot product.  The waves' sums meet in LDS and the workgroup
// writes one f32 partial row block W[blockIdx.y][m][its 512 columns].
template <int kM, bool kF16>
__global__ __launch_bounds__(256) void gemm_kn_skinny_partial(const unsigned short* __restrict__ A, const unsigned short* __restrict__ B,
                                                               float* __restrict__ W, int M, int N, int K, int rows_per_group) {
    __shared__ float red[4][kM][512];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const long col0 = (long)blockIdx.x * 512 + lane * 8;
    const bool active = col0 < N;                              // N is a multiple of 8: a lane's columns are all inside or all outside
    const long col = active ? col0 : 0;
    const int k_begin = blockIdx.y * rows_per_group;
    const int k_end = k_begin + rows_per_group < K ? k_begin + rows_per_group : K;
    const int per_wave = rows_per_group >> 2;                  // a multiple of 8
    int k = k_begin + wave * per_wave;
    int kw_end = k + per_wave;
    kw_end = kw_end < k_end ? kw_end : k_end;                  // (K is a multiple of 8, so runs end on even rows)
    const unsigned* a32[kM];                                   // rows of A as (k, k + 1) pairs
#pragma unroll
    for (int m = 0; m < kM; m++) a32[m] = reinterpret_cast<const unsigned*>(A + (size_t)(m < M ? m : M - 1) * K);
    float acc[kM][8];
#pragma unroll
    for (int m = 0; m < kM; m++)
#pragma unroll
        for (int c = 0; c < 8; c++) acc[m][c] = 0.0f;
    // two k-rows' eight columns -> eight (k, k + 1) pairs, multiplied with A's pair of every row
    auto pair_rows = [&](const u32x4& lo, const u32x4& hi, int kk) {
        unsigned pr[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            pr[2 * i] = __builtin_amdgcn_perm(hi[i], lo[i], 0x05040100u);
            pr[2 * i + 1] = __builtin_amdgcn_perm(hi[i], lo[i], 0x07060302u);
        }
#pragma unroll
        for (int m = 0; m < kM; m++) {
            const unsigned xp = a32[m][kk >> 1];               // wave-uniform
#pragma unroll
            for (int c = 0; c < 8; c++) acc[m][c] = dot2<kF16>(xp, pr[c], acc[m][c]);
        }
    };
    const u32x4* b_col = reinterpret_cast<const u32x4*>(B + col);  // + k * N / 8 per row
    const size_t row_stride = (size_t)N >> 3;                        // in 16-byte words
    for (; k + 8 <= kw_end; k += 8) {
        // the step's four pairs of every row of A in one scalar load each (k is a multiple of 8 here: 16-byte aligned)
        u32x4 xq[kM];
#pragma unroll
        for (int m = 0; m < kM; m++) xq[m] = *reinterpret_cast<const u32x4*>(a32[m] + (k >> 1));
        u32x4 r[8];
#pragma unroll
        for (int j = 0; j < 8; j++) r[j] = __builtin_nontemporal_load(b_col + (size_t)(k + j) * row_stride);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            unsigned pr[8];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                pr[2 * i] = __builtin_amdgcn_perm(r[2 * j + 1][i], r[2 * j][i], 0x05040100u);
                pr[2 * i + 1] = __builtin_amdgcn_perm(r[2 * j + 1][i], r[2 * j][i], 0x07060302u);
            }
#pragma unroll
            for (int m = 0; m < kM; m++)
#pragma unroll
                for (int c = 0; c < 8; c++) acc[m][c] = dot2<kF16>(xq[m][j], pr[c], acc[m][c]);
        }
    }
    for (; k + 2 <= kw_end; k += 2) {
        const u32x4 lo = __builtin_nontemporal_load(b_col + (size_t)k * row_stride);
        const u32x4 hi = __builtin_nontemporal_load(b_col + (size_t)(k + 1) * row_stride);
        pair_rows(lo, hi, k);
    }
#pragma unroll
    for (int m = 0; m < kM; m++)
#pragma unroll
        for (int c = 0; c < 8; c += 4)
            *reinterpret_cast<float4*>(&red[wave][m][lane * 8 + c]) = make_float4(acc[m][c], acc[m][c + 1], acc[m][c + 2], acc[m][c + 3]);
    __syncthreads();
    // 256 work-items add the four waves' sums: element e = m * 512 + column, two columns apart per step
    for (int e = threadIdx.x; e < kM * 512; e += 256) {
        const int m = e >> 9, c = e & 511;
        const long n = (long)blockIdx.x * 512 + c;
        if (m < M && n < N) W[((size_t)blockIdx.y * M + m) * N + n] = ((red[0][m][c] + red[1][m][c]) + red[2][m][c]) + red[3][m][c];
    }
}


// 2 to 16 rows (to 64 against a narrow weight) against a weight stored [K, N], on the matrix pipes: the matrix instruction wants eight consecutive k
// of one weight column per lane, and in this layout consecutive bytes are consecutive columns, so the weight goes
// through LDS and comes back through the transposing read.  A workgroup of eight waves owns 64 * kCB columns and
// (blockIdx.y) a range of K; the waves take the range's 32-row chunks in turn.  A wave copies its chunk with direct
// global -> LDS loads (1 KB per instruction = eight k-rows x 128 bytes, non-temporal), the 32-byte granules (16
// columns) of a k-row stored at granule ^ f(k-row) with f = bit 1 | bit 3 << 1 of the row, so that the rows a
// transposing read touches in one pass fall into different banks; ds_read_b64_tr_b16 then hands lane j of a
// 16-lane block column j's four k (two reads: eight), which is the matrix instruction's operand.  A's fragment
// (16 rows x 64 bytes, cache hits) is loaded straight from memory.  The region is private to the wave: no barrier
// in the loop.  The waves' sums meet in LDS; the workgroup writes f32 partial sums W[blockIdx.y][M][N] for
// gemm_kn_rows_reduce, or with a single K range the rounded result.
template <int kMT, int kCB, bool kF16>
__global__ __launch_bounds__(512) void gemm_kn_rows(const unsigned short* __restrict__ A, const unsigned short* __restrict__ B,
                                                    unsigned short* __restrict__ C, float* __restrict__ W, int M, int N, int K, int k_per_split,
                                                    const unsigned short* __restrict__ add, long add_pitch) {
    constexpr int kWaves = 8;
    constexpr int kBlockBytes = 32 * 128;  // 32 k-rows x 64 columns
    constexpr int kWaveBytes = kCB * kBlockBytes;
    constexpr int kTiles = kCB * 4 * kMT;  // 16 x 16 accumulator blocks per wave
    constexpr int kSumBytes = kWaves * kTiles * 1024;
    constexpr int kLds = kWaves * kWaveBytes > kSumBytes ? kWaves * kWaveBytes : kSumBytes;
    __shared__ __attribute__((aligned(1024))) char smem[kLds];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const long n0 = (long)blockIdx.x * (64 * kCB);
    const int k_begin = blockIdx.y * k_per_split;
    const int k_end = k_begin + k_per_split < K ? k_begin + k_per_split : K;
    const unsigned lds_wave = (unsigned)(uintptr_t)MRK_LDS_PTR(char, smem) + wave * kWaveBytes;
    // copy side: copy i of a block covers k-rows 8 i .. 8 i + 7; lane -> k-row 8 i + lane / 8, position lane % 8 of the row
    const int prow = lane >> 3, ppos = lane & 7;
    unsigned b_off[kCB][4];  // byte offset from (the chunk's first k-row, column n0)
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int kr = 8 * i + prow;
        const int f = ((kr >> 1) & 1) | (((kr >> 3) & 1) << 1);
        const int q = (((ppos >> 1) ^ f) << 1) | (ppos & 1);  // 16-byte piece of the row this lane fetches
#pragma unroll
        for (int c = 0; c < kCB; c++) {
            long col = n0 + c * 64 + q * 8;
            col = col < N ? col : N - 8;  // a piece past the end repeats the last one (not written)
            b_off[c][i] = (unsigned)kr * (unsigned)N * 2u + (unsigned)(col - n0) * 2u;
        }
    }
    // read side: 16-lane block blk covers k-rows 8 blk .. 8 blk + 7 in two reads of four; lane jl of the block points
    // at k-row jl / 4 of the four, 8-byte unit jl % 4 of the column block's granule
    const int jl = lane & 15, blk = lane >> 4;
    const int fr = ((jl >> 3) & 1) | ((blk & 1) << 1);
    unsigned rd[4];
#pragma unroll
    for (int c4 = 0; c4 < 4; c4++) rd[c4] = lds_wave + (8 * blk + (jl >> 2)) * 128 + ((c4 ^ fr) << 5) + (jl & 3) * 8;
    const u32x4* a_row[kMT];
#pragma unroll
    for (int t = 0; t < kMT; t++) {
        const int m = t * 16 + jl;
        a_row[t] = reinterpret_cast<const u32x4*>(A + (size_t)(m < M ? m : M - 1) * K);
    }
    f32x4 acc[kCB * 4][kMT];
#pragma unroll
    for (int c = 0; c < kCB * 4; c++)
#pragma unroll
        for (int t = 0; t < kMT; t++) acc[c][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int chunks = (k_end - k_begin + 31) / 32;
    const int first = (int)(blockIdx.x % (unsigned)chunks);
    for (int ci = wave; ci < chunks; ci += kWaves) {
        int cc = ci + first;
        if (cc >= chunks) cc -= chunks;
        const int k0 = k_begin + cc * 32;
        const bool full = k0 + 32 <= k_end;  // else the last chunk of a range that is no multiple of 32 (it is one of 8)
        const char* base = reinterpret_cast<const char*>(B) + ((size_t)k0 * N + n0) * 2;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int c = 0; c < kCB; c++) {
                unsigned off = b_off[c][i];
                if (!full) {  // a k-row past the end repeats the range's last one (zeroed below)
                    const int kr = 8 * i + prow;
                    if (k0 + kr >= k_end) off -= (unsigned)(k0 + kr - (k_end - 1)) * (unsigned)N * 2u;
                }
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                             :
                             : "s"(lds_wave + c * kBlockBytes + i * 1024), "v"(off), "s"(base)
                             : "m0", "memory");
            }
        }
        const bool in = full || k0 + 8 * blk < k_end;
        u32x4 x[kMT];
#pragma unroll
        for (int t = 0; t < kMT; t++) {
            x[t] = a_row[t][(k0 >> 3) + (in ? blk : 0)];
            if (!full) x[t] = in ? x[t] : u32x4{0u, 0u, 0u, 0u};
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int c = 0; c < kCB; c++)
#pragma unroll
            for (int c4 = 0; c4 < 4; c4++) {
                const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(MRK_LDS_PTR(bf16x4, rd[c4] + c * kBlockBytes));
                const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(MRK_LDS_PTR(bf16x4, rd[c4] + c * kBlockBytes + 4 * 128));
                u32x4 w = __builtin_bit_cast(u32x4, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                if (!full) w = in ? w : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
                for (int t = 0; t < kMT; t++) {
                    f32x4& d = acc[c * 4 + c4][t];
                    if constexpr (kF16) d = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, w), __builtin_bit_cast(f16x8, x[t]), d, 0, 0, 0);
                    else d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, x[t]), d, 0, 0, 0);
                }
            }
    }
    __syncthreads();
    f32x4* partial = reinterpret_cast<f32x4*>(smem);  // [kWaves][kTiles][64]
#pragma unroll
    for (int c = 0; c < kCB * 4; c++)
#pragma unroll
        for (int t = 0; t < kMT; t++) partial[(wave * kTiles + c * kMT + t) * 64 + lane] = acc[c][t];
    __syncthreads();
    for (int e = threadIdx.x; e < kTiles * 64; e += kWaves * 64) {
        const int tile = e >> 6, l = e & 63;
        f32x4 s = partial[tile * 64 + l];
#pragma unroll
        for (int w = 1; w < kWaves; w++) s += partial[(w * kTiles + tile) * 64 + l];
        const int c = tile / kMT, m = (tile % kMT) * 16 + (l & 15);
        const long n = n0 + c * 16 + 4 * (l >> 4);
        if (m >= M || n >= N) continue;  // N is a multiple of 8: a lane's four columns are all inside or all outside
        if (W) {
            *reinterpret_cast<f32x4*>(W + ((size_t)blockIdx.y * M + m) * N + n) = s;
        } else {
            const unsigned short* ad = add ? add + (size_t)m * add_pitch : nullptr;  // (the addend's row: pitch 0 for a bias)
            unsigned short o[4];
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] = round_out<kF16>(s[i], ad, n + i);
            *reinterpret_cast<u32x2*>(C + (size_t)m * N + n) = u32x2{(unsigned)o[0] | ((unsigned)o[1] << 16), (unsigned)o[2] | ((unsigned)o[3] << 16)};
        }
    }
}


// C[i] = round(W[0][i] + W[1][i] + ... + W[splits - 1][i]) for the partial sums above, which come in many
// more slices than the tiled kernels' split-K leaves (up to 128): a workgroup folds 64 outputs, 32
// work-items per group of eight outputs each taking every 32nd slice, then one of them adds the 32
// sums in order.  The order is fixed, so the result does not depend on timing.
template <bool kF16>
__global__ __launch_bounds__(256) void gemm_kn_skinny_reduce(const float* __restrict__ W, unsigned short* __restrict__ C, long total, int splits,
                                                             const unsigned short* __restrict__ add, long add_period) {
    __shared__ float4 red[32][8][2];
    const int eg = threadIdx.x & 7, sl = threadIdx.x >> 3;
    const long i = ((long)blockIdx.x * 8 + eg) * 8;
    float4 lo = make_float4(0.f, 0.f, 0.f, 0.f), hi = lo;
    if (i < total)
        for (int s = sl; s < splits; s += 32) {
            const float4* p = reinterpret_cast<const float4*>(W + (size_t)s * total + i);
            const float4 a = p[0], b = p[1];
            lo.x += a.x, lo.y += a.y, lo.z += a.z, lo.w += a.w;
            hi.x += b.x, hi.y += b.y, hi.z += b.z, hi.w += b.w;
        }
    red[sl][eg][0] = lo;
    red[sl][eg][1] = hi;
    __syncthreads();
    if (sl == 0 && i < total) {
        for (int l = 1; l < 32; l++) {
            const float4 a = red[l][eg][0], b = red[l][eg][1];
            lo.x += a.x, lo.y += a.y, lo.z += a.z, lo.w += a.w;
            hi.x += b.x, hi.y += b.y, hi.z += b.z, hi.w += b.w;
        }
        const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        unsigned short o[8];
        // (the addend: a matrix of the result's shape, add_period 0, or one row repeated every add_period elements)
        const unsigned short* ad = add ? add + (add_period ? i % add_period : i) : nullptr;
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] = round_out<kF16>(v[e], ad, e);
        u32x4 pk = {(unsigned)o[0] | ((unsigned)o[1] << 16), (unsigned)o[2] | ((unsigned)o[3] << 16), (unsigned)o[4] | ((unsigned)o[5] << 16),
                    (unsigned)o[6] | ((unsigned)o[7] << 16)};
        *reinterpret_cast<u32x4*>(C + i) = pk;
    }
}


// C[i] = round(W[0][i] + ... + W[splits - 1][i]) for the few ranges gemm_kn_rows leaves (at most a few dozen):
// a work-item adds its four outputs' partial sums in the order of the ranges.
template <bool kF16>
__global__ __launch_bounds__(256) void gemm_kn_rows_reduce(const float* __restrict__ W, unsigned short* __restrict__ C, long total, int splits,
                                                           const unsigned short* __restrict__ add, long add_period) {
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= total) return;
    f32x4 s = *reinterpret_cast<const f32x4*>(W + i);
    for (int k = 1; k < splits; k++) s += *reinterpret_cast<const f32x4*>(W + (size_t)k * total + i);
    const unsigned short* ad = add ? add + (add_period ? i % add_period : i) : nullptr;
    unsigned short o[4];
#pragma unroll
    for (int j = 0; j < 4; j++) o[j] = round_out<kF16>(s[j], ad, j);
    *reinterpret_cast<u32x2*>(C + i) = u32x2{(unsigned)o[0] | ((unsigned)o[1] << 16), (unsigned)o[2] | ((unsigned)o[3] << 16)};
}

}  // namespace mrk::dev

namespace mrk {

bool gemm_nt_skinny_supported(long M, long N, long K, long batch) {
    return M >= 1 && M <= 2 && N >= 1 && K >= 8 && K % 8 == 0 && K <= 0x7fffffffL && N <= 0x7fffffffL && batch >= 1 && batch <= 65535;
}

namespace {
int launch_nt_skinny(void* stream, const void* A, const void* Bt, void* C, long M, long N, long K, long batch, bool f16, const void* add,
                     long add_pitch) {
    using namespace mrk::dev;
    const unsigned short* bs = static_cast<const unsigned short*>(add);
    const long bp = add_pitch;
    if (!gemm_nt_skinny_supported(M, N, K, batch)) return (int)hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(Bt)) % 16 || reinterpret_cast<uintptr_t>(C) % 2) return (int)hipErrorInvalidValue;
    (void)hipGetLastError();
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned short* a = static_cast<const unsigned short*>(A);
    const unsigned short* b = static_cast<const unsigned short*>(Bt);
    unsigned short* c = static_cast<unsigned short*>(C);
    // (one row: two weight rows per workgroup stream fastest, 6.2 against 6.0 TB/s with four; every workgroup reads
    // all of A, so with two rows four weight rows per workgroup halve A's share of the traffic)
#define MRK_SKINNY(KM, KR)                                                                                  \
    do {                                                                                                    \
        const dim3 grid((unsigned)((N + KR - 1) / KR), (unsigned)batch);                                    \
        if (f16) gemm_nt_skinny<KM, KR, true><<<grid, 256, 0, s>>>(a, b, c, (int)M, (int)N, (int)K, bs, bp); \
        else gemm_nt_skinny<KM, KR, false><<<grid, 256, 0, s>>>(a, b, c, (int)M, (int)N, (int)K, bs, bp);    \
    } while (0)
    if (M == 1) MRK_SKINNY(1, 2);
    else MRK_SKINNY(2, 4);
#undef MRK_SKINNY
    return (int)hipGetLastError();
}
}  // namespace

int launch_gemm_nt_skinny(void* stream, const void* A, const void* Bt, void* C, long M, long N, long K, long batch, bool f16) {
    return launch_nt_skinny(stream, A, Bt, C, M, N, K, batch, f16, nullptr, 0);
}

// 3 to 64 rows on the matrix pipes (gemm_nt_rows).  Byte offsets inside a workgroup's rows are 32-bit.
bool gemm_nt_rows_supported(long M, long N, long K, long batch) {
    return M >= 1 && M <= 64 && N >= 1 && N <= 0x7fffffffL && K >= 8 && K % 8 == 0 && K <= (1L << 23) && batch >= 1 && batch <= 65535;
}

namespace {
// Weight blocks (16 rows) per workgroup.  More of them spread the traffic of A (every workgroup reads all of it:
// kMT / kRT of the weight's bytes) over more weight rows; what costs more is an uneven spread over the 256 CUs:
// the memory system serves the CUs about evenly, so the launch lasts as long as the CU with the most workgroups
// needs (344 workgroups, i.e. two on 88 CUs and one on the rest, measured 15 % slower than 230 or 459).
int rows_blocks_per_group(long N, int mt) {
    const long tiles = (N + 15) / 16;
    int best = 1;
    double best_score = -1.0;
    for (int rt : {6, 4, 3, 2, 1}) {
        if (rt * mt > 18) continue;  // (not instantiated: the partial sums of 8 waves would not fit the LDS)
        const long groups = (tiles + rt - 1) / rt;
        const long per_cu = (groups + 255) / 256;
        const double even = (double)groups / (double)(256 * per_cu);
        const double score = even / (1.0 + 0.25 * mt / rt);
        if (score > best_score) best_score = score, best = rt;
    }
    return best;
}
}  // namespace

namespace {
int launch_nt_rows(void* stream, const void* A, const void* Bt, void* C, long M, long N, long K, long batch, bool f16, const void* add,
                   long add_pitch) {
    using namespace mrk::dev;
    const unsigned short* bs = static_cast<const unsigned short*>(add);
    const long bp = add_pitch;
    if (!gemm_nt_rows_supported(M, N, K, batch)) return (int)hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(Bt)) % 16 || reinterpret_cast<uintptr_t>(C) % 8) return (int)hipErrorInvalidValue;
    (void)hipGetLastError();
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned short* a = static_cast<const unsigned short*>(A);
    const unsigned short* b = static_cast<const unsigned short*>(Bt);
    unsigned short* c = static_cast<unsigned short*>(C);
    const int mt = (int)((M + 15) / 16);
    const int rt = rows_blocks_per_group(N, mt);
#define MRK_ROWS(MT, RT, WV)                                                                              \
    do {                                                                                                  \
        const dim3 grid((unsigned)((N + 16 * RT - 1) / (16 * RT)), (unsigned)batch);                      \
        if (f16) gemm_nt_rows<MT, RT, WV, true><<<grid, WV * 64, 0, s>>>(a, b, c, (int)M, (int)N, (int)K, bs, bp); \
        else gemm_nt_rows<MT, RT, WV, false><<<grid, WV * 64, 0, s>>>(a, b, c, (int)M, (int)N, (int)K, bs, bp); \
    } while (0)
#define MRK_ROWS_UP_TO_4(MT)                  \
    do {                                      \
        if (rt == 1) MRK_ROWS(MT, 1, 16);     \
        else if (rt == 2) MRK_ROWS(MT, 2, 8); \
        else if (rt == 3) MRK_ROWS(MT, 3, 8); \
        else MRK_ROWS(MT, 4, 8);              \
    } while (0)
#define MRK_ROWS_MT(MT)                      \
    do {                                     \
        if (rt == 6) MRK_ROWS(MT, 6, 8);     \
        else MRK_ROWS_UP_TO_4(MT);           \
    } while (0)
    if (mt == 1) MRK_ROWS_MT(1);
    else if (mt == 2) MRK_ROWS_MT(2);
    else if (mt == 3) MRK_ROWS_MT(3);
    else MRK_ROWS_UP_TO_4(4);  // (six blocks of 4 x 16 rows: not instantiated, rows_blocks_per_group never asks for it)
#undef MRK_ROWS_UP_TO_4
#undef MRK_ROWS_MT
#undef MRK_ROWS
    return (int)hipGetLastError();
}
}  // namespace

int launch_gemm_nt_rows(void* stream, const void* A, const void* Bt, void* C, long M, long N, long K, long batch, bool f16) {
    return launch_nt_rows(stream, A, Bt, C, M, N, K, batch, f16, nullptr, 0);
}

// c[M, F] = silu(a gate) * (a up) over a weight [2 F, K] (gate rows first) for the shapes the matrix-pipe kernel takes,
// bf16: the gated form of gemm_nt_rows.  Row offsets of the up blocks from the workgroup's first row are 32-bit.
bool gemm_nt_swiglu_streamed(long M, long F, long K) {
    return gemm_nt_rows_supported(M, 2 * F, K, 1) && (F + 96) * K * 2 < (1L << 32);
}

int launch_gemm_nt_swiglu_streamed(void* stream, const void* A, const void* Bt, void* C, long M, long F, long K) {
    using namespace mrk::dev;
    if (!gemm_nt_swiglu_streamed(M, F, K)) return (int)hipErrorInvalidValue;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(Bt)) % 16 || reinterpret_cast<uintptr_t>(C) % 8) return (int)hipErrorInvalidValue;
    (void)hipGetLastError();
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned short* a = static_cast<const unsigned short*>(A);
    const unsigned short* b = static_cast<const unsigned short*>(Bt);
    unsigned short* c = static_cast<unsigned short*>(C);
    const int mt = (int)((M + 15) / 16);
    // gate and up blocks together: as many weight blocks per workgroup as the plain kernel would take, in pairs
    int rt = rows_blocks_per_group(2 * F, mt) / 2;
    rt = rt < 1 ? 1 : rt > 3 ? 3 : rt;
    if (2 * rt * mt > 18) rt = mt == 4 ? 2 : rt;
#define MRK_GATE(MT, RT)                                                                                                       \
    do {                                                                                                                       \
        const dim3 grid((unsigned)((F + 16 * RT - 1) / (16 * RT)), 1);                                                         \
        gemm_nt_rows<MT, RT, 8, false, true><<<grid, 512, 0, s>>>(a, b, c, (int)M, (int)F, (int)K, nullptr, 0);                \
    } while (0)
#define MRK_GATE_MT(MT)                \
    do {                               \
        if (rt == 1) MRK_GATE(MT, 1);  \
        else if (rt == 2) MRK_GATE(MT, 2); \
        else MRK_GATE(MT, 3);          \
    } while (0)
    if (mt == 1) MRK_GATE_MT(1);
    else if (mt == 2) MRK_GATE_MT(2);
    else if (mt == 3) MRK_GATE_MT(3);
    else if (rt == 1) MRK_GATE(4, 1);
    else MRK_GATE(4, 2);
#undef MRK_GATE_MT
#undef MRK_GATE
    return (int)hipGetLastError();
}

bool gemm_nt_bias_streamed(long M, long N, long K, long batch) {
    return batch == 1 && (gemm_nt_skinny_supported(M, N, K, 1) || gemm_nt_rows_supported(M, N, K, 1));
}

int launch_gemm_nt_bias_streamed(void* stream, const void* A, const void* Bt, const void* add, void* C, long M, long N, long K, bool f16,
                                 bool add_is_row) {
    if (!add || reinterpret_cast<uintptr_t>(add) % 2) return (int)hipErrorInvalidValue;
    const long pitch = add_is_row ? 0 : N;
    if (gemm_nt_skinny_supported(M, N, K, 1)) return launch_nt_skinny(stream, A, Bt, C, M, N, K, 1, f16, add, pitch);
    return launch_nt_rows(stream, A, Bt, C, M, N, K, 1, f16, add, pitch);
}

// Plan of the [K, N] form for one row on the vector ALUs: K split into `splits` groups of `rows_per_group` rows
// (a multiple of 32), enough of them to fill the chip with workgroups of 512 columns, few enough
// that the f32 partial sums stay a small part of the weight's bytes (and within 32 MiB).
bool gemm_kn_skinny_plan(long M, long N, long K, long batch, long* splits, long* rows_per_group) {
    // One row, up to 24576 columns: measured against split-K over the tiled kernels, 9.3 against 12.5 us at
    // 1 x 4096 x 4096, 18.8 against 20.1 at N = 12288, 34 against 39 at N = 22016, 18.3 against 21.8 at 4096 x 11008
    // (with 32000 columns 46.6 against 42.9 us).  Two and more rows, and one row against wider weights, take the
    // matrix-pipe kernel (gemm_kn_rows_plan), which measured faster from two rows on.
    if (M != 1 || batch != 1 || N < 8 || N > 24576 || N % 8 || K < 256 || K % 8 || K > 0x7fffffffL) return false;
    const long col_groups = (N + 511) / 512;
    long want = (2048 + col_groups - 1) / col_groups;
    const long by_traffic = K / (16 * M) > 0 ? K / (16 * M) : 1;          // 2 * S * M * N * 4 <= K * N * 2 / 4
    const long by_bytes = (32L << 20) / (M * N * 4) > 0 ? (32L << 20) / (M * N * 4) : 1;
    want = want < by_traffic ? want : by_traffic;
    want = want < by_bytes ? want : by_bytes;
    want = want < K / 32 ? want : K / 32;
    if (want < 2) return false;
    long rows = ((K + want - 1) / want + 31) / 32 * 32;
    const long s = (K + rows - 1) / rows;
    if (s < 2 || s > 65535) return false;
    *splits = s;
    *rows_per_group = rows;
    return true;
}

int launch_gemm_kn_skinny(void* stream, const void* A, const void* B, void* C, void* W, long M, long N, long K, long splits, long rows_per_group,
                          bool f16, const void* add, bool add_is_row) {
    using namespace mrk::dev;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(W) | reinterpret_cast<uintptr_t>(C)) % 16)
        return (int)hipErrorInvalidValue;
    (void)hipGetLastError();
    const dim3 grid((unsigned)((N + 511) / 512), (unsigned)splits);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned short* a = static_cast<const unsigned short*>(A);
    const unsigned short* b = static_cast<const unsigned short*>(B);
    float* w = static_cast<float*>(W);
#define MRK_KN(KM)                                                                                                  \
    do {                                                                                                            \
        if (f16) gemm_kn_skinny_partial<KM, true><<<grid, 256, 0, s>>>(a, b, w, (int)M, (int)N, (int)K, (int)rows_per_group);  \
        else gemm_kn_skinny_partial<KM, false><<<grid, 256, 0, s>>>(a, b, w, (int)M, (int)N, (int)K, (int)rows_per_group);     \
    } while (0)
    MRK_KN(1);
#undef MRK_KN
    const long total = M * N;  // (a multiple of 8)
    const unsigned blocks = (unsigned)((total + 63) / 64);
    const unsigned short* ad = static_cast<const unsigned short*>(add);
    const long period = add_is_row ? N : 0;
    if (f16) gemm_kn_skinny_reduce<true><<<blocks, 256, 0, s>>>(w, static_cast<unsigned short*>(C), total, (int)splits, ad, period);
    else gemm_kn_skinny_reduce<false><<<blocks, 256, 0, s>>>(w, static_cast<unsigned short*>(C), total, (int)splits, ad, period);
    return (int)hipGetLastError();
}


// Plan of the [K, N] form for up to 16 rows (one row: where gemm_kn_skinny_plan does not take it), and up to 64 rows against a weight of at most 4096 columns and 8192 rows,
// where the tiled kernels have the fewest tiles to spread (gemm_kn_rows): column groups of 128 (64 for a narrow weight),
// K split into enough ranges (multiples of 32 rows) for about one workgroup per CU, few enough that the f32 partial sums
// stay a small part of the weight's bytes.  splits == 1: one launch, no scratch.
bool gemm_kn_rows_plan(long M, long N, long K, long batch, long* splits, long* k_per_split) {
    if (M < 1 || M > 64 || batch != 1 || N < 8 || N % 8 || N > (1L << 24) || K < 256 || K % 8 || K > (1L << 23)) return false;
    if (M > 16 && (N > 4096 || K > 8192)) return false;
    const long groups = N >= 8192 ? (N + 127) / 128 : (N + 63) / 64;
    long want = 256 / groups;
    const long by_traffic = K / (16 * M), by_rows = K / 256;
    want = want < by_traffic ? want : by_traffic;
    want = want < by_rows ? want : by_rows;
    if (want < 1) want = 1;
    const long per = ((K + want - 1) / want + 31) / 32 * 32;
    const long s = (K + per - 1) / per;
    if (s > 65535 || s * M * N * 4 > (32L << 20)) return false;
    *splits = s;
    *k_per_split = per;
    return true;
}

int launch_gemm_kn_rows(void* stream, const void* A, const void* B, void* C, void* W, long M, long N, long K, long splits, long k_per_split,
                        bool f16, const void* add, bool add_is_row) {
    using namespace mrk::dev;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(W) | reinterpret_cast<uintptr_t>(C)) % 16)
        return (int)hipErrorInvalidValue;
    if (splits > 1 && !W) return (int)hipErrorInvalidValue;
    (void)hipGetLastError();
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned short* a = static_cast<const unsigned short*>(A);
    const unsigned short* b = static_cast<const unsigned short*>(B);
    unsigned short* c = static_cast<unsigned short*>(C);
    float* w = splits > 1 ? static_cast<float*>(W) : nullptr;
    const unsigned short* ad = static_cast<const unsigned short*>(add);
    const long pitch = add_is_row ? 0 : N;
#define MRK_KN_ROWS(MT, CB)                                                                                              \
    do {                                                                                                                 \
        const dim3 grid((unsigned)((N + 64 * CB - 1) / (64 * CB)), (unsigned)splits);                                    \
        if (f16) gemm_kn_rows<MT, CB, true><<<grid, 512, 0, s>>>(a, b, c, w, (int)M, (int)N, (int)K, (int)k_per_split, ad, pitch);  \
        else gemm_kn_rows<MT, CB, false><<<grid, 512, 0, s>>>(a, b, c, w, (int)M, (int)N, (int)K, (int)k_per_split, ad, pitch);     \
    } while (0)
    if (M > 32) MRK_KN_ROWS(4, 1);
    else if (M > 16) MRK_KN_ROWS(2, 1);
    else if (N >= 8192) MRK_KN_ROWS(1, 2);
    else MRK_KN_ROWS(1, 1);
#undef MRK_KN_ROWS
    if (splits > 1) {
        const long total = M * N;  // (a multiple of 8)
        const unsigned blocks = (unsigned)((total / 4 + 255) / 256);
        if (f16) gemm_kn_rows_reduce<true><<<blocks, 256, 0, s>>>(w, c, total, (int)splits, ad, add_is_row ? N : 0);
        else gemm_kn_rows_reduce<false><<<blocks, 256, 0, s>>>(w, c, total, (int)splits, ad, add_is_row ? N : 0);
    }
    return (int)hipGetLastError();
}

}  // namespace mrk
