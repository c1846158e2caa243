// Attention for a handful of queries against a long key sequence (a decode step over a key/value cache,
// tensor/src/transformer.rs:78-137 with Sq of 1 to 32): O = softmax(Q K^T * scale) V is a stream over K and V,
// 4 * Sk * D bytes per (batch, head) against a few flops per byte, and with few (batch, head) pairs the kernel that
// gives every pair one workgroup leaves most of the chip without work.  Here the key sequence is split as well:
// grid = (splits, pairs), a workgroup owns a contiguous range of keys, its waves take the range's 32-key
// chunks in turn.  A wave copies its chunk of K and of V (32 rows each) with direct global -> LDS loads into a
// region of its own (1 KB per instruction, non-temporal: every byte is read once), so the loop has no barrier,
// and what streams is bounded by the bytes in flight per CU, i.e. by what the LDS holds.
// S^T = K Q^T on v_mfma_f32_16x16x32_bf16 (operand A: 16 keys x 32 d read back from LDS, rows swizzled by the key
// so that the 16 rows of a read fall into different banks; operand B: the queries, 16 columns, loaded once;
// queries beyond Sq repeat the last one and are not written; from 17 on a second block of 16 takes the same K and V
// fragments): a lane then holds, for query l % 16, the keys
// 4 * (l / 16) + 0..3 of each of the chunk's two 16-key blocks.  Those eight values, exponentiated against the
// running maximum and rounded to bf16, are directly the lane's operand of O^T += V^T P^T if the instruction's
// eight k-slots of lane group g are taken to be exactly those keys; V's side follows through the transposing
// LDS read (ds_read_b64_tr_b16: lane j of a 16-lane group receives column j of the four rows the group's lanes
// point at), pointed at rows 4 g + 0..3 of either block.  Running maximum and sum per query as in any online
// softmax; a query's maximum sits in four lanes (l % 16 equal), two exchanges per chunk.
// At the end the waves' (maximum, sum, O) meet in LDS and are merged in a fixed order; with one split the
// workgroup writes O, otherwise f32 partial results W[split][pair][16][D + 2] (the unnormalised O, then
// maximum and sum), which flash_decode_merge folds the same way.  Results do not depend on scheduling.
// A pair is a (batch, head), or a (batch, run of consecutive heads) when those heads share their K and V (zero
// head strides: multi-query / grouped-query attention): the run's heads then occupy the query slots together
// and K and V are read once for all of them.  attn_mask (Bool bytes or additive bf16, any broadcast layout) and
// softcap of the reference (transformer.rs:112-132) are template options: a lane loads the mask of its eight keys
// with the chunk's copies and applies it, then the cap, to its scores before the maximum.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace mrk::dev {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

#define MRK_FD_LDS(T, p) ((__attribute__((address_space(3))) T*)(p))

constexpr int kChunkKeys = 32;  // keys a wave handles per step
constexpr int kMaxQueries = 32;  // query slots of a pair: one or two blocks of 16

struct DecodeLayout {
    long long q_batch, q_head, k_batch, k_head, v_batch, v_head, o_batch, o_head;  // element strides
    unsigned q_row, k_row, v_row, o_row;                                           // byte strides of a row
    int heads;  // pairs per batch: the head count divided by `group`
    int group;  // consecutive heads folded into one pair's query slots (they share K and V: zero head strides), 1 = none
};

// attn_mask of the reference (transformer.rs:112-125) as a [batch, head, query, key] view with contiguous keys:
// element strides per batch, head and query row (0 broadcasts).  Kind 1: Bool bytes, nonzero = attend; 2: additive bf16.
struct DecodeMask {
    const void* mask;
    long long batch, head, row;
    float cap;  // softcap in score units (transformer.rs:128-132), used by the kCap instantiations
};

template <int kD>
constexpr int decode_waves() {
    return kD == 256 ? 4 : 8;  // a wave's region is 4 * 32 * kD bytes: 128 KB of LDS for 128 and 256, 64 KB for 64
}

// kQB: 16-slot query blocks a workgroup carries (1 or 2: up to 32 query slots per pair); the K and V fragments a wave
// reads from LDS serve every block.
template <int kD, int kMask, bool kCap, int kQB>
__global__ __launch_bounds__(decode_waves<kD>() * 64) void flash_decode_split(
    const unsigned short* __restrict__ Q, const unsigned short* __restrict__ K, const unsigned short* __restrict__ V,
    unsigned short* __restrict__ O, float* __restrict__ W, int Sq, int Sk, int keys_per_split, float scale_log2e, DecodeLayout lay,
    DecodeMask dm) {
    constexpr int kWaves = decode_waves<kD>();
    constexpr int kRowBytes = kD * 2;
    constexpr int kPieces = kD / 8;                      // 16-byte pieces of a row
    constexpr int kRowsPerCopy = 1024 / kRowBytes;       // 8, 4, 2
    constexpr int kCopies = kChunkKeys / kRowsPerCopy;   // per operand and chunk
    constexpr int kOperandBytes = kChunkKeys * kRowBytes;
    constexpr int kWaveBytes = 2 * kOperandBytes;
    constexpr int kSteps = kD / 32;                      // matrix steps of a score block
    constexpr int kColBlocks = kD / 16;                  // 16-column blocks of O
    constexpr int kSlots = 16 * kQB;                     // query slots of a pair
    constexpr int kPartBytes = kQB * (kColBlocks * 1024 + 128);  // a wave's O blocks, then maximum and sum, per query block
    constexpr int kLds = kWaves * kWaveBytes > kWaves * kPartBytes ? kWaves * kWaveBytes : kWaves * kPartBytes;
    static_assert(kLds <= 160 * 1024, "LDS");
    __shared__ __attribute__((aligned(1024))) char smem[kLds];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int jl = lane & 15, blk = lane >> 4;
    const int bh = blockIdx.y, b = bh / lay.heads, h = (bh % lay.heads) * lay.group;  // h: the pair's first head
    const int k_begin = blockIdx.x * keys_per_split;
    const int k_end = k_begin + keys_per_split < Sk ? k_begin + keys_per_split : Sk;
    const unsigned lds_k = (unsigned)(uintptr_t)MRK_FD_LDS(char, smem) + wave * kWaveBytes;
    const unsigned lds_v = lds_k + kOperandBytes;
    const char* k_head = reinterpret_cast<const char*>(K + b * lay.k_batch + h * lay.k_head);
    const char* v_head = reinterpret_cast<const char*>(V + b * lay.v_batch + h * lay.v_head);

    // the queries: operand B, query slot 16 qb + jl (the last one again beyond the pair's slots), eight d at 32 s + 8 blk
    // (query slots: head g of a folded run, row r of its Sq rows, slot g * Sq + r)
    u32x4 qf[kQB][kSteps];
    const int nq = Sq * lay.group;
    // the mask row of a lane's query: a lane needs the mask of its eight keys per chunk, two groups of four
    // consecutive ones (the key count is a multiple of 4 under a mask, so a group is inside the sequence or outside)
    const char* mrow[kQB];
#pragma unroll
    for (int qb = 0; qb < kQB; qb++) {
        const int want = 16 * qb + jl;
        const int slot = want < nq ? want : nq - 1;
        const int qg = slot / Sq, qi = slot - qg * Sq;
        mrow[qb] = nullptr;
        if constexpr (kMask != 0)
            mrow[qb] = static_cast<const char*>(dm.mask) + (b * dm.batch + (h + qg) * dm.head + qi * dm.row) * (kMask == 2 ? 2 : 1);
        const char* qrow = reinterpret_cast<const char*>(Q + b * lay.q_batch + (h + qg) * lay.q_head) + (size_t)qi * lay.q_row;
#pragma unroll
        for (int s = 0; s < kSteps; s++) qf[qb][s] = *reinterpret_cast<const u32x4*>(qrow + 64 * s + 16 * blk);
    }
    // copy side: copy i covers rows i * kRowsPerCopy ..; lane -> row rsub of them, position pos of the row in LDS.
    // K: position p holds piece p ^ key(row), key = row & 15 (rows of 256 bytes and more) or (row >> 1) & 7
    // (128-byte rows, two to a bank period).  V: 32-byte granule G at granule G ^ key(row), key = row & 7
    // or (row >> 1) & 3.
    const int pos = lane % kPieces, rsub = lane / kPieces;
    unsigned k_piece[kCopies], v_piece[kCopies];
#pragma unroll
    for (int i = 0; i < kCopies; i++) {
        const int r = i * kRowsPerCopy + rsub;
        const int kk = kD >= 128 ? (r & 15) : ((r >> 1) & 7);
        const int vk = kD >= 128 ? (r & 7) : ((r >> 1) & 3);
        k_piece[i] = (unsigned)(pos ^ kk) * 16u;
        v_piece[i] = (unsigned)((((pos >> 1) ^ vk) << 1) | (pos & 1)) * 16u;
    }
    // read side, K: row jl of a 16-key block, piece 4 s + blk of it
    const unsigned kx = (unsigned)(kD >= 128 ? jl : ((jl >> 1) & 7));
    const unsigned rd_k = lds_k + jl * kRowBytes;
    // read side, V: rows 4 blk + (jl >> 2) of either block, 8-byte unit jl & 3 of column block c's granule
    const int vr = 4 * blk + (jl >> 2);
    const unsigned vx = (unsigned)(kD >= 128 ? (vr & 7) : ((vr >> 1) & 3));
    const unsigned rd_v = lds_v + vr * kRowBytes + (jl & 3) * 8;

    f32x4 acc[kQB][kColBlocks];
    float m_run[kQB], l_run[kQB];  // l_run: this lane's share of the sum (its eight keys per chunk)
#pragma unroll
    for (int qb = 0; qb < kQB; qb++) {
#pragma unroll
        for (int c = 0; c < kColBlocks; c++) acc[qb][c] = f32x4{0.f, 0.f, 0.f, 0.f};
        m_run[qb] = -INFINITY;
        l_run[qb] = 0.0f;
    }

    const int chunks = (k_end - k_begin + kChunkKeys - 1) / kChunkKeys;
    for (int ci = wave; ci < chunks; ci += kWaves) {
        const int k0 = k_begin + ci * kChunkKeys;
        const bool full = k0 + kChunkKeys <= k_end;
        const int last = k_end - 1 - k0;  // the chunk's last valid row
        const char* kb = k_head + (size_t)k0 * lay.k_row;
        const char* vb = v_head + (size_t)k0 * lay.v_row;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the previous chunk's fragment reads are done
#pragma unroll
        for (int i = 0; i < kCopies; i++) {
            int r = i * kRowsPerCopy + rsub;
            if (!full) r = r < last ? r : last;  // a row past the end repeats the last one (masked below)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                         :
                         : "s"(lds_k + i * 1024), "v"((unsigned)r * lay.k_row + k_piece[i]), "s"(kb)
                         : "m0", "memory");
        }
#pragma unroll
        for (int i = 0; i < kCopies; i++) {
            int r = i * kRowsPerCopy + rsub;
            if (!full) r = r < last ? r : last;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                         :
                         : "s"(lds_v + i * 1024), "v"((unsigned)r * lay.v_row + v_piece[i]), "s"(vb)
                         : "m0", "memory");
        }
        // the mask of this lane's keys, requested together with the copies
        unsigned mb0[kQB], mb1[kQB];  // Bool: four bytes per group
        u32x2 ma0[kQB], ma1[kQB];     // additive: four bf16 per group
#pragma unroll
        for (int qb = 0; qb < kQB; qb++) {
            mb0[qb] = mb1[qb] = 0u;
            ma0[qb] = ma1[qb] = u32x2{0u, 0u};
            if constexpr (kMask != 0) {
                const int g0 = k0 + 4 * blk, g1 = g0 + 16;
                if constexpr (kMask == 1) {
                    if (g0 < k_end) mb0[qb] = *reinterpret_cast<const unsigned*>(mrow[qb] + g0);
                    if (g1 < k_end) mb1[qb] = *reinterpret_cast<const unsigned*>(mrow[qb] + g1);
                } else {
                    if (g0 < k_end) ma0[qb] = *reinterpret_cast<const u32x2*>(mrow[qb] + 2 * (size_t)g0);
                    if (g1 < k_end) ma1[qb] = *reinterpret_cast<const u32x2*>(mrow[qb] + 2 * (size_t)g1);
                }
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        // scores of the two 16-key blocks, per query block
        f32x4 s0[kQB], s1[kQB];
#pragma unroll
        for (int qb = 0; qb < kQB; qb++) s0[qb] = s1[qb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            const unsigned po = (((unsigned)(4 * s + blk)) ^ kx) * 16u;
            const u32x4 f0 = *MRK_FD_LDS(u32x4, rd_k + po);
            const u32x4 f1 = *MRK_FD_LDS(u32x4, rd_k + 16 * kRowBytes + po);
#pragma unroll
            for (int qb = 0; qb < kQB; qb++) {
                s0[qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, f0), __builtin_bit_cast(bf16x8, qf[qb][s]), s0[qb], 0, 0, 0);
                s1[qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, f1), __builtin_bit_cast(bf16x8, qf[qb][s]), s1[qb], 0, 0, 0);
            }
        }
        bf16x8 pb[kQB];
        float alpha[kQB];
#pragma unroll
        for (int qb = 0; qb < kQB; qb++) {
            float x[8];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                x[r] = s0[qb][r] * scale_log2e;
                x[4 + r] = s1[qb][r] * scale_log2e;
            }
            if constexpr (kMask == 1) {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    if (((mb0[qb] >> (8 * r)) & 0xffu) == 0u) x[r] = -INFINITY;
                    if (((mb1[qb] >> (8 * r)) & 0xffu) == 0u) x[4 + r] = -INFINITY;
                }
            }
            if constexpr (kMask == 2) {
                // scale, then the mask (transformer.rs:96-125), both in exp2 units here
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const unsigned w0 = ma0[qb][r >> 1], w1 = ma1[qb][r >> 1];
                    x[r] += __builtin_bit_cast(float, (r & 1) ? (w0 & 0xffff0000u) : (w0 << 16)) * 1.4426950408889634f;
                    x[4 + r] += __builtin_bit_cast(float, (r & 1) ? (w1 & 0xffff0000u) : (w1 << 16)) * 1.4426950408889634f;
                }
            }
            if constexpr (kCap) {
                // cap * tanh(x / cap) after the mask, with tanh(y) = 1 - 2 / (exp(2 y) + 1); x in exp2 units, so
                // exp(2 x / cap) = exp2(2 t / cap); a masked score (-inf) becomes -cap and still takes part, as in
                // the reference's graph
                const float cap_out = dm.cap * 1.4426950408889634f, cap_in = 2.0f / dm.cap;
#pragma unroll
                for (int r = 0; r < 8; r++) {
                    const float z = __builtin_amdgcn_exp2f(x[r] * cap_in);
                    x[r] = cap_out * (1.0f - 2.0f * __builtin_amdgcn_rcpf(z + 1.0f));
                }
            }
            if (!full) {  // keys that do not exist
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    if (4 * blk + r > last) x[r] = -INFINITY;
                    if (16 + 4 * blk + r > last) x[4 + r] = -INFINITY;
                }
            }
            float mx = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
            mx = fmaxf(mx, __shfl_xor(mx, 16));
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run[qb], mx);  // without a mask finite: the chunk's first key is valid
            // under a mask every key so far may be masked out (maximum -inf): such keys weigh nothing, and nothing has
            // been summed yet; the differences below must not become -inf - -inf
            const float m_ref = kMask != 0 && !kCap && m_new == -INFINITY ? 0.0f : m_new;
            alpha[qb] = __builtin_amdgcn_exp2f(m_run[qb] - m_ref);
            m_run[qb] = m_new;
            f32x8 p;
            float psum = 0.0f;
#pragma unroll
            for (int r = 0; r < 8; r++) {
                p[r] = __builtin_amdgcn_exp2f(x[r] - m_ref);
                psum += p[r];
            }
            l_run[qb] = l_run[qb] * alpha[qb] + psum;
            pb[qb] = __builtin_convertvector(p, bf16x8);
        }
#pragma unroll
        for (int c = 0; c < kColBlocks; c++) {
            const unsigned off = rd_v + (((unsigned)c ^ vx) << 5);
            bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(MRK_FD_LDS(bf16x4, off));
            bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(MRK_FD_LDS(bf16x4, off + 16 * kRowBytes));
            if (!full) {
                // the rows past the end hold copies of the last row; their weights are zero, but a zero times an
                // infinity or a NaN of that row must not reach the sum
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    if (4 * blk + r > last) lo[r] = (__bf16)0.0f;
                    if (16 + 4 * blk + r > last) hi[r] = (__bf16)0.0f;
                }
            }
            const bf16x8 vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
            for (int qb = 0; qb < kQB; qb++) acc[qb][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb[qb], acc[qb][c] * alpha[qb], 0, 0, 0);
        }
    }
    // a query's sum over the four lanes that share it
#pragma unroll
    for (int qb = 0; qb < kQB; qb++) {
        l_run[qb] += __shfl_xor(l_run[qb], 16);
        l_run[qb] += __shfl_xor(l_run[qb], 32);
    }

    // the waves' results meet in LDS, over the copy regions: per wave and query block, the O blocks, then maxima and sums
    __syncthreads();
    char* part = smem;  // [kWaves][kQB][kColBlocks * 1024 + 128]
    constexpr int kBlockPart = kColBlocks * 1024 + 128;
#pragma unroll
    for (int qb = 0; qb < kQB; qb++) {
        f32x4* po = reinterpret_cast<f32x4*>(part + wave * kPartBytes + qb * kBlockPart);
#pragma unroll
        for (int c = 0; c < kColBlocks; c++) po[c * 64 + lane] = acc[qb][c];
        if (blk == 0) {
            float* ml = reinterpret_cast<float*>(part + wave * kPartBytes + qb * kBlockPart + kColBlocks * 1024);
            ml[jl] = m_run[qb];
            ml[16 + jl] = l_run[qb];
        }
    }
    __syncthreads();
    // element e: query block, column block c, lane l of it: slot 16 qb + l % 16, columns 16 c + 4 (l / 16) + 0..3
    for (int e = threadIdx.x; e < kQB * kColBlocks * 64; e += kWaves * 64) {
        const int qb = e / (kColBlocks * 64), c = (e >> 6) % kColBlocks, l = e & 63, ql = l & 15, q = 16 * qb + ql;
        if (q >= nq) continue;
        const char* mine = part + qb * kBlockPart;
        float m_tot = -INFINITY;
#pragma unroll
        for (int w = 0; w < kWaves; w++) m_tot = fmaxf(m_tot, reinterpret_cast<const float*>(mine + w * kPartBytes + kColBlocks * 1024)[ql]);
        f32x4 o = {0.f, 0.f, 0.f, 0.f};
        float l_tot = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; w++) {
            const float* ml = reinterpret_cast<const float*>(mine + w * kPartBytes + kColBlocks * 1024);
            // a wave without a chunk, or whose keys are all masked out: maximum -inf, weight 0; a workgroup of such waves
            // only leaves (0, -inf, 0), which weighs nothing among other ranges and ends as 0 / 0 = NaN without them
            // (the softmax over -inf only of the reference)
            const float wgt = m_tot == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(ml[ql] - m_tot);
            o += reinterpret_cast<const f32x4*>(mine + w * kPartBytes)[c * 64 + l] * wgt;
            l_tot += ml[16 + ql] * wgt;
        }
        const int d = 16 * c + 4 * (l >> 4);
        if (W) {
            float* dst = W + (((size_t)blockIdx.x * gridDim.y + bh) * kSlots + q) * (kD + 2);
            *reinterpret_cast<float2*>(dst + d) = make_float2(o[0], o[1]);
            *reinterpret_cast<float2*>(dst + d + 2) = make_float2(o[2], o[3]);
            if (d == 0) {
                dst[kD] = m_tot;
                dst[kD + 1] = l_tot;
            }
        } else {
            const float inv = 1.0f / l_tot;
            const f32x4 v = {o[0] * inv, o[1] * inv, o[2] * inv, o[3] * inv};
            const int og = q / Sq, orw = q - og * Sq;
            char* orow = reinterpret_cast<char*>(O + b * lay.o_batch + (h + og) * lay.o_head) + (size_t)orw * lay.o_row;
            *reinterpret_cast<bf16x4*>(orow + d * 2) = __builtin_convertvector(v, bf16x4);
        }
    }
}

// O[bh][q][d] from the splits' partial results: the same merge as inside a workgroup, splits in order.
// One work-item per four columns; grid = ceil(pairs * slots * D / 4 / 256) with slots = Sq * group query slots per pair.
template <int kD>
__global__ __launch_bounds__(256) void flash_decode_merge(const float* __restrict__ W, unsigned short* __restrict__ O, int BH, int Sq, int splits,
                                                          int slot_cap, DecodeLayout lay) {
    const long e = (long)blockIdx.x * 256 + threadIdx.x;
    constexpr int kQuads = kD / 4;
    const int nq = Sq * lay.group;
    if (e >= (long)BH * nq * kQuads) return;
    const int d = (int)(e % kQuads) * 4;
    const int q = (int)((e / kQuads) % nq);
    const int bh = (int)(e / ((long)kQuads * nq));
    const size_t slice = (size_t)BH * slot_cap * (kD + 2);  // slot_cap: 16 or 32 slots per pair, as the split kernel laid them out
    const float* src = W + ((size_t)bh * slot_cap + q) * (kD + 2);
    // (both loops unrolled by four: the loads of four ranges are in flight together, the sums keep their order)
    float m_tot = -INFINITY;
#pragma unroll 4
    for (int s = 0; s < splits; s++) m_tot = fmaxf(m_tot, src[s * slice + kD]);
    f32x4 o = {0.f, 0.f, 0.f, 0.f};
    float l_tot = 0.0f;
#pragma unroll 4
    for (int s = 0; s < splits; s++) {
        const float* p = src + s * slice;
        const float wgt = __builtin_amdgcn_exp2f(p[kD] - m_tot);
        const float2 a = *reinterpret_cast<const float2*>(p + d), c = *reinterpret_cast<const float2*>(p + d + 2);
        o += f32x4{a.x, a.y, c.x, c.y} * wgt;
        l_tot += p[kD + 1] * wgt;
    }
    const float inv = 1.0f / l_tot;
    const f32x4 v = {o[0] * inv, o[1] * inv, o[2] * inv, o[3] * inv};
    const int b = bh / lay.heads, h = (bh % lay.heads) * lay.group, og = q / Sq, orw = q - og * Sq;
    char* orow = reinterpret_cast<char*>(O + b * lay.o_batch + (h + og) * lay.o_head) + (size_t)orw * lay.o_row;
    *reinterpret_cast<bf16x4*>(orow + d * 2) = __builtin_convertvector(v, bf16x4);
}

}  // namespace mrk::dev

namespace mrk {
using namespace mrk::dev;

// Shapes the split kernel takes and the number of key ranges it uses: up to 32 query slots of a pair (two blocks
// of 16: 17 and more cost a second set of matrix instructions per chunk, still far from what the stream of K and V
// leaves room for), no causal rule, at least 256 keys.  Measured against one workgroup per 128 queries of a (batch, head) pair it streams K and V
// faster at every count of pairs (7.0 against 6.1 TB/s with 1024 and more), so the count does not limit it.
// Ranges are multiples of 32 keys and at least 512 keys long (two chunks per wave and more); about 192
// workgroups measured best where the pairs alone are fewer (4096 keys, 32 pairs: 41 us in one range, 20 in
// four to eight, 27 in sixteen: the second kernel and the ranges' fixed cost grow with the count).
bool flash_decode_plan(long BH, long Sq, long Sk, long D, int causal, long* splits, long* keys_per_split) {
    if (causal || Sq < 1 || Sq > kMaxQueries || Sk < 256 || Sk > (1L << 24) || BH < 1 || BH > 65535) return false;
    if (D != 256 && D != 128 && D != 64) return false;
    // (two chunks per wave and range at least: 512 keys with eight waves, 256 with the four of head dim 256, whose
    // workgroups, one per CU, measured best at one per CU: 21 against 24 us at [1, 16, 1, 4096], 30 against 33 with 32 pairs)
    const long min_keys = D == 256 ? 256 : 512, target = D == 256 ? 256 : 192;
    const long max_splits = Sk / min_keys > 0 ? Sk / min_keys : 1;
    long want = (target + BH / 2) / BH;
    want = want < max_splits ? want : max_splits;
    want = want < 1 ? 1 : want;
    const long per = ((Sk + want - 1) / want + kChunkKeys - 1) / kChunkKeys * kChunkKeys;
    *keys_per_split = per;
    *splits = (Sk + per - 1) / per;
    return true;
}

// Query slots the partial results of a pair are laid out for: 16, or 32 from 17 slots on.
long flash_decode_slot_capacity(long slots) { return slots <= 16 ? 16 : 32; }

// The workspace a caller provides for (batch * heads) pairs: enough for the plan over those pairs and for the plans
// over fewer pairs that folding heads which share their keys gives (the launchers see the strides, the caller of this
// function need not).
size_t flash_fwd_workspace_bytes(long BH, long Sq, long Sk, long D, int causal) {
    size_t most = 0;
    for (long g = 1; g * Sq <= kMaxQueries && g <= BH; g++) {
        if (BH % g) continue;
        long splits = 0, per = 0;
        if (!flash_decode_plan(BH / g, Sq * g, Sk, D, causal, &splits, &per) || splits <= 1) continue;
        const size_t need = (size_t)splits * (BH / g) * flash_decode_slot_capacity(Sq * g) * (D + 2) * sizeof(float);
        most = need > most ? need : most;
    }
    return most;
}

// strides: (batch, head, row) element strides of q, k, v and o (validated by the caller: multiples of 8, rows
// addressable in 32 bits, pointers 16-byte aligned); W: splits * pairs * flash_decode_slot_capacity(group * Sq) * (D + 2)
// floats, needed with several splits (pairs = B * H / group).
// mask_kind 0: none; 1: Bool bytes, 2: additive bf16, with (batch, head, query row) element strides that are multiples
// of 4, a mask pointer aligned to four elements and Sk a multiple of 4 (validated by the caller as well).  softcap 0: none.
int launch_flash_decode(void* stream, const void* q, const void* k, const void* v, void* o, long B, long H, long Sq, long Sk, long D,
                        float scale, const long* strides, long splits, long keys_per_split, void* W, const void* mask, int mask_kind,
                        const long* mask_strides, float softcap, long group) {
    // group > 1: runs of `group` consecutive heads share K and V (zero head strides) and become query slots of one pair
    if (B <= 0 || H <= 0 || group < 1 || H % group || !strides || !q || !k || !v || !o) return (int)hipErrorInvalidValue;
    const long pairs = B * (H / group), slots = group * Sq;
    if (Sq < 1 || slots > kMaxQueries || Sk < 1 || splits < 1 || pairs > 65535) return (int)hipErrorInvalidValue;
    if (group > 1 && (strides[4] != 0 || strides[7] != 0)) return (int)hipErrorInvalidValue;
    if (keys_per_split < kChunkKeys || keys_per_split % kChunkKeys || splits * keys_per_split < Sk || (splits - 1) * keys_per_split >= Sk)
        return (int)hipErrorInvalidValue;
    if (splits > 1 && !W) return (int)hipErrorInvalidValue;
    DecodeLayout lay;
    lay.q_batch = strides[0], lay.q_head = strides[1], lay.q_row = (unsigned)(strides[2] * 2);
    lay.k_batch = strides[3], lay.k_head = strides[4], lay.k_row = (unsigned)(strides[5] * 2);
    lay.v_batch = strides[6], lay.v_head = strides[7], lay.v_row = (unsigned)(strides[8] * 2);
    lay.o_batch = strides[9], lay.o_head = strides[10], lay.o_row = (unsigned)(strides[11] * 2);
    lay.heads = (int)(H / group);
    lay.group = (int)group;
    if (mask_kind < 0 || mask_kind > 2 || (mask_kind != 0 && (!mask || !mask_strides || Sk % 4)) || !(softcap >= 0.0f)) return (int)hipErrorInvalidValue;
    DecodeMask dm{};
    dm.cap = softcap;
    const bool cap = softcap > 0.0f;
    if (mask_kind != 0) {
        dm.mask = mask;
        dm.batch = mask_strides[0], dm.head = mask_strides[1], dm.row = mask_strides[2];
    }
    const float scale_log2e = scale * 1.4426950408889634f;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)splits, (unsigned)pairs);
    float* w = splits > 1 ? static_cast<float*>(W) : nullptr;
    auto qp = static_cast<const unsigned short*>(q);
    auto kp = static_cast<const unsigned short*>(k);
    auto vp = static_cast<const unsigned short*>(v);
    auto op = static_cast<unsigned short*>(o);
    (void)hipGetLastError();
    const long quads = pairs * slots * (D / 4);
    const unsigned merge_blocks = (unsigned)((quads + 255) / 256);
    const int slot_cap = (int)flash_decode_slot_capacity(slots);
#define MRK_DECODE_QB(DIM, MASK, CAP, QB) \
    flash_decode_split<DIM, MASK, CAP, QB><<<grid, decode_waves<DIM>() * 64, 0, s>>>(qp, kp, vp, op, w, (int)Sq, (int)Sk, (int)keys_per_split, scale_log2e, lay, dm)
#define MRK_DECODE(DIM, MASK)                              \
    do {                                                   \
        if (cap) {                                         \
            if (slot_cap == 16) MRK_DECODE_QB(DIM, MASK, true, 1);  \
            else MRK_DECODE_QB(DIM, MASK, true, 2);        \
        } else {                                           \
            if (slot_cap == 16) MRK_DECODE_QB(DIM, MASK, false, 1); \
            else MRK_DECODE_QB(DIM, MASK, false, 2);       \
        }                                                  \
    } while (0)
#define MRK_DECODE_DIM(DIM)                                                                                         \
    do {                                                                                                            \
        if (mask_kind == 0) MRK_DECODE(DIM, 0);                                                                     \
        else if (mask_kind == 1) MRK_DECODE(DIM, 1);                                                                \
        else MRK_DECODE(DIM, 2);                                                                                    \
        if (w) flash_decode_merge<DIM><<<merge_blocks, 256, 0, s>>>(w, op, (int)pairs, (int)Sq, (int)splits, slot_cap, lay); \
    } while (0)
    if (D == 128) MRK_DECODE_DIM(128);
    else if (D == 64) MRK_DECODE_DIM(64);
    else if (D == 256) MRK_DECODE_DIM(256);
    else return (int)hipErrorInvalidValue;
#undef MRK_DECODE_DIM
#undef MRK_DECODE
#undef MRK_DECODE_QB
    return (int)hipGetLastError();
}

}  // namespace mrk
