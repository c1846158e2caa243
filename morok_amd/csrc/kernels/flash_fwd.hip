// Flash-attention forward for gfx950: O = softmax(Q K^T * scale [+ causal mask]) V in one
// kernel with an online softmax, bf16 operands, f32 scores / statistics / accumulators.
//
// Replaces the composed graph of Tensor::scaled_dot_product_attention
// (tensor/src/transformer.rs:78-137: matmul, scale, tril -> where(-inf), softmax, matmul),
// which the reference schedules as >= 6 kernels that materialise the [B,H,Sq,Sk] score
// tensor (tensor/src/test/unit/fusion.rs:90-104).  Causal rule as in the reference:
// key j is visible to query i iff j <= i (tril(0) over [Sq, Sk], transformer.rs:103-109).
//
// Layout: Q [BH, Sq, D], K [BH, Sk, D], V [BH, Sk, D], O [BH, Sq, D], row-major, D = 256, 128 or 64
// (one instantiation of the same body per head dim; the comments below give the D = 128 numbers).
//
// attn_mask and softcap (transformer.rs:112-132) run in instantiations of their own
// (flash_fwd_ext_*), in the reference's order: scale, causal where(-inf), mask (Bool: true =
// attend, else -inf added; float: added), then cap * tanh(score / cap).  The reference caps
// after masking, so under a softcap a masked score becomes -cap instead of -inf and still takes
// part in the softmax: those kernels visit every key tile and apply the causal rule per element.
//
// Work split: one workgroup = 128 queries of one (batch, head); 4 waves x 32 queries.
// K and V tiles of 64 keys travel global -> LDS directly (global_load_lds), two stages.
// Everything is computed transposed so that softmax statistics stay inside a lane:
//   S^T[key][q] = K_tile Q^T        MFMA 32x32x16, A = K rows from LDS, B = Q^T in registers
//   lane l owns query q = l % 32 and 16 of every 32 keys; the other 16 sit in lane l ^ 32
//   O^T[d][q]  += V^T P^T           A = V^T through the transposing LDS load, B = P^T taken
//                                   straight from the S^T accumulator registers
// The k index of the second product is whatever order the accumulator registers hold the
// keys in; the V^T fragment is fetched in that same order, so no register shuffle is needed.
#include <hip/hip_runtime.h>

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

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

constexpr int kQT = 128;       // queries per workgroup
constexpr int kKT = 64;        // keys per tile

// max(x of lane l, x of lane l ^ 32): the swap exchanges the upper 32 lanes of its first
// register with the lower 32 lanes of its second, which leaves one register holding the
// lower half twice and the other the upper half twice.
__device__ __forceinline__ float max_with_other_half(float x) {
    float a = x, b = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return fmaxf(a, b);
}

// Where the rows of one (batch, head) lie, in elements: the first row of head h of batch b is
// at b * batch + h * head, consecutive rows are `row` apart, the 128 elements of a row are
// contiguous.  With these a caller hands over views (a slice of a fused QKV product, a
// [batch, seq, heads, dim] activation) without copying them into [batch, heads, seq, dim].
struct RowLayout {
    long long batch, head;
    unsigned row_bytes;
};
struct FlashLayout {
    RowLayout q, k, v, o;
    int heads;
};

// attn_mask / softcap of the extended kernels.  The mask is a [batch, head, query, key] view
// with contiguous keys: element strides per batch, head and query row (0 = broadcast).
struct FlashExt {
    const void* mask;
    long long batch, head, row;
    float cap;        // softcap in score units (> 0 when the kernel applies one)
    int causal_elem;  // apply the causal rule per element while every key tile is visited
};

// kD: head dim, 128 or 64.  Rows of K and V are kD * 2 bytes in LDS (256 or 128): with 256-byte
// rows one row spans all 64 banks and the swizzles spread 16 consecutive rows over the 16-byte
// chunks; with 128-byte rows two consecutive rows span the banks, so the K swizzle uses
// (row >> 1) & 7 over the 8 chunks of a row and the V granule swizzle (row & 3 over 32-byte
// granules) needs no change.
// kMask: 0 none, 1 Bool (one byte per element, nonzero = attend), 2 additive bf16.  kCap: softcap.
template <int kD, bool kStrided, int kMask = 0, bool kCap = false>
__device__ __forceinline__ void flash_fwd_body(const __bf16* __restrict__ Q, const __bf16* __restrict__ K,
                                               const __bf16* __restrict__ V, __bf16* __restrict__ O, int BH, int Sq, int Sk,
                                               float scale_log2e, int causal, int q_tiles, int units, const FlashLayout& lay,
                                               const FlashExt& ext = FlashExt{}) {
    static_assert(kD == 256 || kD == 128 || kD == 64, "head dims with an instantiation: 256, 128 and 64");
    static_assert(kStrided || (kMask == 0 && !kCap), "the extended kernels take their operands as views");
    // The extended kernels turn every score into its final value in exp2 units (scale, masks,
    // softcap, log2 e) as soon as the score product has drained; from there on the online softmax
    // is the plain kernel's with a scale of one.
    constexpr bool kExt = kMask != 0 || kCap;
    const float sc = kExt ? 1.0f : scale_log2e;
    constexpr int kRow = kD * 2;          // bytes per K/V row in LDS: 256 (128)
    constexpr int kTile = kKT * kRow;     // 16 KB (8 KB)
    constexpr int kDS = kD / 16;          // 16-deep steps of the score product: 8 (4)
    constexpr int kDB = kD / 32;          // 32-row blocks of O^T: 4 (2)
    constexpr int kCh = kD / 8;           // 16-byte chunks per row: 16 (8)
    constexpr int kRowsPerDma = 64 / kCh; // rows one 1 KB copy covers: 4 (8)
    constexpr int kDmaPerWave = 16 / kRowsPerDma;  // copies per wave and tile: 4 (2)
    __shared__ __attribute__((aligned(1024))) char smem[4 * kTile];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroup ids congruent mod 8 run on the same XCD and share its L2.  Each XCD walks
    // its own heads one after another, all work units of a head back to back, so the units
    // of a head run concurrently and stream the head's K and V through that L2 once
    // instead of re-reading them from HBM per query tile.
    // A work unit is one query tile, or under the causal mask a pair (latest remaining
    // tile, earliest remaining tile): tile t costs about t+1 key steps, so every pair
    // costs the same and the workgroups of a launch finish together.
    int bh, unit;
    {
        const int bid = blockIdx.x;
        if ((BH & 7) == 0) {
            const int idx = bid >> 3;
            bh = (bid & 7) + 8 * (idx / units);
            unit = idx % units;
        } else {
            bh = bid / units;
            unit = bid % units;
        }
    }
    const int lq = lane & 31, lg = lane >> 5;
    const __bf16 *Qh, *Kh_, *Vh_;
    __bf16* Oh;
    unsigned q_row, k_row, v_row, o_row;  // bytes between consecutive rows
    const char* mask_row = nullptr;  // the mask of this (batch, head)
    if constexpr (kStrided) {
        const int bb = bh / lay.heads, hh = bh - bb * lay.heads;
        if constexpr (kMask != 0)
            mask_row = static_cast<const char*>(ext.mask) + (bb * ext.batch + hh * ext.head) * (kMask == 2 ? 2 : 1);
        Qh = Q + bb * lay.q.batch + hh * lay.q.head;
        Kh_ = K + bb * lay.k.batch + hh * lay.k.head;
        Vh_ = V + bb * lay.v.batch + hh * lay.v.head;
        Oh = O + bb * lay.o.batch + hh * lay.o.head;
        q_row = lay.q.row_bytes, k_row = lay.k.row_bytes, v_row = lay.v.row_bytes, o_row = lay.o.row_bytes;
    } else {
        Qh = Q + (size_t)bh * Sq * kD;
        Kh_ = K + (size_t)bh * Sk * kD;
        Vh_ = V + (size_t)bh * Sk * kD;
        Oh = O + (size_t)bh * Sq * kD;
        q_row = k_row = v_row = o_row = kRow;
    }
    const char* Kh = reinterpret_cast<const char*>(Kh_);
    const char* Vh = reinterpret_cast<const char*>(Vh_);
    const int first_qt = causal ? q_tiles - 1 - unit : unit;
    const int npass = (causal && unit != first_qt) ? 2 : 1;
    // key tiles a query tile visits
    auto tiles_of = [&](int qt) {
        int kend = Sk;
        if (causal && qt * kQT + kQT < kend) kend = qt * kQT + kQT;
        return (kend + kKT - 1) / kKT;
    };
    // The key tiles of the (up to) two passes form one sequence g = 0 .. ntot-1; the copies run
    // two (K) and one (V) tiles ahead along that sequence, across the pass boundary, and tile
    // g lives in LDS stage g & 1.
    const int n0 = tiles_of(first_qt), n1 = npass > 1 ? tiles_of(unit) : 0, ntot = n0 + n1;
    for (int pass = 0; pass < npass; pass++) {
    const int qt = pass == 0 ? first_qt : unit;
    const int q0 = qt * kQT;
    const int qw0 = q0 + wave * 32;  // first query of this wave
    const int ntiles = pass == 0 ? n0 : n1;
    const int base = pass == 0 ? 0 : n0;  // sequence index of this pass's tile 0

    // ---- direct global -> LDS tile copies.  One instruction = 1 KB = 4 rows of 256 B.
    // wave w copies rows 16w .. 16w+15 of both tiles (4 instructions each).
    const unsigned lds_base = (unsigned)(uintptr_t)LDS_PTR(char, smem);
    const int c16 = lane % kCh, r4 = lane / kCh;  // chunk inside the row, row inside the copy
    auto dma = [&](unsigned lds_addr, unsigned voff, const char* sbase) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_addr), "v"(voff), "s"(sbase)
                     : "m0");
    };
    // LDS map: K stage s at s*16 KB, V stage s at 32 KB + s*16 KB
    auto dma_k = [&](int j, int stage) {
#pragma unroll
        for (int c = 0; c < kDmaPerWave; c++) {
            const int row = wave * 16 + c * kRowsPerDma + r4;  // row inside the tile
            int key = j * kKT + row;
            key = key < Sk ? key : Sk - 1;  // ragged tail: re-read the last row, masked later
            // 16 B chunk c16 of the LDS row holds logical chunk c16 ^ (row & 15): the LDS
            // serves 16 lanes x 16 B per cycle over 64 banks, so 16 consecutive rows must
            // land in 16 different chunk slots (128-byte rows: c16 ^ ((row >> 1) & 7), the
            // parity of the row selects the half of the banks)
            const int ksw = kD >= 128 ? (row & 15) : ((row >> 1) & 7);
            const unsigned kvoff = (unsigned)key * k_row + ((c16 ^ ksw) << 4);
            dma(lds_base + stage * kTile + (wave * 16 + c * kRowsPerDma) * kRow, kvoff, Kh);
        }
    };
    auto dma_v = [&](int j, int stage) {
#pragma unroll
        for (int c = 0; c < kDmaPerWave; c++) {
            const int row = wave * 16 + c * kRowsPerDma + r4;
            int key = j * kKT + row;
            key = key < Sk ? key : Sk - 1;
            // 32 B granule (c16 >> 1) holds logical granule (c16 >> 1) ^ (row & 3)
            const unsigned vvoff = (unsigned)key * v_row + (((((c16 >> 1) ^ (row & 3)) << 1) | (c16 & 1)) << 4);
            dma(lds_base + 2 * kTile + stage * kTile + (wave * 16 + c * kRowsPerDma) * kRow, vvoff, Vh);
        }
    };
    auto tile_barrier = [&]() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    auto seq_k = [&](int g) {
        if (g < ntot) dma_k(g < n0 ? g : g - n0, g & 1);
    };
    auto seq_v = [&](int g) {
        if (g < ntot) dma_v(g < n0 ? g : g - n0, g & 1);
    };
    // the first pass starts its copies before anything else; a second pass finds its first
    // tiles already copied (or on their way) by the first
    if (pass == 0) {
        seq_k(0);
        seq_v(0);
        seq_k(1);
    }

    // ---- Q^T fragments: lane holds q = qw0 + l%32, d = 16*ds + 8*(l/32) .. +8
    bf16x8 qf[kDS];
    {
        int qrow = qw0 + lq;
        qrow = qrow < Sq ? qrow : Sq - 1;
        const __bf16* qp = Qh + (size_t)qrow * (q_row / 2) + 8 * lg;
#pragma unroll
        for (int ds = 0; ds < kDS; ds++) qf[ds] = *reinterpret_cast<const bf16x8*>(qp + 16 * ds);
        // Make the compiler wait for these loads here, before the loop: inside the loop the
        // only outstanding vector-memory operations must be the direct-to-LDS copies it does
        // not know about, which are drained explicitly in tile_barrier().
#pragma unroll
        for (int ds = 0; ds < kDS; ds++) asm volatile("" : "+v"(qf[ds]));
    }

    f32x16 o[kDB];
#pragma unroll
    for (int db = 0; db < kDB; db++)
#pragma unroll
        for (int e = 0; e < 16; e++) o[db][e] = 0.0f;
    float m_run = -INFINITY;  // running max of raw scores (before scale)
    float l_run = 0.0f;       // this lane's partial row sum
    const float lazy_thresh = 8.0f / sc;  // kLazy = 8: probabilities stay below 256

    // lane-constant LDS offsets
    // K fragment (A operand): row = kb*32 + l%32, logical chunk 2*ds + l/32
    const int k_row_off = lq * kRow;
    const int k_sw = kD >= 128 ? (lq & 15) : ((lq >> 1) & 7);
    // V^T fragment via transposing read: 16-lane block b = l/16 covers d half (b & 1) and
    // key group g = b >> 1; inside the block lane j' = l%16 points at key row j'/4,
    // 8-byte unit j'%4 of the 32-byte granule.
    const int v_rr = (lane & 15) >> 2;
    const int v_row_off = (4 * lg + v_rr) * kRow + 8 * (lane & 3);
    const int v_half = (lane >> 4) & 1;

    // first tile that needs masking for this wave: the causal diagonal (a tile is clear of
    // it iff its last key <= the wave's first query) or the ragged tail of the keys
    int first_masked = (Sk % kKT) ? Sk / kKT : ntiles;
    if ((causal || (kExt && ext.causal_elem)) && qw0 / kKT < first_masked) first_masked = qw0 / kKT;
    const int qidx = qw0 + lq;
    const int lim = causal ? (qidx < Sk - 1 ? qidx : Sk - 1) : Sk - 1;  // last visible key
    // ---- extended kernels: mask values of a tile and the score transform
    // A lane's 32 scores of a tile are eight groups of four consecutive keys (block kb, group g:
    // keys key0 + kb*32 + 8*g + 4*(l/32) + 0..3); the mask values of a group are one 8-byte
    // (bf16) or 4-byte (Bool) load.  Groups past the last key re-read the last group (Sk is a
    // multiple of 4 here) and are masked as non-existent keys afterwards.
    using MaskGroup = std::conditional_t<kMask == 2, bf16x4, unsigned>;
    struct MaskTile {
        MaskGroup g[2][4];
    };
    const char* mask_q = nullptr;  // this lane's query row of the mask (of this pass)
    if constexpr (kMask != 0) mask_q = mask_row + (long long)(qidx < Sq ? qidx : Sq - 1) * ext.row * (kMask == 2 ? 2 : 1);
    auto load_mask = [&](int key0, MaskTile& mt) {
        if constexpr (kMask != 0) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    int key = key0 + kb * 32 + 8 * g + 4 * lg;
                    key = key < Sk - 4 ? key : Sk - 4;
                    mt.g[kb][g] = *reinterpret_cast<const MaskGroup*>(mask_q + (long long)key * (kMask == 2 ? 2 : 1));
                }
        }
    };
    const int lim_causal = ext.causal_elem ? qidx : 0x7fffffff;  // reference mask: -inf before the softcap
    constexpr float kLog2e = 1.4426950408889634f;
    const float cap_out = kCap ? ext.cap * kLog2e : 0.0f;  // the cap in exp2 units
    const float cap_in = kCap ? 2.0f / ext.cap : 0.0f;
    // raw score (sum of q k) of key `key` -> final score in exp2 units
    // `limits`: the tile touches the causal diagonal or the end of the keys (the others skip the compares)
    auto ext_score = [&](float s, int key, const MaskTile& mt, int kb, int e, bool limits) -> float {
        float t = s * scale_log2e;  // scaled score, in exp2 units for now
        // without a softcap -inf before or after the mask is the same thing: one compare against the
        // smaller limit; with one the causal limit applies here and the end of the keys after the cap
        if (limits && key > (kCap ? lim_causal : (lim_causal < Sk - 1 ? lim_causal : Sk - 1))) t = -INFINITY;
        if constexpr (kMask == 1) {
            if (((mt.g[kb][e >> 2] >> (8 * (e & 3))) & 0xffu) == 0) t = -INFINITY;
        } else if constexpr (kMask == 2) {
            t += (float)mt.g[kb][e >> 2][e & 3] * kLog2e;
        }
        if constexpr (kCap) {
            // cap * tanh(x / cap) with tanh(y) = 1 - 2 / (exp(2 y) + 1) and x = t / log2 e, so
            // exp(2 x / cap) = exp2(2 t / cap); x = -inf gives -cap, x = +inf gives cap
            const float z = __builtin_amdgcn_exp2f(t * cap_in);
            t = cap_out * (1.0f - 2.0f * __builtin_amdgcn_rcpf(z + 1.0f));
        }
        if (kCap && limits && key > Sk - 1) t = -INFINITY;  // keys that do not exist
        return t;
    };

    // S^T = K Q^T for one tile (K fragments fetched one d-step ahead of their MFMAs),
    // then the mask and the row maximum.  Register e of block kb is key
    // key0 + kb*32 + 8*(e/4) + 4*(l/32) + e%4.
    auto qk_tile = [&](const char* sK, f32x16 (&st)[2]) {
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int e = 0; e < 16; e++) st[kb][e] = 0.0f;
        bf16x8 kf[2][2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
            kf[0][kb] = *LDS_PTR(bf16x8, sK + kb * 32 * kRow + k_row_off + (((0 + lg) ^ k_sw) << 4));
#pragma unroll
        for (int ds = 0; ds < kDS; ds++) {
            if (ds + 1 < kDS) {
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
                    kf[(ds + 1) & 1][kb] =
                        *LDS_PTR(bf16x8, sK + kb * 32 * kRow + k_row_off + (((2 * (ds + 1) + lg) ^ k_sw) << 4));
            }
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
                st[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ds & 1][kb], qf[ds], st[kb], 0, 0, 0);
        }
    };
    auto mask_and_max = [&](f32x16 (&st)[2], int key0, bool mask) -> float {
        if constexpr (kExt) {
            MaskTile mt;
            load_mask(key0, mt);
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int e = 0; e < 16; e++)
                    st[kb][e] = ext_score(st[kb][e], key0 + kb * 32 + 8 * (e >> 2) + 4 * lg + (e & 3), mt, kb, e, mask);
        } else if (mask) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int key = key0 + kb * 32 + 8 * (e >> 2) + 4 * lg + (e & 3);
                    if (key > lim) st[kb][e] = -INFINITY;
                }
        }
        float mx0 = st[0][0], mx1 = st[1][0];
#pragma unroll
        for (int e = 1; e < 16; e++) {
            mx0 = fmaxf(mx0, st[0][e]);
            mx1 = fmaxf(mx1, st[1][e]);
        }
        const float mx = fmaxf(mx0, mx1);
        // the other 16 keys of every 32 sit in lane l ^ 32
        return max_with_other_half(mx);
    };

    // One loop iteration, software-pipelined inside the wave: while the matrix pipe runs
    // S(j+1) = K(j+1) Q^T the vector ALUs turn S(j) into P(j); while it runs
    // O += V(j)^T P(j)^T they find the row maximum of S(j+1).  The iteration starts with the
    // (rare) rescale decided by that maximum, so the pipelined part is one basic block.
    // Lazy rescaling: exponentials are taken relative to m_run, which only moves (and the
    // accumulators are rescaled) when some row's maximum has grown by more than
    // kLazy / scale_log2e, i.e. when a probability could exceed 2^kLazy.  Rounding P to bf16
    // is relative and the row sum is f32, so the result does not depend on the reference
    // point.  The first tile always rescales (m_run = -inf); key 0 is visible to every
    // query, so m_run is finite from then on.
    auto body = [&](int j, f32x16 (&cur)[2], float mx_cur, f32x16 (&nxt)[2], float& mx_nxt, auto mask_next, auto last_tile) {
        constexpr bool kLast = decltype(last_tile)::value;  // the wave's last tile: there is no S(j+1) to compute
        if (__builtin_amdgcn_ballot_w64(mx_cur > m_run + lazy_thresh) != 0) {
            const float m_new = fmaxf(m_run, mx_cur);
            // (a row with nothing visible yet keeps -inf: its empty accumulators are left as they are)
            const float alpha = kExt && m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f((m_run - m_new) * sc);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < kDB; db++) o[db] *= alpha;
        }
        // K(j+1) and V(j) have landed; every wave is done with K(j) and V(j-1)
        tile_barrier();
        const int g = base + j;
        // (the copies go out at the highest priority of the iteration: the sooner all four waves have issued theirs,
        // the longer the tiles have to land; +0.9 % over issuing them at the previous phase's priority)
        __builtin_amdgcn_s_setprio(2);
        seq_k(g + 2);
        seq_v(g + 1);
        const char* sKn = smem + ((g + 1) & 1) * kTile;
        const char* sV = smem + 2 * kTile + (g & 1) * kTile;
        // (a row whose keys so far are all masked has m_run = -inf: its probabilities must come out as 0, not NaN)
        const float mb = kExt && m_run == -INFINITY ? 0.0f : m_run * sc;

        // (the wave asks for the SIMD's issue slots first while it is in this phase, the one with the
        // exponentials: with two waves per SIMD that measured +0.5 to +2 % at D = 128 and up to +3.7 % at D = 64
        // over leaving both phases at one priority; raising the other phase instead measured nothing)
        __builtin_amdgcn_s_setprio(1);
        // ---- phase A: S(j+1) = K(j+1) Q^T on the matrix pipe, P(j) = exp2(S(j)*c - m*c) on
        // the vector ALUs: each of the 16 (8; 32) MFMAs is followed by the exponentials of two (four; every second one by two)
        // score registers (a wave's last tile has no successor: that instantiation runs the exponentials alone).  The fences keep the
        // compiler from regrouping the two instruction streams.
        float psum0 = 0.0f, psum1 = 0.0f;
        bf16x8 pb[2][2];
        {
            bf16x8 kf[2][2];
            if constexpr (!kLast) {
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
#pragma unroll
                    for (int e = 0; e < 16; e++) nxt[kb][e] = 0.0f;
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
                    kf[0][kb] = *LDS_PTR(bf16x8, sKn + kb * 32 * kRow + k_row_off + (((0 + lg) ^ k_sw) << 4));
            }
            f32x8 p;
            constexpr int kMfmaA = 2 * kDS;  // score MFMAs of this phase; the 16 pairs of score registers are spread over them:
                                             // one per MFMA (D = 128), two (64), one after every second (256)
#pragma unroll
            for (int ds = 0; ds < kDS; ds++) {
                if constexpr (!kLast) {
                    if (ds + 1 < kDS) {
#pragma unroll
                        for (int kb = 0; kb < 2; kb++)
                            kf[(ds + 1) & 1][kb] =
                                *LDS_PTR(bf16x8, sKn + kb * 32 * kRow + k_row_off + (((2 * (ds + 1) + lg) ^ k_sw) << 4));
                    }
                }
#pragma unroll
                for (int kb = 0; kb < 2; kb++) {
                    if constexpr (!kLast)
                        nxt[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ds & 1][kb], qf[ds], nxt[kb], 0, 0, 0);
#pragma unroll
                    for (int idx = (ds * 2 + kb) * 16 / kMfmaA; idx < (ds * 2 + kb + 1) * 16 / kMfmaA; idx++) {  // 0..15: score registers 2*idx, 2*idx+1
                        const int pk = idx >> 3, pe = (idx & 7) * 2;  // block, register inside the block
                        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(cur[pk][pe], sc, -mb));
                        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(cur[pk][pe + 1], sc, -mb));
                        psum0 += p0;
                        psum1 += p1;
                        p[pe & 7] = p0;
                        p[(pe & 7) + 1] = p1;
                        if ((idx & 3) == 3) pb[pk][(idx >> 2) & 1] = __builtin_convertvector(p, bf16x8);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        l_run += psum0 + psum1;
        __builtin_amdgcn_s_setprio(0);

        // ---- phase B: O^T += V(j)^T P(j)^T on the matrix pipe, mask and row maximum of
        // S(j+1) on the vector ALUs.  MFMA (kb, t) contracts over the 16 keys held in
        // registers 8t .. 8t+7 of block kb: keys kb*32 + 16t + {0, 8} + 4*(l/32) + 0..3.
        float mx0 = -INFINITY, mx1 = -INFINITY;
        {
            constexpr int kNB = 4 * kDB;  // MFMAs of this phase: 16 (8)
            MaskTile mt;  // the next tile's mask values: requested here, used in the second half of the phase
            if constexpr (kExt && !kLast) load_mask((j + 1) * kKT, mt);
            auto vfrag = [&](int n) {  // n = (kb*2 + t)*kDB + db
                const int kbt = n / kDB, db = n % kDB;
                const int off = (kbt * 16) * kRow + v_row_off + (((db * 2 + v_half) ^ v_rr) << 5);
                bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sV + off));
                bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(LDS_PTR(bf16x4, sV + off + 8 * kRow));
                return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            };
            bf16x8 vf[3];
            vf[0] = vfrag(0);
            vf[1] = vfrag(1);
            const int key0n = (j + 1) * kKT;
#pragma unroll
            for (int n = 0; n < kNB; n++) {
                if (n + 2 < kNB) vf[(n + 2) % 3] = vfrag(n + 2);
                const int kbt = n / kDB, db = n % kDB;
                o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[n % 3], pb[kbt >> 1][kbt & 1], o[db], 0, 0, 0);
                if (!kLast && n >= kNB / 2) {  // the score MFMAs have drained by now: 4 (8) registers per slot
                    constexpr int kSlotsPerKb = kNB / 4, kRegs = 16 / kSlotsPerKb;
                    const int kb = (n - kNB / 2) / kSlotsPerKb, e0 = ((n - kNB / 2) % kSlotsPerKb) * kRegs;
#pragma unroll
                    for (int e = e0; e < e0 + kRegs; e++) {
                        if constexpr (kExt) {
                            nxt[kb][e] = ext_score(nxt[kb][e], key0n + kb * 32 + 8 * (e >> 2) + 4 * lg + (e & 3), mt, kb, e, decltype(mask_next)::value);
                        } else if (decltype(mask_next)::value) {
                            const int key = key0n + kb * 32 + 8 * (e >> 2) + 4 * lg + (e & 3);
                            if (key > lim) nxt[kb][e] = -INFINITY;
                        }
                        if (e & 1) mx1 = fmaxf(mx1, nxt[kb][e]);
                        else mx0 = fmaxf(mx0, nxt[kb][e]);
                    }
                    // pins the partial maxima to this slot (pure operations are otherwise
                    // free to sink below the last MFMA)
                    asm volatile("" : "+v"(mx0), "+v"(mx1));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if constexpr (!kLast) {
            const float mx = fmaxf(mx0, mx1);
            // the other 16 keys of every 32 sit in lane l ^ 32
            mx_nxt = max_with_other_half(mx);
        }
    };

    if (pass == 0) tile_barrier();
    f32x16 sa[2], sb[2];
    float mxa, mxb = 0.0f;
    qk_tile(smem + (base & 1) * kTile, sa);
    mxa = mask_and_max(sa, 0, first_masked <= 0);
    {
        int j = 0;
        // under the causal mask the tiles past the wave's own diagonal are invisible to it: it
        // only keeps the barrier rhythm and copies its share of them for the other waves
        int nmine = ntiles;
        if (causal && (qw0 + 31) / kKT + 1 < nmine) nmine = (qw0 + 31) / kKT + 1;
        constexpr std::false_type more{};
        if constexpr (kD < 256) {
            const int nl = nmine - 1;  // iterations that have a next tile; the wave's last one is a body of its own
            const int jm = first_masked - 1 < nl ? first_masked - 1 : nl;  // iterations whose next tile is unmasked
            for (; j + 1 < jm; j += 2) {
                body(j, sa, mxa, sb, mxb, std::false_type{}, more);
                body(j + 1, sb, mxb, sa, mxa, std::false_type{}, more);
            }
            if (j < jm) {
                body(j, sa, mxa, sb, mxb, std::false_type{}, more);
                sa[0] = sb[0];
                sa[1] = sb[1];
                mxa = mxb;
                j++;
            }
            for (; j + 1 < nl; j += 2) {
                body(j, sa, mxa, sb, mxb, std::true_type{}, more);
                body(j + 1, sb, mxb, sa, mxa, std::true_type{}, more);
            }
            if (j < nl) {
                body(j, sa, mxa, sb, mxb, std::true_type{}, more);
                sa[0] = sb[0];
                sa[1] = sb[1];
                mxa = mxb;
                j++;
            }
            body(j, sa, mxa, sb, mxb, std::false_type{}, std::true_type{});
            j++;
        } else {
            // with 512-byte rows one more instantiation of the body would push the kernel over
            // its register budget: the last tile runs the ordinary body and its S(j+1) goes unused
            const int jm = first_masked - 1 < nmine ? first_masked - 1 : nmine;
            for (; j + 1 < jm; j += 2) {
                body(j, sa, mxa, sb, mxb, std::false_type{}, more);
                body(j + 1, sb, mxb, sa, mxa, std::false_type{}, more);
            }
            if (j < jm) {
                body(j, sa, mxa, sb, mxb, std::false_type{}, more);
                sa[0] = sb[0];
                sa[1] = sb[1];
                mxa = mxb;
                j++;
            }
            for (; j + 1 < nmine; j += 2) {
                body(j, sa, mxa, sb, mxb, std::true_type{}, more);
                body(j + 1, sb, mxb, sa, mxa, std::true_type{}, more);
            }
            if (j < nmine) {
                body(j, sa, mxa, sb, mxb, std::true_type{}, more);
                j++;
            }
        }
        for (; j < ntiles; j++) {
            tile_barrier();
            seq_k(base + j + 2);
            seq_v(base + j + 1);
        }
    }

    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // ---- normalise and store: lane holds O[q = qw0 + l%32][d = db*32 + 8*(e/4) + 4*(l/32) + e%4]
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const float inv = 1.0f / l_tot;
    const int qrow = qw0 + lq;
    if (qrow < Sq) {
        __bf16* op = Oh + (size_t)qrow * (o_row / 2) + 4 * lg;
#pragma unroll
        for (int db = 0; db < kDB; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                f32x4 v = {o[db][4 * g] * inv, o[db][4 * g + 1] * inv, o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv};
                *reinterpret_cast<bf16x4*>(op + db * 32 + 8 * g) = __builtin_convertvector(v, bf16x4);
            }
    }
    }  // pass
}

__global__ __launch_bounds__(256, 2) void flash_fwd_d128(const __bf16* __restrict__ Q, const __bf16* __restrict__ K,
                                                         const __bf16* __restrict__ V, __bf16* __restrict__ O, int BH,
                                                         int Sq, int Sk, float scale_log2e, int causal, int q_tiles, int units) {
    flash_fwd_body<128, false>(Q, K, V, O, BH, Sq, Sk, scale_log2e, causal, q_tiles, units, FlashLayout{});
}
__global__ __launch_bounds__(256, 2) void flash_fwd_d64(const __bf16* __restrict__ Q, const __bf16* __restrict__ K,
                                                        const __bf16* __restrict__ V, __bf16* __restrict__ O, int BH,
                                                        int Sq, int Sk, float scale_log2e, int causal, int q_tiles, int units) {
    flash_fwd_body<64, false>(Q, K, V, O, BH, Sq, Sk, scale_log2e, causal, q_tiles, units, FlashLayout{});
}

__global__ __launch_bounds__(256, 2) void flash_fwd_d128_strided(const __bf16* __restrict__ Q, const __bf16* __restrict__ K,
                                                                 const __bf16* __restrict__ V, __bf16* __restrict__ O,
                                                                 int BH, int Sq, int Sk, float scale_log2e, int causal,
                                                                 int q_tiles, int units, FlashLayout lay) {
    flash_fwd_body<128, true>(Q, K, V, O, BH, Sq, Sk, scale_log2e, causal, q_tiles, units, lay);
}
__global__ __launch_bounds__(256, 2) void flash_fwd_d64_strided(const __bf16* __restrict__ Q, const __bf16* __restrict__ K,
                                                                const __bf16* __restrict__ V, __bf16* __restrict__ O, int BH,
                                                                int Sq, int Sk, float scale_log2e, int causal, int q_tiles,
                                                                int units, FlashLayout lay) {
    flash_fwd_body<64, true>(Q, K, V, O, BH, Sq, Sk, scale_log2e, causal, q_tiles, units, lay);
}

// 512-byte rows: one workgroup's four tiles fill 128 KB of LDS, one workgroup per CU
__global__ __launch_bounds__(256, 1) void flash_fwd_d256(const __bf16* __restrict__ Q, const __bf16* __restrict__ K,
                                                         const __bf16* __restrict__ V, __bf16* __restrict__ O, int BH,
                                                         int Sq, int Sk, float scale_log2e, int causal, int q_tiles, int units) {
    flash_fwd_body<256, false>(Q, K, V, O, BH, Sq, Sk, scale_log2e, causal, q_tiles, units, FlashLayout{});
}
__global__ __launch_bounds__(256, 1) void flash_fwd_d256_strided(const __bf16* __restrict__ Q, const __bf16* __restrict__ K,
                                                                 const __bf16* __restrict__ V, __bf16* __restrict__ O, int BH,
                                                                 int Sq, int Sk, float scale_log2e, int causal, int q_tiles,
                                                                 int units, FlashLayout lay) {
    flash_fwd_body<256, true>(Q, K, V, O, BH, Sq, Sk, scale_log2e, causal, q_tiles, units, lay);
}

// attn_mask / softcap instantiations; operands always as views
#define MRK_FLASH_EXT_KERNEL(NAME, D, WG, MASK, CAP)                                                                            \
    __global__ __launch_bounds__(256, WG) void NAME(const __bf16* __restrict__ Q, const __bf16* __restrict__ K,                   \
                                                    const __bf16* __restrict__ V, __bf16* __restrict__ O, int BH, int Sq, int Sk, \
                                                    float scale_log2e, int causal, int q_tiles, int units, FlashLayout lay,       \
                                                    FlashExt ext) {                                                               \
        flash_fwd_body<D, true, MASK, CAP>(Q, K, V, O, BH, Sq, Sk, scale_log2e, causal, q_tiles, units, lay, ext);                \
    }
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d128_bool, 128, 2, 1, false)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d128_add, 128, 2, 2, false)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d128_cap, 128, 2, 0, true)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d128_bool_cap, 128, 2, 1, true)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d128_add_cap, 128, 2, 2, true)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d64_bool, 64, 2, 1, false)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d64_add, 64, 2, 2, false)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d64_cap, 64, 2, 0, true)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d64_bool_cap, 64, 2, 1, true)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d64_add_cap, 64, 2, 2, true)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d256_bool, 256, 1, 1, false)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d256_add, 256, 1, 2, false)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d256_cap, 256, 1, 0, true)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d256_bool_cap, 256, 1, 1, true)
MRK_FLASH_EXT_KERNEL(flash_fwd_ext_d256_add_cap, 256, 1, 2, true)
#undef MRK_FLASH_EXT_KERNEL

}  // namespace mrk::dev

namespace mrk {

// A handful of queries against a long key sequence: the kernel that splits the keys (flash_decode.hip), in as many
// ranges as the workspace allows (one range needs none).
static bool decode_route(void* stream, const void* q, const void* k, const void* v, void* o, long B, long H, long Sq, long Sk, long D,
                         float scale, int causal, const long* strides, void* workspace, size_t workspace_bytes, int* rc,
                         const void* mask = nullptr, int mask_kind = 0, const long* mask_strides = nullptr, float softcap = 0.0f) {
    using namespace mrk::dev;
    // heads that share K and V (zero head strides) become query slots of one pair: K and V are read once per batch
    // (runs of consecutive heads: the largest divisor of the head count that gives at most 32 slots)
    long group = 1;
    if (H > 1 && strides[4] == 0 && strides[7] == 0 && Sq >= 1)
        for (long g = 32 / Sq; g > 1; g--)
            if (H % g == 0) {
                group = g;
                break;
            }
    const long pairs = B * (H / group), slots = group * Sq;
    long splits = 0, per = 0;
    if (!flash_decode_plan(pairs, slots, Sk, D, causal, &splits, &per)) return false;
    const void* ptrs[4] = {q, k, v, o};
    for (const void* p : ptrs)
        if (reinterpret_cast<uintptr_t>(p) % 16) return false;
    if (splits > 1) {  // as many key ranges as the workspace holds
        const size_t slice = (size_t)pairs * flash_decode_slot_capacity(slots) * (D + 2) * sizeof(float);
        const long fit = workspace ? (long)(workspace_bytes / slice) : 0;
        if (fit < splits) {
            const long want = fit < 2 ? 1 : fit;
            per = ((Sk + want - 1) / want + 31) / 32 * 32;
            splits = (Sk + per - 1) / per;
        }
    }
    *rc = launch_flash_decode(stream, q, k, v, o, B, H, Sq, Sk, D, scale, strides, splits, per, workspace, mask, mask_kind, mask_strides,
                              softcap, group);
    return true;
}

int launch_flash_fwd_bf16(void* stream, const void* q, const void* k, const void* v, void* o, long BH, long Sq, long Sk,
                          long D, float scale, int causal, void* workspace, size_t workspace_bytes) {
    using namespace mrk::dev;
    if (BH <= 0 || Sq <= 0) return 0;
    if ((D != 256 && D != 128 && D != 64) || Sk <= 0 || !(scale > 0.0f)) return (int)hipErrorInvalidValue;
    if (Sq > (1L << 24) || Sk > (1L << 24) || BH > (1L << 24)) return (int)hipErrorInvalidValue;
    // row offsets inside a head are formed in 32 bits (row * row bytes): the last row must end below 4 GiB
    if (!flash_fwd_rows_addressable(Sq, D * 2, D) || !flash_fwd_rows_addressable(Sk, D * 2, D)) return (int)hipErrorInvalidValue;
    {
        const long dense[12] = {Sq * D, 0, D, Sk * D, 0, D, Sk * D, 0, D, Sq * D, 0, D};  // (batch * head, -, row) per operand
        int rc = 0;
        if (decode_route(stream, q, k, v, o, BH, 1, Sq, Sk, D, scale, causal, dense, workspace, workspace_bytes, &rc)) return rc;
    }
    const long q_tiles = (Sq + kQT - 1) / kQT;
    const long units = causal ? (q_tiles + 1) / 2 : q_tiles;
    const long blocks = BH * units;
    if (blocks > 0x7fffffffL) return (int)hipErrorInvalidValue;
    (void)hipGetLastError();
    const float scale_log2e = scale * 1.4426950408889634f;
    auto kernel = D == 256 ? flash_fwd_d256 : D == 128 ? flash_fwd_d128 : flash_fwd_d64;
    kernel<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const __bf16*>(q), static_cast<const __bf16*>(k), static_cast<const __bf16*>(v),
        static_cast<__bf16*>(o), (int)BH, (int)Sq, (int)Sk, scale_log2e, causal, (int)q_tiles, (int)units);
    return (int)hipGetLastError();
}

int launch_flash_fwd_bf16_strided(void* stream, const void* q, const void* k, const void* v, void* o, long B, long H, long Sq,
                                  long Sk, long D, float scale, int causal, const long* strides, void* workspace, size_t workspace_bytes) {
    using namespace mrk::dev;
    if (B < 0 || H < 0 || !strides) return (int)hipErrorInvalidValue;
    const long BH = B * H;
    if (BH == 0 || Sq <= 0) return 0;
    if ((D != 256 && D != 128 && D != 64) || Sk <= 0 || !(scale > 0.0f)) return (int)hipErrorInvalidValue;
    if (Sq > (1L << 24) || Sk > (1L << 24) || BH > (1L << 24)) return (int)hipErrorInvalidValue;
    // strides: (batch, head, row) of q, k, v, o in elements.  Rows are read and written in
    // 16-byte pieces from 16-byte aligned addresses; row offsets inside a head are 32-bit
    const void* ptrs[4] = {q, k, v, o};
    const long rows[4] = {Sq, Sk, Sk, Sq};
    bool dense = true;
    for (int t = 0; t < 4; t++) {
        const long sb = strides[3 * t], sh = strides[3 * t + 1], sr = strides[3 * t + 2];
        if (sb < 0 || sh < 0 || sr < 0 || sb % 8 || sh % 8 || sr % 8) return (int)hipErrorInvalidValue;
        if (reinterpret_cast<uintptr_t>(ptrs[t]) % 16) return (int)hipErrorInvalidValue;
        if (sr > (1L << 30) || !flash_fwd_rows_addressable(rows[t], sr * 2, D)) return (int)hipErrorInvalidValue;
        // the output must not alias itself: distinct rows, heads and batches at distinct places
        // (the stride of an axis of extent one is never multiplied by anything but zero: any value will do)
        if (t == 3 && ((Sq > 1 && sr < D) || (H > 1 && sh == 0) || (B > 1 && sb == 0))) return (int)hipErrorInvalidValue;
        dense = dense && sr == D && sh == rows[t] * D && sb == H * rows[t] * D;
    }
    if (dense) return launch_flash_fwd_bf16(stream, q, k, v, o, BH, Sq, Sk, D, scale, causal, workspace, workspace_bytes);
    {
        int rc = 0;
        if (decode_route(stream, q, k, v, o, B, H, Sq, Sk, D, scale, causal, strides, workspace, workspace_bytes, &rc)) return rc;
    }
    const long q_tiles = (Sq + kQT - 1) / kQT;
    const long units = causal ? (q_tiles + 1) / 2 : q_tiles;
    const long blocks = BH * units;
    if (blocks > 0x7fffffffL) return (int)hipErrorInvalidValue;
    FlashLayout lay;
    RowLayout* rl[4] = {&lay.q, &lay.k, &lay.v, &lay.o};
    for (int t = 0; t < 4; t++) {
        rl[t]->batch = strides[3 * t];
        rl[t]->head = strides[3 * t + 1];
        rl[t]->row_bytes = (unsigned)(strides[3 * t + 2] * 2);
    }
    lay.heads = (int)H;
    (void)hipGetLastError();
    const float scale_log2e = scale * 1.4426950408889634f;
    auto kernel = D == 256 ? flash_fwd_d256_strided : D == 128 ? flash_fwd_d128_strided : flash_fwd_d64_strided;
    kernel<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const __bf16*>(q), static_cast<const __bf16*>(k), static_cast<const __bf16*>(v),
        static_cast<__bf16*>(o), (int)BH, (int)Sq, (int)Sk, scale_log2e, causal, (int)q_tiles, (int)units, lay);
    return (int)hipGetLastError();
}

int launch_flash_fwd_bf16_ext(void* stream, const void* q, const void* k, const void* v, void* o, long B, long H, long Sq, long Sk,
                              long D, float scale, int causal, const long* strides, const void* mask, int mask_kind,
                              const long* mask_strides, float softcap, void* workspace, size_t workspace_bytes) {
    using namespace mrk::dev;
    if (B < 0 || H < 0 || !strides) return (int)hipErrorInvalidValue;
    if (mask_kind < 0 || mask_kind > 2 || (mask_kind != 0 && (!mask || !mask_strides)) || !(softcap >= 0.0f)) return (int)hipErrorInvalidValue;
    if (mask_kind == 0 && !(softcap > 0.0f))
        return launch_flash_fwd_bf16_strided(stream, q, k, v, o, B, H, Sq, Sk, D, scale, causal, strides, workspace, workspace_bytes);
    const long BH = B * H;
    if (BH == 0 || Sq <= 0) return 0;
    if ((D != 256 && D != 128 && D != 64) || Sk <= 0 || !(scale > 0.0f)) return (int)hipErrorInvalidValue;
    if (Sq > (1L << 24) || Sk > (1L << 24) || BH > (1L << 24)) return (int)hipErrorInvalidValue;
    const void* ptrs[4] = {q, k, v, o};
    const long rows[4] = {Sq, Sk, Sk, Sq};
    for (int t = 0; t < 4; t++) {
        const long sb = strides[3 * t], sh = strides[3 * t + 1], sr = strides[3 * t + 2];
        if (sb < 0 || sh < 0 || sr < 0 || sb % 8 || sh % 8 || sr % 8) return (int)hipErrorInvalidValue;
        if (reinterpret_cast<uintptr_t>(ptrs[t]) % 16) return (int)hipErrorInvalidValue;
        if (sr > (1L << 30) || !flash_fwd_rows_addressable(rows[t], sr * 2, D)) return (int)hipErrorInvalidValue;
        // (the stride of an axis of extent one is never multiplied by anything but zero: any value will do)
        if (t == 3 && ((Sq > 1 && sr < D) || (H > 1 && sh == 0) || (B > 1 && sb == 0))) return (int)hipErrorInvalidValue;
    }
    FlashExt ext{};
    if (mask_kind != 0) {
        // a lane reads the mask in groups of four keys: rows, heads and batches start on multiples of
        // four elements, and so does the end of a row
        const long esize = mask_kind == 2 ? 2 : 1;
        if (Sk % 4 || reinterpret_cast<uintptr_t>(mask) % (4 * esize)) return (int)hipErrorInvalidValue;
        for (int i = 0; i < 3; i++)
            if (mask_strides[i] < 0 || mask_strides[i] % 4) return (int)hipErrorInvalidValue;
        ext.mask = mask;
        ext.batch = mask_strides[0], ext.head = mask_strides[1], ext.row = mask_strides[2];
    }
    const bool cap = softcap > 0.0f;
    {  // a handful of queries without the causal rule: the kernel that splits the keys
        int rc = 0;
        if (decode_route(stream, q, k, v, o, B, H, Sq, Sk, D, scale, causal, strides, workspace, workspace_bytes, &rc, mask, mask_kind, mask_strides,
                         softcap))
            return rc;
    }
    ext.cap = softcap;
    ext.causal_elem = causal ? 1 : 0;
    // under a softcap a causally masked score becomes -cap and still counts: every key tile is visited
    const int causal_tiles = causal && !cap;
    const long q_tiles = (Sq + kQT - 1) / kQT;
    const long units = causal_tiles ? (q_tiles + 1) / 2 : q_tiles;
    const long blocks = BH * units;
    if (blocks > 0x7fffffffL) return (int)hipErrorInvalidValue;
    FlashLayout lay;
    RowLayout* rl[4] = {&lay.q, &lay.k, &lay.v, &lay.o};
    for (int t = 0; t < 4; t++) {
        rl[t]->batch = strides[3 * t];
        rl[t]->head = strides[3 * t + 1];
        rl[t]->row_bytes = (unsigned)(strides[3 * t + 2] * 2);
    }
    lay.heads = (int)H;
    (void)hipGetLastError();
    const float scale_log2e = scale * 1.4426950408889634f;
    using Kernel = void (*)(const __bf16*, const __bf16*, const __bf16*, __bf16*, int, int, int, float, int, int, int, FlashLayout, FlashExt);
    // [head dim][mask kind][cap]
    static const Kernel table[3][3][2] = {
        {{nullptr, flash_fwd_ext_d64_cap}, {flash_fwd_ext_d64_bool, flash_fwd_ext_d64_bool_cap}, {flash_fwd_ext_d64_add, flash_fwd_ext_d64_add_cap}},
        {{nullptr, flash_fwd_ext_d128_cap}, {flash_fwd_ext_d128_bool, flash_fwd_ext_d128_bool_cap}, {flash_fwd_ext_d128_add, flash_fwd_ext_d128_add_cap}},
        {{nullptr, flash_fwd_ext_d256_cap}, {flash_fwd_ext_d256_bool, flash_fwd_ext_d256_bool_cap}, {flash_fwd_ext_d256_add, flash_fwd_ext_d256_add_cap}}};
    const Kernel kernel = table[D == 64 ? 0 : D == 128 ? 1 : 2][mask_kind][cap ? 1 : 0];
    kernel<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const __bf16*>(q), static_cast<const __bf16*>(k), static_cast<const __bf16*>(v), static_cast<__bf16*>(o), (int)BH,
        (int)Sq, (int)Sk, scale_log2e, causal_tiles, (int)q_tiles, (int)units, lay, ext);
    return (int)hipGetLastError();
}

}  // namespace mrk
