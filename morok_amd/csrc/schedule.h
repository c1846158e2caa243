// Host-side scheduling pieces the HIP backend needs from morok's `schedule` crate, restated
// for gfx950: renderer capability descriptor and tensor-core tables
// (schedule/src/optimizer/renderer.rs:80-129,290-303,358-417,538-558,724-733), tensor-core
// selection and operand layouts (schedule/src/optimizer/tc.rs:126-236,621-638), GPU dimension
// limiting (schedule/src/gpudims.rs:387-463,529-642) and builders of the linearized kernels
// the optimizer would hand to the renderer for the matmul shapes on the hot path.
#pragma once
#include <array>
#include <string>
#include <unordered_map>
#include <vector>

#include "uop.h"

namespace mrk {

struct TcOpt {
    char kind;  // 'l' local, 'u' upcast
    int axis;   // 0 = N, 1 = M
};
struct SwizzleAxis {
    char kind;  // 'l', 'u', 'r'
    int idx;
};

// renderer.rs:358-417
struct TensorCore {
    std::array<int, 3> dims;  // (N, M, K)
    int threads;
    std::array<int, 3> elements_per_thread;  // (A, B, C) elements held by one lane
    Scalar dtype_in, dtype_out;
    std::vector<TcOpt> opts;
    // ((A_local, A_upcast, A_reduce), (B_local, B_upcast, B_reduce))
    std::array<std::array<std::vector<SwizzleAxis>, 3>, 2> swizzle;
};

// renderer.rs:80-129
struct RendererCaps {
    std::string device;
    bool has_local = false, has_shared = false, has_threads = false;
    size_t shared_max = 0;
    std::vector<size_t> global_max;
    size_t local_max = 0;
    size_t upcast_max = 0;
    std::vector<TensorCore> tensor_cores;
};

// renderer.rs:290-303 with two corrections for the real part: gfx950 has 160 KB of LDS per
// workgroup (the reference lists 65536) - everything else as upstream.
RendererCaps amd_cdna4_caps();
// renderer.rs:724-733 entry for entry, then the 32x32x16 shape of gfx950 for f16 and bf16
std::vector<TensorCore> cdna4_tensor_cores();
// tc.rs:126-168: first table entry whose input and accumulator dtypes match; -1 if none.
int select_tensor_core(const std::vector<TensorCore>& tcs, Scalar in0, Scalar in1, Scalar acc);
// tc.rs:621-638,677-688: WMMA_{N}_{M}_{K}_{in}_{out}
std::string wmma_name(const TensorCore& tc);

// Where a lane's operand element comes from, derived from opts + swizzle exactly as
// base_shape / generate_remaps do (tc.rs:175-215): operand 0 = A (rows m), 1 = B (columns n).
// Returns the (m or n) index and the k index of element `elem` held by `lane`.
void tc_operand_element(const TensorCore& tc, int operand, int lane, int elem, int* mn, int* k);
// Accumulator element -> (m, n).
void tc_acc_element(const TensorCore& tc, int lane, int elem, int* m, int* n);

// ---- gpudims.rs:387-463
size_t find_smallest_divisor(size_t n);
bool group_dims(const std::vector<size_t>& dims, const std::vector<size_t>& max_sizes, std::vector<size_t>* out);
std::vector<size_t> split_dims(const std::vector<size_t>& dims, const std::vector<size_t>& max_sizes);
std::vector<size_t> limit_dims(const std::vector<size_t>& dims, const std::vector<size_t>& max_sizes);
// gpudims.rs:529-584
bool get_contraction(const std::vector<size_t>& original, const std::vector<size_t>& limited,
                     std::vector<std::vector<size_t>>* out);
// gpudims.rs:331-382,479-505,587-642: the launch extents for `dims` under `max_sizes` and,
// for a given tuple of raw hardware indices, the index of every original dimension.
class KernelBuilder;
// How global dims are turned around (local dims never are):
//   kReverseDims   - the dims are reversed before limiting and the indices after it, so the
//                    innermost axis lands on gidx0 whatever regrouping happened.  This is what
//                    this backend launches and what tinygrad's get_grouped_dims does.
//   kReverseResult - the reference's literal code (schedule/src/gpudims.rs:331-382): dims are
//                    limited as given and only the resulting index list is reversed.  Equal to
//                    kReverseDims when the dims read the same in both directions; otherwise it
//                    hands dimension i an index whose extent is that of dimension n-1-i.  Offered
//                    for comparison with the reference, never launched.
enum class DimOrder { kForward = 0, kReverseDims = 1, kReverseResult = 2 };
struct GroupedDims {
    std::vector<size_t> original;  // in the caller's order
    std::vector<size_t> launch;    // extents of gidx0.. / lidx0..
    DimOrder order = DimOrder::kForward;
    // raw[i] in [0, launch[i])  ->  index per original dimension
    std::vector<size_t> map(const std::vector<size_t>& raw) const;
    // The same mapping as nodes of a kernel under construction: raw[i] is the SPECIAL of launch
    // extent i; the result holds one index node per original dimension (mod / idiv chains where
    // dims were regrouped, the SPECIALs themselves where they were not).
    std::vector<uint32_t> map_nodes(KernelBuilder& b, const std::vector<uint32_t>& raw) const;
};
GroupedDims get_grouped_dims(const std::vector<size_t>& dims, const std::vector<size_t>* max_sizes, DimOrder order);
inline GroupedDims get_grouped_dims(const std::vector<size_t>& dims, const std::vector<size_t>* max_sizes, bool reverse) {
    return get_grouped_dims(dims, max_sizes, reverse ? DimOrder::kReverseDims : DimOrder::kForward);
}

// ---- small builder for linearized kernels (C++ twin of morok_amd/uop.py)
class KernelBuilder {
  public:
    uint32_t add(Op op, DType dt, std::vector<uint32_t> src = {}, int64_t arg_i = 0, double arg_f = 0.0,
                 uint16_t sub = 0, std::string str = "", std::vector<int64_t> extra = {});
    static DType scalar(Scalar s, int vcount = 1) {
        DType d;
        d.scalar = s;
        d.vcount = static_cast<uint16_t>(vcount);
        return d;
    }
    static DType pointer(Scalar s, int64_t size, AddrSpace sp = AddrSpace::Global, int vcount = 1) {
        DType d = scalar(s, vcount);
        d.is_ptr = true;
        d.space = sp;
        d.ptr_size = size;
        return d;
    }
    uint32_t param(int slot, Scalar s, int64_t size) { return add(Op::Param, pointer(s, size), {}, slot); }
    uint32_t ci(int64_t v, Scalar s = Scalar::Int32) { return add(Op::Const, scalar(s), {}, v); }
    uint32_t cf(double v, Scalar s = Scalar::Float32) { return add(Op::Const, scalar(s), {}, 0, v); }
    uint32_t special(const std::string& name, int64_t extent) {
        return add(Op::Special, scalar(Scalar::Int32), {ci(extent)}, 0, 0.0, 0, name);
    }
    uint32_t range(int64_t end, int axis_id, AxisType t = AxisType::Reduce) {
        return add(Op::Range, scalar(Scalar::Int32), {ci(end)}, axis_id, 0.0, static_cast<uint16_t>(t));
    }
    uint32_t end(std::vector<uint32_t> ranges) { return add(Op::End, scalar(Scalar::Void), std::move(ranges)); }
    uint32_t index(uint32_t buf, uint32_t idx) { return add(Op::Index, dtype(buf), {buf, idx}); }
    uint32_t index_gated(uint32_t buf, uint32_t idx, uint32_t gate) { return add(Op::Index, dtype(buf), {buf, idx, gate}, 0, 0, 1); }
    // vcount 0 keeps the element type of the pointer (scalar or vector)
    uint32_t load(uint32_t idx, int vcount = 0) {
        DType d = dtype(idx);
        d.is_ptr = false;
        if (vcount > 0) d.vcount = static_cast<uint16_t>(vcount);
        return add(Op::Load, d, {idx});
    }
    uint32_t load_alt(uint32_t idx, uint32_t alt) {
        DType d = dtype(idx);
        d.is_ptr = false;
        return add(Op::Load, d, {idx, alt});
    }
    uint32_t store(uint32_t idx, uint32_t v) { return add(Op::Store, scalar(Scalar::Void), {idx, v}); }
    uint32_t unary(UnaryOp op, uint32_t x) { return add(Op::Unary, dtype(x), {x}, 0, 0, static_cast<uint16_t>(op)); }
    uint32_t binary(BinaryOp op, uint32_t a, uint32_t b);
    uint32_t where(uint32_t c, uint32_t t, uint32_t f) { return add(Op::Where, dtype(t), {c, t, f}); }
    uint32_t mulacc(uint32_t a, uint32_t b, uint32_t c) { return add(Op::MulAcc, dtype(c), {a, b, c}); }
    uint32_t cast(uint32_t x, Scalar s) { return add(Op::Cast, scalar(s, dtype(x).vcount), {x}); }
    uint32_t gep(uint32_t v, int i) { return add(Op::Gep, scalar(dtype(v).scalar), {v}, 0, 0, 0, "", {i}); }
    uint32_t vectorize(std::vector<uint32_t> e) {
        DType d = scalar(dtype(e[0]).scalar, static_cast<int>(e.size()));
        return add(Op::Vectorize, d, std::move(e));
    }
    uint32_t reduce(ReduceOp op, uint32_t v, std::vector<uint32_t> ranges) {
        std::vector<uint32_t> s{v};
        s.insert(s.end(), ranges.begin(), ranges.end());
        return add(Op::Reduce, dtype(v), std::move(s), 0, 0, static_cast<uint16_t>(op));
    }
    uint32_t wave_reduce(ReduceOp op, uint32_t v) { return add(Op::WaveReduce, dtype(v), {v}, 0, 0, static_cast<uint16_t>(op)); }
    uint32_t define_local(int id, Scalar s, int64_t size) { return add(Op::DefineLocal, pointer(s, size, AddrSpace::Local), {}, id); }
    uint32_t barrier() { return add(Op::Barrier, scalar(Scalar::Void)); }
    // gfx950 local-memory extensions (uop.h): transposing 4-element load, direct global -> local
    // copy of 16 bytes per lane, wait until at most n such copies of this wave are in flight
    uint32_t load_tr(uint32_t local_index) { return add(Op::LoadTr, scalar(dtype(local_index).scalar, 4), {local_index}); }
    uint32_t async_copy(uint32_t global_index, uint32_t local_index) {
        return add(Op::AsyncCopy, scalar(Scalar::Void), {global_index, local_index});
    }
    uint32_t wait_async(int n) { return add(Op::WaitAsync, scalar(Scalar::Void), {}, n); }
    uint32_t define_reg(int id, Scalar s, int64_t size, int vcount = 1) {
        return add(Op::DefineReg, pointer(s, size, AddrSpace::Reg, vcount), {}, id);
    }
    uint32_t if_(uint32_t c) { return add(Op::If, scalar(Scalar::Void), {c}); }
    uint32_t endif() { return add(Op::EndIf, scalar(Scalar::Void)); }
    // arithmetic helpers on int32 indices with constant folding of the trivial cases
    uint32_t iadd(uint32_t a, uint32_t b);
    uint32_t imul(uint32_t a, int64_t c);
    uint32_t idiv(uint32_t a, int64_t c);
    uint32_t imod(uint32_t a, int64_t c);

    const DType& dtype(uint32_t id) const { return k_.nodes[id - 1].dtype; }
    const UOp& node(uint32_t id) const { return k_.nodes[id - 1]; }
    // Finishes the kernel: computes the content hash over a canonical serialization.
    LinearKernel finish();
    std::vector<uint8_t> serialize() const;

    // Turns on common-subexpression elimination of pure value nodes (scope-aware).
    void enable_cse() { cse_ = true; }

  private:
    LinearKernel k_;
    bool cse_ = false;
    std::unordered_map<std::string, uint32_t> cse_map_;
    std::vector<std::vector<std::string>> cse_scopes_;
};

// Linearized kernels for the matmul shapes on the hot path.
// f32 matmul, one kernel (tensor/src/test/unit/fusion.rs:28-33): LOCAL 16x16, UPCAST 4x4,
// K as a REDUCE loop of MULACCs into register accumulators (the shape the heuristics of
// schedule/src/optimizer/heuristics.rs:37-82 aim for: upcast 4, local <= 128..256).
// Requires M % 64 == 0 and N % 64 == 0.
LinearKernel build_matmul_f32_kernel(int64_t M, int64_t N, int64_t K);
// The same kernel shape with the optimisation choices left open: the action space a beam
// search explores (LOCAL extents, UPCAST of N as a vector and of M as rows per work-item,
// UNROLL of the reduce axis; schedule/src/optimizer/beam.rs:36-120).
struct MatmulF32Opts {
    int local_x = 16, local_y = 16;  // LOCAL
    int up_n = 4, up_m = 4;          // UPCAST
    int unroll_k = 1;                // UNROLL
    // GROUP through local memory (schedule/src/optimizer/heuristics.rs:37-82, transforms.rs:1085-1089):
    // 0 = operands straight from global memory; 8 / 16 / 32 = the workgroup stages A and B tiles
    // of that depth in LDS (A transposed, so a work-item's rows are one vector), the next tiles'
    // global loads issued before this tile's multiply-adds, two barriers per tile.
    int lds_k = 0;
};
bool matmul_f32_opts_valid(const MatmulF32Opts& o, int64_t M, int64_t N, int64_t K);
LinearKernel build_matmul_f32_kernel(int64_t M, int64_t N, int64_t K, const MatmulF32Opts& o);
// Tensor-core matmul (tc.rs:358-674 applied to C[M,N] = A[M,K] B[K,N]): one wave per
// um x un grid of 16x16 output tiles, operands gathered per lane as the tensor core's
// swizzle prescribes, WMMA per K step, accumulate in dtype_out, result cast to `out`.
// Post-TC upcasts of M and N by the first of [5,4,3,2] that divides (heuristics.rs:787-821).
int build_wmma_matmul_kernel(const TensorCore& tc, int64_t M, int64_t N, int64_t K, Scalar out, LinearKernel* k);
// The same product with the operands staged through local memory (GROUP / LOCAL of the
// optimizer, schedule/src/optimizer/heuristics.rs:37-82, transforms.rs:1085-1089): a workgroup
// of waves_m x waves_n waves owns a (waves_m * up_m * 16) x (waves_n * up_n * 16) output tile;
// per K step the work-items copy the A and B tiles global -> registers -> LDS with 16-byte
// loads (the next step's loads are issued before this step's WMMAs); A fragments are read back
// as one vector per lane, B fragments as pairs of consecutive k (rows k and k+1 are kept
// interleaved in LDS); two barriers per step.  The defaults are 2 x 2 waves of 4 x 4 tiles
// (128 x 128) and as many tensor-core K steps per barrier pair as divide K, up to 64 elements.
// Extents the workgroup tile does not divide are padded (PADTO, tc.rs:400-432): the grid is
// rounded up, loads past the operands are gated to zero, stores past the result are skipped.
// Requires N and K to be multiples of 8 (16-byte copies) and a tensor core whose lanes hold
// consecutive k.
struct WmmaLdsOpts {
    int waves_m = 2, waves_n = 2;  // LOCAL
    int up_m = 4, up_n = 4;        // UPCAST: tensor-core tiles per wave
    int unroll_k = 0;              // UNROLL: tensor-core K steps per barrier pair; 0 = choose by K
    // 0: tiles travel global -> registers -> local memory (above).  2: two stages of each tile in
    // local memory filled by direct global -> local copies (ASYNC_COPY / WAIT_ASYNC), B fragments
    // read with the transposing load (LOAD_TR), one barrier per 64-deep K step, workgroups
    // mapped to tiles in compact blocks per XCD, result rows written as 8-byte vectors.  Needs a
    // 16x16x32 tensor core, M, N, K divisible by the tile and a K step of 64.  3: the same with a
    // third stage of the second operand's tile (workgroups of at most four waves, more than two K
    // steps): the copies of tile r + 2 are spread over the whole of step r, B chunks behind the
    // first half's tensor-core instructions, A chunks behind the second half's.
    int stages = 0;
};
// Extents of the workgroup tile these choices give (false if the choices are not buildable at all)
bool wmma_lds_tile(const TensorCore& tc, const WmmaLdsOpts& o, int64_t K, int* bm, int* bn, int* bk);
bool wmma_lds_opts_valid(const TensorCore& tc, const WmmaLdsOpts& o, int64_t M, int64_t N, int64_t K);
int build_wmma_matmul_lds_kernel(const TensorCore& tc, int64_t M, int64_t N, int64_t K, Scalar out, const WmmaLdsOpts& o,
                                 LinearKernel* k);
int build_wmma_matmul_lds_kernel(const TensorCore& tc, int64_t M, int64_t N, int64_t K, Scalar out, LinearKernel* k);

}  // namespace mrk
