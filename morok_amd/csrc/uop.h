// The linearized UOp kernel as it reaches Renderer::render: the Vec<Arc<UOp>> that
// linearize_with_cfg + line_rewrite_cleanups produce (schedule/src/linearize/mod.rs:172-177,
// 308-310; consumed by codegen/src/c/mod.rs:50-53).  Every node carries
// { id, op, dtype, sources (by id), argument } (ir/src/uop/core.rs:102-142).
//
// Wire format (little endian), what a host-side shim serialises the stream into:
//   u32 magic 'MRKL', u32 version, u32 node_count, then per node
//   u32 id | u16 op | u8 scalar | u8 flags (bit0 pointer, bits1-2 address space)
//   u16 vcount | i64 ptr_size (-1 none) | u16 nsrc | u32 src[nsrc]
//   i64 arg_i | f64 arg_f | u16 sub | u16 strlen | bytes | u16 nextra | i64 extra[nextra]
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace mrk {

// Vocabulary of ir/src/op.rs:33-305 that survives to the renderer (the set handled by
// codegen/src/c/ops.rs:127-458) plus the GPU-only ops the C backend ignores
// (Special, Barrier, DefineLocal as shared memory).
enum class Op : uint16_t {
    Param = 0,        // arg_i = slot                                  (op.rs:81-85)
    DefineVar = 1,    // str = name, extra = {min, max}                 (codegen/src/c/mod.rs:97-103)
    DefineLocal = 2,  // arg_i = id, dtype Ptr{base, Local, size}       (op.rs:41)
    DefineReg = 3,    // arg_i = id, dtype Ptr{base, Reg, size}         (op.rs:223-228)
    Const = 4,        // arg_i / arg_f by dtype                         (codegen/src/c/types.rs:66-142)
    Special = 5,      // str = "gidxN" | "lidxN", src0 = extent         (op.rs:71-74)
    Range = 6,        // src0 = end, arg_i = axis_id, sub = AxisType    (op.rs:175-180)
    End = 7,          // srcs = ranges closed (innermost first)
    Index = 8,        // src0 = buffer, src1.. = indices; sub = 1: last src is the gate (op.rs:101-105)
    Load = 9,         // src0 = index, optional src1 = alt              (op.rs:295-299)
    Store = 10,       // src0 = index, src1 = value                     (op.rs:300-304)
    Unary = 11,       // sub = UnaryOp
    Binary = 12,      // sub = BinaryOp
    Where = 13,       // cond, t, f
    MulAcc = 14,      // a, b, c
    Cast = 15,
    BitCast = 16,
    Gep = 17,         // src0 = vector, extra = element indices
    Vectorize = 18,   // srcs = elements
    Wmma = 19,        // a, b, c; str = metadata.name (WMMA_N_M_K_in_out), op.rs:231-236
    If = 20,          // src0 = condition
    EndIf = 21,
    Barrier = 22,     // op.rs:185-188
    After = 23,       // src0 = passthrough
    Noop = 24,
    Sink = 25,
    Reduce = 26,      // src0 = value, src1.. = ranges, sub = ReduceOp  (op.rs:156-160)
    // Extension for wave64 hardware (not in the reference vocabulary): all-lanes reduction
    // of src0 over the 64 lanes of a wavefront, sub = ReduceOp.  A host scheduler emits it
    // for a GROUP_REDUCE axis of extent 64 instead of the local-memory tree.
    WaveReduce = 27,
    // Extensions for the gfx950 local-memory path of tensor-core kernels (not in the reference
    // vocabulary; what the hand-written GEMM uses, made available to generated kernels).
    // LoadTr: transposing load of 16-bit elements from local memory, src0 = Index into a
    // DEFINE_LOCAL, dtype = vector of 4.  Within each group of 16 lanes, lane i addresses 4
    // consecutive elements (row i / 4, columns 4 * (i % 4) .. + 3 of a 4 x 16 block); lane i
    // receives column i of the block, rows 0..3.
    LoadTr = 28,
    // AsyncCopy: direct global -> local copy of 16 bytes per lane that bypasses registers,
    // src0 = Index into a PARAM (per lane, 16-byte aligned), src1 = Index into a DEFINE_LOCAL
    // that must be the same for all 64 lanes of a wavefront (its first lane is used): lane i's
    // bytes land at that address + 16 * i.  Completion is not tracked by later loads: a WaitAsync
    // followed by a Barrier makes the data visible to the workgroup.
    AsyncCopy = 29,
    // WaitAsync: blocks the wavefront until at most arg_i of its AsyncCopies are in flight
    // (they complete in issue order).
    WaitAsync = 30,
};

// dtype/src/lib.rs:129-154
enum class Scalar : uint8_t {
    Bool = 0, Int8, UInt8, Int16, UInt16, Int32, UInt32, Int64, UInt64, Float16, BFloat16, Float32, Float64, Void,
    Index,
    // dtype/src/lib.rs:142-143: OCP 8-bit floats (E4M3 has no infinity, maximum 448; E5M2 is the top
    // byte of a half, maximum 57344).  One byte of storage, `unsigned char` in C
    // (codegen/src/c/types.rs:26); they appear as tensor-core operands only.
    Fp8E4M3,
    Fp8E5M2,
};

enum class AddrSpace : uint8_t { Global = 0, Local = 1, Reg = 2 };  // dtype/src/lib.rs:103-110

// ir/src/types.rs:377-405
enum class AxisType : uint16_t { Global = 0, Warp, Local, Loop, GroupReduce, Reduce, Upcast, Unroll, Thread, Outer };

// ir/src/types.rs:567-724 (subset that reaches a renderer after the late rewrites)
enum class UnaryOp : uint16_t {
    Neg = 0, Abs, Sqrt, Rsqrt, Reciprocal, Exp, Exp2, Log, Log2, Sin, Cos, Tan, Floor, Ceil, Trunc, Round, Erf, Sign,
    Square, Not,
};
enum class BinaryOp : uint16_t {
    Add = 0, Sub, Mul, Fdiv, Mod, Max, Pow, And, Or, Xor, Shl, Shr, Idiv, Lt, Le, Gt, Ge, Eq, Ne, Threefry,
};
enum class ReduceOp : uint16_t { Add = 0, Mul, Max, Min };

struct DType {
    Scalar scalar = Scalar::Void;
    uint16_t vcount = 1;
    bool is_ptr = false;
    AddrSpace space = AddrSpace::Global;
    int64_t ptr_size = -1;

    bool is_float() const {
        return scalar == Scalar::Float16 || scalar == Scalar::BFloat16 || scalar == Scalar::Float32 ||
               scalar == Scalar::Float64;
    }
    bool is_fp8() const { return scalar == Scalar::Fp8E4M3 || scalar == Scalar::Fp8E5M2; }
    bool is_bool() const { return scalar == Scalar::Bool; }
    bool is_signed() const {
        return scalar == Scalar::Int8 || scalar == Scalar::Int16 || scalar == Scalar::Int32 ||
               scalar == Scalar::Int64 || scalar == Scalar::Index || is_float();
    }
};

struct UOp {
    uint32_t id = 0;
    Op op = Op::Noop;
    DType dtype;
    std::vector<uint32_t> src;
    int64_t arg_i = 0;
    double arg_f = 0.0;
    uint16_t sub = 0;
    std::string str;
    std::vector<int64_t> extra;
};

struct LinearKernel {
    std::vector<UOp> nodes;
    // Content hash of the serialized stream (stands for the hash-consed AST identity the
    // kernel cache keys on, runtime/src/kernel_cache.rs:87-118).
    uint64_t content_hash = 0;
};

// Parses the wire format; returns kRenderError with a message on malformed input.
int parse_linear_kernel(const uint8_t* data, size_t len, LinearKernel* out);
uint64_t fnv1a64(const uint8_t* data, size_t len);

}  // namespace mrk
