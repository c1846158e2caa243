// HIP-C renderer for gfx950: linearized UOp kernel -> `extern "C" __global__` source +
// ProgramSpec.  The counterpart of CRenderer::render (codegen/src/c/mod.rs:47-270) and
// render_uop (codegen/src/c/ops.rs:127-458) for a GPU target: same SSA-with-inlining
// scheme, same op semantics (ops.rs:489-606, types.rs:10-28,66-142,206-261), plus the
// ops the C backend does not lower:
//   Special  -> blockIdx / threadIdx (extent -> launch dims)       (schedule/src/gpudims.rs:331-382)
//   DefineLocal -> __shared__ array                                (schedule/src/rangeify/transforms.rs:1085-1089)
//   Barrier  -> __syncthreads()                                    (transforms.rs:1159-1161)
//   Wmma     -> gfx950 MFMA builtin named from WmmaMetadata.name   (schedule/src/optimizer/tc.rs:621-638)
//   WaveReduce (extension) -> wave64 DPP / ds_swizzle reduction
#include <algorithm>
#include <array>
#include <cctype>
#include <cinttypes>
#include <cmath>
#include <cstdarg>
#include <cstring>
#include <functional>
#include <map>
#include <set>
#include <sstream>
#include <unordered_map>
#include <unordered_set>

#include "device.h"
#include "error.h"
#include "uop.h"

namespace mrk {

uint64_t fnv1a64(const uint8_t* data, size_t len) {
    uint64_t h = 1469598103934665603ull;
    for (size_t i = 0; i < len; i++) {
        h ^= data[i];
        h *= 1099511628211ull;
    }
    return h;
}

namespace {

struct Reader {
    const uint8_t* p;
    size_t left;
    bool ok = true;
    template <class T>
    T get() {
        T v{};
        if (left < sizeof(T)) {
            ok = false;
            return v;
        }
        std::memcpy(&v, p, sizeof(T));
        p += sizeof(T);
        left -= sizeof(T);
        return v;
    }
};

std::string fmt(const char* f, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, f);
    vsnprintf(buf, sizeof(buf), f, ap);
    va_end(ap);
    return buf;
}

}  // namespace

int parse_linear_kernel(const uint8_t* data, size_t len, LinearKernel* out) {
    Reader r{data, len};
    if (r.get<uint32_t>() != 0x4C4B524Du) return fail(kRenderError, "linearized kernel: bad magic");
    if (r.get<uint32_t>() != 1u) return fail(kRenderError, "linearized kernel: unsupported version");
    uint32_t n = r.get<uint32_t>();
    if (!r.ok || n > (1u << 22)) return fail(kRenderError, "linearized kernel: bad node count");
    out->nodes.clear();
    out->nodes.reserve(n);
    for (uint32_t i = 0; i < n; i++) {
        UOp u;
        u.id = r.get<uint32_t>();
        uint16_t op = r.get<uint16_t>();
        uint8_t scalar = r.get<uint8_t>();
        uint8_t flags = r.get<uint8_t>();
        u.dtype.vcount = r.get<uint16_t>();
        u.dtype.ptr_size = r.get<int64_t>();
        uint16_t nsrc = r.get<uint16_t>();
        if (!r.ok) break;
        if (op > static_cast<uint16_t>(Op::WaitAsync))
            return failf(kRenderError, "linearized kernel: unknown op tag %u at node %u", op, i);
        if (scalar > static_cast<uint8_t>(Scalar::Fp8E5M2))
            return failf(kRenderError, "linearized kernel: unknown scalar dtype %u at node %u", scalar, i);
        u.op = static_cast<Op>(op);
        u.dtype.scalar = static_cast<Scalar>(scalar);
        u.dtype.is_ptr = flags & 1;
        u.dtype.space = static_cast<AddrSpace>((flags >> 1) & 3);
        if (u.dtype.vcount == 0) u.dtype.vcount = 1;
        for (uint16_t s = 0; s < nsrc; s++) u.src.push_back(r.get<uint32_t>());
        u.arg_i = r.get<int64_t>();
        u.arg_f = r.get<double>();
        u.sub = r.get<uint16_t>();
        uint16_t sl = r.get<uint16_t>();
        if (!r.ok || r.left < sl) {
            r.ok = false;
            break;
        }
        u.str.assign(reinterpret_cast<const char*>(r.p), sl);
        r.p += sl;
        r.left -= sl;
        uint16_t ne = r.get<uint16_t>();
        for (uint16_t e = 0; e < ne; e++) u.extra.push_back(r.get<int64_t>());
        if (!r.ok) break;
        out->nodes.push_back(std::move(u));
    }
    if (!r.ok || out->nodes.size() != n) return fail(kRenderError, "linearized kernel: truncated stream");
    out->content_hash = fnv1a64(data, len);
    return kOk;
}

namespace {

// ---------------------------------------------------------------- types and constants
const char* c_scalar(Scalar s) {  // codegen/src/c/types.rs:10-28
    switch (s) {
        case Scalar::Bool: return "bool";
        case Scalar::Int8: return "signed char";
        case Scalar::UInt8: return "unsigned char";
        case Scalar::Int16: return "short";
        case Scalar::UInt16: return "unsigned short";
        case Scalar::Int32: return "int";
        case Scalar::UInt32: return "unsigned int";
        case Scalar::Int64:
        case Scalar::Index: return "long long";
        case Scalar::Fp8E4M3:
        case Scalar::Fp8E5M2: return "unsigned char";  // types.rs:26
        case Scalar::UInt64: return "unsigned long long";
        case Scalar::Float16: return "_Float16";
        case Scalar::BFloat16: return "__bf16";
        case Scalar::Float32: return "float";
        case Scalar::Float64: return "double";
        case Scalar::Void: return "void";
    }
    return "void";
}
const char* c_vector_base(Scalar s) {  // types.rs:31-49, prefixed to stay clear of HIP's own float4 etc.
    switch (s) {
        case Scalar::Bool: return "mrk_bool";
        case Scalar::Int8: return "mrk_schar";
        case Scalar::UInt8: return "mrk_uchar";
        case Scalar::Int16: return "mrk_short";
        case Scalar::UInt16: return "mrk_ushort";
        case Scalar::Int32: return "mrk_int";
        case Scalar::UInt32: return "mrk_uint";
        case Scalar::Int64:
        case Scalar::Index: return "mrk_llong";
        case Scalar::Fp8E4M3: return "mrk_f8e4m3_";
        case Scalar::Fp8E5M2: return "mrk_f8e5m2_";
        case Scalar::UInt64: return "mrk_ullong";
        case Scalar::Float16: return "mrk_half";
        case Scalar::BFloat16: return "mrk_bhalf";
        case Scalar::Float32: return "mrk_float";
        case Scalar::Float64: return "mrk_double";
        case Scalar::Void: return "mrk_void";
    }
    return "mrk_void";
}
size_t scalar_bytes(Scalar s) {
    switch (s) {
        case Scalar::Bool:
        case Scalar::Int8:
        case Scalar::Fp8E4M3:
        case Scalar::Fp8E5M2:
        case Scalar::UInt8: return 1;
        case Scalar::Int16:
        case Scalar::UInt16:
        case Scalar::Float16:
        case Scalar::BFloat16: return 2;
        case Scalar::Int32:
        case Scalar::UInt32:
        case Scalar::Float32: return 4;
        default: return 8;
    }
}
std::string c_value_type(const DType& d) {  // type of a value (ignoring pointer-ness)
    if (d.vcount > 1) return std::string(c_vector_base(d.scalar)) + std::to_string(d.vcount);
    return c_scalar(d.scalar);
}
std::string c_dtype(const DType& d) {  // types.rs:54-63
    if (d.is_ptr) {
        const char* q = d.space == AddrSpace::Local ? "__shared__ " : "";
        (void)q;
        return c_value_type(d) + "*";
    }
    return c_value_type(d);
}
std::string c_float_literal(double f, Scalar s) {  // types.rs:90-142
    if (std::isnan(f)) return s == Scalar::Float64 ? "__builtin_nan(\"\")" : "__builtin_nanf(\"\")";
    if (std::isinf(f)) {
        std::string sign = f < 0 ? "-" : "";
        return sign + (s == Scalar::Float64 ? "__builtin_inf()" : "__builtin_inff()");
    }
    if (s == Scalar::Float64) return fmt("%.17g%s", f, (std::floor(f) == f && std::fabs(f) < 1e15) ? ".0" : "");
    float v = static_cast<float>(f);
    std::string lit = fmt("%.9g", v);
    if (lit.find('.') == std::string::npos && lit.find('e') == std::string::npos && lit.find("inf") == std::string::npos)
        lit += ".0";
    lit += "f";
    if (s == Scalar::Float16) return "((_Float16)" + lit + ")";
    if (s == Scalar::BFloat16) return "((__bf16)" + lit + ")";
    return lit;
}
std::string c_const(const UOp& u) {  // types.rs:66-88
    const Scalar s = u.dtype.scalar;
    std::string one;
    if (u.dtype.is_float()) one = c_float_literal(u.arg_f, s);
    else if (s == Scalar::Bool) one = u.arg_i ? "true" : "false";
    else if (s == Scalar::Int64 || s == Scalar::Index) one = fmt("%" PRId64 "LL", u.arg_i);
    else if (s == Scalar::UInt64) one = fmt("%" PRIu64 "ULL", static_cast<uint64_t>(u.arg_i));
    else if (s == Scalar::UInt32) one = fmt("%" PRIu64 "u", static_cast<uint64_t>(u.arg_i) & 0xffffffffull);
    else one = fmt("%" PRId64, u.arg_i);
    if (u.dtype.vcount > 1) {
        std::string v = "(" + c_value_type(u.dtype) + "){";
        for (int i = 0; i < u.dtype.vcount; i++) v += (i ? ", " : "") + one;
        return v + "}";
    }
    return one;
}
std::string reduce_identity(ReduceOp op, const DType& d) {  // types.rs:206-261
    const bool f64 = d.scalar == Scalar::Float64;
    switch (op) {
        case ReduceOp::Add: return d.is_float() ? (f64 ? "0.0" : "0.0f") : "0";
        case ReduceOp::Mul: return d.is_float() ? (f64 ? "1.0" : "1.0f") : "1";
        case ReduceOp::Max:
            if (d.is_float()) return f64 ? "-__builtin_inf()" : "-__builtin_inff()";
            switch (d.scalar) {
                case Scalar::Int64:
                case Scalar::Index: return "(-9223372036854775807LL - 1)";
                case Scalar::Int32: return "(-2147483647 - 1)";
                case Scalar::Int16: return "-32768";
                case Scalar::Int8: return "-128";
                default: return "0";
            }
        case ReduceOp::Min:
            if (d.is_float()) return f64 ? "__builtin_inf()" : "__builtin_inff()";
            switch (d.scalar) {
                case Scalar::Int64:
                case Scalar::Index: return "9223372036854775807LL";
                case Scalar::Int32: return "2147483647";
                case Scalar::Int16: return "32767";
                case Scalar::Int8: return "127";
                case Scalar::UInt64: return "18446744073709551615ULL";
                case Scalar::UInt32: return "4294967295u";
                case Scalar::UInt16: return "65535";
                case Scalar::UInt8: return "255";
                default: return "0";
            }
    }
    return "0";
}

// float math on half / bfloat goes through float (types.rs:195-203)
std::string math_call(const char* fn, const DType& d, const std::string& args) {
    if (d.scalar == Scalar::Float64) return std::string(fn) + "(" + args + ")";
    if (d.scalar == Scalar::Float32) return std::string(fn) + "f(" + args + ")";
    return "((" + std::string(c_scalar(d.scalar)) + ")" + fn + "f(" + args + "))";
}
std::string as_float_arg(const std::string& v, const DType& d) {
    if (d.scalar == Scalar::Float16 || d.scalar == Scalar::BFloat16) return "(float)" + v;
    return v;
}

std::string render_unary(UnaryOp op, const std::string& s, const DType& d) {  // ops.rs:533-584
    const std::string one = d.scalar == Scalar::Float64 ? "1.0" : "1.0f";
    const std::string a = as_float_arg(s, d);
    auto narrow = [&](const std::string& e) {
        if (d.scalar == Scalar::Float16 || d.scalar == Scalar::BFloat16)
            return "((" + std::string(c_scalar(d.scalar)) + ")" + e + ")";
        return e;
    };
    switch (op) {
        case UnaryOp::Neg: return "(-" + s + ")";
        case UnaryOp::Not: return d.is_bool() ? "(!" + s + ")" : "(~" + s + ")";
        case UnaryOp::Abs: return d.is_float() ? math_call("fabs", d, a) : "(" + s + " < 0 ? -" + s + " : " + s + ")";
        case UnaryOp::Sqrt: return math_call("sqrt", d, a);
        case UnaryOp::Rsqrt: return narrow("(" + one + " / " + math_call("sqrt", DType{d.scalar == Scalar::Float64 ? Scalar::Float64 : Scalar::Float32}, a) + ")");
        case UnaryOp::Reciprocal: return narrow("(" + one + " / " + a + ")");
        case UnaryOp::Exp: return math_call("exp", d, a);
        case UnaryOp::Exp2: return math_call("exp2", d, a);
        case UnaryOp::Log: return math_call("log", d, a);
        case UnaryOp::Log2: return math_call("log2", d, a);
        case UnaryOp::Sin: return math_call("sin", d, a);
        case UnaryOp::Cos: return math_call("cos", d, a);
        case UnaryOp::Tan: return math_call("tan", d, a);
        case UnaryOp::Floor: return math_call("floor", d, a);
        case UnaryOp::Ceil: return math_call("ceil", d, a);
        case UnaryOp::Trunc: return math_call("trunc", d, a);
        case UnaryOp::Round: return math_call("rint", d, a);
        case UnaryOp::Erf: return math_call("erf", d, a);
        case UnaryOp::Sign: {
            const std::string z = d.is_float() ? (d.scalar == Scalar::Float64 ? "0.0" : "0.0f") : "0";
            return "((" + std::string(c_scalar(d.scalar)) + ")((" + a + " > " + z + ") - (" + a + " < " + z + ")))";
        }
        case UnaryOp::Square: return "(" + s + " * " + s + ")";
    }
    return "/*?*/" + s;
}

std::string render_binary(BinaryOp op, const std::string& l, const std::string& r, const DType& d) {  // ops.rs:489-531
    auto infix = [&](const char* o) { return "(" + l + " " + o + " " + r + ")"; };
    switch (op) {
        case BinaryOp::Add: return infix("+");
        case BinaryOp::Sub: return infix("-");
        case BinaryOp::Mul: return infix("*");
        case BinaryOp::Fdiv: return infix("/");
        case BinaryOp::Idiv: return infix("/");
        case BinaryOp::Mod:
            return d.is_float() ? math_call("fmod", d, as_float_arg(l, d) + ", " + as_float_arg(r, d)) : infix("%");
        case BinaryOp::Max:
            return d.is_float() ? math_call("fmax", d, as_float_arg(l, d) + ", " + as_float_arg(r, d))
                                : "(" + l + " > " + r + " ? " + l + " : " + r + ")";
        case BinaryOp::Pow:
            return d.is_float() ? math_call("pow", d, as_float_arg(l, d) + ", " + as_float_arg(r, d))
                                : "((" + std::string(c_scalar(d.scalar)) + ")pow((double)" + l + ", (double)" + r + "))";
        case BinaryOp::Lt: return infix("<");
        case BinaryOp::Le: return infix("<=");
        case BinaryOp::Gt: return infix(">");
        case BinaryOp::Ge: return infix(">=");
        case BinaryOp::Eq: return infix("==");
        case BinaryOp::Ne: return infix("!=");
        case BinaryOp::And: return infix("&");
        case BinaryOp::Or: return infix("|");
        case BinaryOp::Xor:
        case BinaryOp::Threefry: return infix("^");
        case BinaryOp::Shl: return infix("<<");
        case BinaryOp::Shr: return infix(">>");
    }
    return "/*?*/" + l;
}

std::string reduce_accumulate(ReduceOp op, const std::string& acc, const std::string& v, const DType& d) {  // ops.rs:587-606
    switch (op) {
        case ReduceOp::Add: return acc + " += " + v + ";";
        case ReduceOp::Mul: return acc + " *= " + v + ";";
        case ReduceOp::Max:
            return d.is_float() ? acc + " = " + math_call("fmax", d, as_float_arg(acc, d) + ", " + as_float_arg(v, d)) + ";"
                                : acc + " = (" + acc + " > " + v + " ? " + acc + " : " + v + ");";
        case ReduceOp::Min:
            return d.is_float() ? acc + " = " + math_call("fmin", d, as_float_arg(acc, d) + ", " + as_float_arg(v, d)) + ";"
                                : acc + " = (" + acc + " < " + v + " ? " + acc + " : " + v + ");";
    }
    return "";
}

// ---------------------------------------------------------------- WMMA -> MFMA
// metadata.name = WMMA_{N}_{M}_{K}_{in}_{out} (schedule/src/optimizer/tc.rs:621-638, dtype
// names 677-688).  Operand sizes per lane follow the CDNA tables
// (schedule/src/optimizer/renderer.rs:538-558): 16x16x32 -> A,B 8 elements, C 4;
// 16x16x16 -> A,B 4 elements, C 4.
// The reference names both 8-bit float cores WMMA_16_16_32_unknown_float (its dtype-name table
// has no entry for them); the operand dtype tells them apart: E4M3 -> ..._fp8_fp8, E5M2 ->
// ..._bf8_bf8, eight bytes per lane handed over as one 64-bit integer.
std::string wmma_callee(const std::string& name, Scalar operand) {
    if (operand == Scalar::Fp8E4M3) return name + "_e4m3";
    if (operand == Scalar::Fp8E5M2) return name + "_e5m2";
    return name;
}
// tied: the instruction written out with the accumulator in the accumulation registers and
// result and accumulator in the same registers (16x16x32 bf16 / f16 only).  Through the builtin
// the device compiler leaves this shape untied when the accumulators need those registers
// (kernels with more than 128 declared registers per work-item, one wave per SIMD) and moves
// whole tiles between the two register files on every step.
bool wmma_wrapper(const std::string& name, Scalar operand, std::string* def, bool tied = false) {
    if (tied) {
        const char* mnemonic = name == "WMMA_16_16_32_bfloat_float" ? "v_mfma_f32_16x16x32_bf16"
                               : name == "WMMA_16_16_32_half_float" ? "v_mfma_f32_16x16x32_f16" : nullptr;
        if (!mnemonic) return false;
        const char* in_t = name == "WMMA_16_16_32_bfloat_float" ? "__bf16" : "_Float16";
        *def = fmt(
            "typedef %s __%s_in __attribute__((ext_vector_type(8)));\n"
            "typedef float __%s_acc __attribute__((ext_vector_type(4)));\n"
            "static __device__ __forceinline__ __%s_acc __%s(__%s_in a, __%s_in b, __%s_acc c) {\n"
            "  asm volatile(\"%s %%0, %%1, %%2, %%0\" : \"+a\"(c) : \"v\"(a), \"v\"(b));\n  return c;\n}\n",
            in_t, name.c_str(), name.c_str(), name.c_str(), name.c_str(), name.c_str(), name.c_str(), name.c_str(), mnemonic);
        return true;
    }
    if (operand == Scalar::Fp8E4M3 || operand == Scalar::Fp8E5M2) {
        if (name != "WMMA_16_16_32_unknown_float") return false;
        const std::string fn = wmma_callee(name, operand);
        *def = fmt(
            "typedef unsigned char __%s_in __attribute__((ext_vector_type(8)));\n"
            "typedef float __%s_acc __attribute__((ext_vector_type(4)));\n"
            "static __device__ __forceinline__ __%s_acc __%s(__%s_in a, __%s_in b, __%s_acc c) {\n"
            "  return %s(__builtin_bit_cast(long, a), __builtin_bit_cast(long, b), c, 0, 0, 0);\n}\n",
            fn.c_str(), fn.c_str(), fn.c_str(), fn.c_str(), fn.c_str(), fn.c_str(), fn.c_str(),
            operand == Scalar::Fp8E4M3 ? "__builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8" : "__builtin_amdgcn_mfma_f32_16x16x32_bf8_bf8");
        return true;
    }
    struct Entry {
        const char* name;
        const char* builtin;
        const char* in_t;
        int in_n, acc_n;
    };
    static const Entry table[] = {
        {"WMMA_16_16_32_bfloat_float", "__builtin_amdgcn_mfma_f32_16x16x32_bf16", "__bf16", 8, 4},
        {"WMMA_16_16_32_half_float", "__builtin_amdgcn_mfma_f32_16x16x32_f16", "_Float16", 8, 4},
        {"WMMA_16_16_16_half_float", "__builtin_amdgcn_mfma_f32_16x16x16f16", "_Float16", 4, 4},
        {"WMMA_16_16_16_bfloat_float", "__builtin_amdgcn_mfma_f32_16x16x16bf16_1k", "__bf16", 4, 4},
        {"WMMA_32_32_16_bfloat_float", "__builtin_amdgcn_mfma_f32_32x32x16_bf16", "__bf16", 8, 16},
        {"WMMA_32_32_16_half_float", "__builtin_amdgcn_mfma_f32_32x32x16_f16", "_Float16", 8, 16},
    };
    for (const Entry& e : table) {
        if (name == e.name) {
            *def = fmt(
                "typedef %s __%s_in __attribute__((ext_vector_type(%d)));\n"
                "typedef float __%s_acc __attribute__((ext_vector_type(%d)));\n"
                "static __device__ __forceinline__ __%s_acc __%s(__%s_in a, __%s_in b, __%s_acc c) {\n"
                "  return %s(a, b, c, 0, 0, 0);\n}\n",
                e.in_t, e.name, e.in_n, e.name, e.acc_n, e.name, e.name, e.name, e.name, e.name, e.builtin);
            return true;
        }
    }
    return false;
}

const char* kWaveReducePreamble = R"(template <int kCtrl> static __device__ __forceinline__ float mrk_dpp(float v) {
  int i = __builtin_bit_cast(int, v);
  i = __builtin_amdgcn_update_dpp(i, i, kCtrl, 0xf, 0xf, false);
  return __builtin_bit_cast(float, i);
}
#define MRK_WAVE_REDUCE(NAME, OP)                                                          \
  static __device__ __forceinline__ float NAME(float v) {                                  \
    v = OP(v, mrk_dpp<0xB1>(v));  /* quad_perm [1,0,3,2] */                               \
    v = OP(v, mrk_dpp<0x4E>(v));  /* quad_perm [2,3,0,1] */                               \
    v = OP(v, mrk_dpp<0x141>(v)); /* row_half_mirror */                                   \
    v = OP(v, mrk_dpp<0x140>(v)); /* row_mirror */                                        \
    float w = __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F)); \
    v = OP(v, w);                                                                          \
    float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));  \
    float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32)); \
    return OP(lo, hi);                                                                     \
  }
#define MRK_OP_ADD(a, b) ((a) + (b))
#define MRK_OP_MUL(a, b) ((a) * (b))
#define MRK_OP_MAX(a, b) fmaxf((a), (b))
#define MRK_OP_MIN(a, b) fminf((a), (b))
MRK_WAVE_REDUCE(mrk_wave_reduce_add, MRK_OP_ADD)
MRK_WAVE_REDUCE(mrk_wave_reduce_mul, MRK_OP_MUL)
MRK_WAVE_REDUCE(mrk_wave_reduce_max, MRK_OP_MAX)
MRK_WAVE_REDUCE(mrk_wave_reduce_min, MRK_OP_MIN)
)";

// ---------------------------------------------------------------- the renderer
class Ctx {
  public:
    std::unordered_map<uint32_t, std::string> names;
    std::unordered_map<uint32_t, size_t> refs;
    std::unordered_set<uint32_t> escaping;
    std::vector<std::string> hoisted;
    std::vector<std::string> body;
    int depth = 1;
    std::map<std::string, int> counters;
    std::vector<std::pair<uint32_t, std::string>> pending_reduces;
    // tensor-core instructions written as assembly (see wmma_wrapper): the register objects that
    // hold their accumulators, (DEFINE_REG id, elements), and how many RANGEs are open
    bool tied_wmma = false;
    // workgroups whose x extent is a whole number of wavefronts: threadIdx.y / .z are the same for
    // the 64 lanes of a wave (declared through readfirstlane, so the compiler keeps what derives
    // from them in scalar registers)
    bool wave_uniform_yz = false;
    std::unordered_map<uint32_t, bool> uniform_memo;
    std::vector<std::pair<uint32_t, int64_t>> acc_regs;
    std::unordered_set<uint32_t> acc_loads_with_other_users;
    int range_depth = 0;
    // The device compiler does not know such a statement as a matrix operation: the wait states it
    // would insert between one and a vector instruction that reads or wrote the same registers
    // are written out, and an empty statement per accumulator keeps its uses on the far side.
    void settle_accumulators(int nops) {
        for (int left = nops; left > 0; left -= 16)
            body.push_back(indent() + fmt("asm volatile(\"s_nop %d\" ::: \"memory\");", (left > 16 ? 16 : left) - 1));
        for (const auto& r : acc_regs) {
            auto it = names.find(r.first);
            if (it == names.end()) continue;
            for (int64_t e = 0; e < r.second; e++)
                body.push_back(indent() + fmt("asm volatile(\"\" : \"+a\"(%s[%" PRId64 "]));", it->second.c_str(), e));
        }
    }

    std::string indent() const { return std::string(static_cast<size_t>(depth) * 2, ' '); }
    std::string next(const std::string& prefix) { return prefix + std::to_string(counters[prefix]++); }
    bool has(uint32_t id) const { return names.count(id) != 0; }
    const std::string& get(uint32_t id) const {
        static const std::string missing = "/*undefined*/";
        auto it = names.find(id);
        return it == names.end() ? missing : it->second;
    }
    // single-use values are inlined into their consumer (ops.rs:85-121)
    std::string emit(const UOp& u, const std::string& expr, const char* prefix, bool force_named = false) {
        size_t rc = refs.count(u.id) ? refs[u.id] : 0;
        if (rc <= 1 && !force_named && !escaping.count(u.id)) {
            names[u.id] = expr;
            return expr;
        }
        std::string name = next(prefix);
        std::string ty = c_dtype(u.dtype);
        if (escaping.count(u.id)) {
            hoisted.push_back("  " + ty + " " + name + ";");
            body.push_back(indent() + name + " = " + expr + ";");
        } else {
            body.push_back(indent() + ty + " " + name + " = " + expr + ";");
        }
        names[u.id] = name;
        return name;
    }
};

class HipRenderer final : public Renderer {
  public:
    explicit HipRenderer(int id) : id_(id) {}
    int device_id() const override { return id_; }

    int render(const LinearKernel& k, const char* name_in, ProgramSpec* out) override {
        const std::string kernel_name = (name_in && *name_in) ? name_in : "kernel";  // device.rs:192-193
        for (char c : kernel_name)
            if (!(std::isalnum(static_cast<unsigned char>(c)) || c == '_'))
                return fail(kRenderError, "render: kernel name is not a C identifier: " + kernel_name);
        const std::vector<UOp>& nodes = k.nodes;
        std::unordered_map<uint32_t, const UOp*> by_id;
        for (const UOp& u : nodes) {
            if (by_id.count(u.id)) return failf(kRenderError, "render: duplicate node id %u", u.id);
            for (uint32_t s : u.src)
                if (!by_id.count(s)) return failf(kRenderError, "render: node %u uses %u before its definition", u.id, s);
            by_id[u.id] = &u;
        }
        auto node = [&](uint32_t id) -> const UOp& { return *by_id.at(id); };

        // ---- buffers sorted by slot -> dataN; variables in stream order (c/mod.rs:56-106)
        std::vector<const UOp*> buffers, variables, specials;
        for (const UOp& u : nodes) {
            if (u.op == Op::Param) buffers.push_back(&u);
            if (u.op == Op::DefineVar) variables.push_back(&u);
            if (u.op == Op::Special) specials.push_back(&u);
        }
        std::stable_sort(buffers.begin(), buffers.end(), [](const UOp* a, const UOp* b) { return a->arg_i < b->arg_i; });
        for (size_t i = 1; i < buffers.size(); i++)
            if (buffers[i]->arg_i == buffers[i - 1]->arg_i)
                return failf(kRenderError, "render: PARAM slot %" PRId64 " appears twice", buffers[i]->arg_i);

        // walk to the PARAM a pointer expression is based on
        std::function<const UOp*(uint32_t)> base_buffer = [&](uint32_t id) -> const UOp* {
            const UOp& u = node(id);
            switch (u.op) {
                case Op::Param:
                case Op::DefineLocal:
                case Op::DefineReg: return &u;
                case Op::Index:
                case Op::Cast:
                case Op::BitCast:
                case Op::After: return u.src.empty() ? nullptr : base_buffer(u.src[0]);
                default: return nullptr;
            }
        };
        std::set<int64_t> out_slots, in_slots;
        for (const UOp& u : nodes) {
            if (u.op == Op::Store && !u.src.empty()) {
                const UOp* b = base_buffer(u.src[0]);
                if (b && b->op == Op::Param) out_slots.insert(b->arg_i);
            }
            if (u.op == Op::Load && !u.src.empty()) {
                const UOp* b = base_buffer(u.src[0]);
                if (b && b->op == Op::Param) in_slots.insert(b->arg_i);
            }
        }

        // ---- launch dims from SPECIAL extents (gpudims.rs:331-382): gidxN -> grid, lidxN -> block
        std::array<size_t, 3> global{1, 1, 1}, local{1, 1, 1};
        for (const UOp* s : specials) {
            if (s->str.size() != 5 || (s->str.compare(0, 4, "gidx") && s->str.compare(0, 4, "lidx")) || s->str[4] < '0' ||
                s->str[4] > '2')
                return fail(kRenderError, "render: SPECIAL name must be gidx0..2 or lidx0..2, got '" + s->str + "'");
            if (s->src.empty() || node(s->src[0]).op != Op::Const)
                return fail(kRenderError, "render: SPECIAL " + s->str + " needs a constant extent");
            int64_t extent = node(s->src[0]).arg_i;
            if (extent <= 0) return fail(kRenderError, "render: SPECIAL " + s->str + " has a non-positive extent");
            auto& dims = s->str[0] == 'g' ? global : local;
            dims[s->str[4] - '0'] = static_cast<size_t>(extent);
        }
        if (local[0] * local[1] * local[2] > 1024)
            return fail(kRenderError, "render: workgroup larger than 1024 work-items");

        Ctx ctx;
        ctx.wave_uniform_yz = local[0] % 64 == 0 && local[1] * local[2] > 1;
        for (const UOp& u : nodes)
            for (uint32_t s : u.src) ctx.refs[s]++;
        ctx.escaping = scope_escaping(nodes, ctx.refs);

        // ---- preamble
        std::vector<std::string> pre;
        std::set<std::pair<int, int>> vec_types;
        for (const UOp& u : nodes)
            if (u.dtype.vcount > 1) vec_types.insert({static_cast<int>(u.dtype.scalar), u.dtype.vcount});
        for (auto& vt : vec_types) {  // types.rs:158-181
            Scalar s = static_cast<Scalar>(vt.first);
            const char* storage = s == Scalar::Bool ? "unsigned char" : c_scalar(s);
            size_t align = 1;
            while (align < scalar_bytes(s) * static_cast<size_t>(vt.second)) align <<= 1;
            pre.push_back(fmt("typedef %s %s%d __attribute__((aligned(%zu), ext_vector_type(%d)));", storage,
                              c_vector_base(s), vt.second, align, vt.second));
        }
        std::set<std::pair<std::string, Scalar>> wmma_names;
        bool uses_wave_reduce = false;
        int64_t reg_bytes = 0;  // per work-item, in declared register objects
        for (const UOp& u : nodes) {
            if (u.op == Op::Wmma) wmma_names.insert({u.str, u.src.empty() ? Scalar::Void : by_id.at(u.src[0])->dtype.scalar});
            if (u.op == Op::WaveReduce) uses_wave_reduce = true;
            if (u.op == Op::DefineReg)
                reg_bytes += (u.dtype.ptr_size > 0 ? u.dtype.ptr_size : 1) * static_cast<int64_t>(scalar_bytes(u.dtype.scalar)) * u.dtype.vcount;
        }
        // A tensor-core kernel with workgroups of four waves or more whose declared registers
        // leave room asks for two waves per SIMD (256 registers each).  Left at one, the device
        // compiler spreads the accumulators over both halves of the 512-entry file and copies
        // them between the halves on every trip of the K loop.  (One-wave workgroups measured
        // slower with the hint, so they go without.)
        const bool two_waves = !wmma_names.empty() && reg_bytes <= 128 * 4 && local[0] * local[1] * local[2] >= 256;
        // more declared registers than half the file: the accumulators go to the accumulation
        // registers, the 16x16x32 instruction is written out (see wmma_wrapper)
        // (one wave per SIMD at most, and operands that reach the tensor core straight from local
        // memory reads, as in the kernels with direct global -> local copies: a vector instruction
        // that produced an operand just before would need wait states nothing inserts)
        bool direct_copies = false;
        for (const UOp& u : nodes) direct_copies = direct_copies || u.op == Op::AsyncCopy;
        if (wmma_names.size() == 1 && reg_bytes > 128 * 4 && direct_copies && local[0] * local[1] * local[2] <= 256) {
            std::string def;
            ctx.tied_wmma = wmma_wrapper(wmma_names.begin()->first, wmma_names.begin()->second, &def, true);
            // ... and only where an accumulator rests for at least eight instructions before the
            // next one adds to it (also around the loop): nothing would make a dependent
            // instruction wait for its predecessor's result
            if (ctx.tied_wmma) {
                auto nf = [&](uint32_t id) -> const UOp& { return *by_id.at(id); };
                std::vector<uint32_t> order;  // register object (or the node itself) each WMMA accumulates into
                for (const UOp& u : nodes)
                    if (u.op == Op::Wmma && u.src.size() >= 3) {
                        const UOp& c = *by_id.at(u.src[2]);
                        const UOp* base = c.op == Op::Load && !c.src.empty() ? base_buffer_of(c.src[0], nf) : nullptr;
                        order.push_back(base && base->op == Op::DefineReg ? base->id : u.src[2]);
                    }
                const size_t n = order.size();
                for (size_t i = 0; i < n && ctx.tied_wmma; i++)
                    for (size_t d = 1; d < 8 && d < n + 1; d++)
                        if (order[(i + d) % n] == order[i]) ctx.tied_wmma = false;
                if (n < 8) ctx.tied_wmma = false;
            }
        }
        if (ctx.tied_wmma) {
            std::set<uint32_t> seen_regs;
            for (const UOp& u : nodes) {
                if (u.op == Op::Store && u.src.size() >= 2 && by_id.at(u.src[1])->op == Op::Wmma) {
                    auto nf = [&](uint32_t id) -> const UOp& { return *by_id.at(id); };
                    const UOp* base = base_buffer_of(u.src[0], nf);
                    if (base && base->op == Op::DefineReg && seen_regs.insert(base->id).second)
                        ctx.acc_regs.push_back({base->id, base->dtype.ptr_size > 0 ? base->dtype.ptr_size : 1});
                }
                if (u.op != Op::Wmma)
                    for (uint32_t sid : u.src)
                        if (by_id.at(sid)->op == Op::Load) ctx.acc_loads_with_other_users.insert(sid);
            }
        }
        for (const auto& w : wmma_names) {
            std::string def;
            if (!wmma_wrapper(w.first, w.second, &def, ctx.tied_wmma)) return fail(kRenderError, "render: no gfx950 MFMA lowering for " + w.first);
            pre.push_back(def);
        }
        if (uses_wave_reduce) pre.push_back(kWaveReducePreamble);
        for (const UOp& u : nodes)
            if (u.op == Op::LoadTr) {
                pre.push_back("typedef __bf16 mrk_tr_bf16x4 __attribute__((__vector_size__(4 * sizeof(__bf16))));\n"
                              "typedef __fp16 mrk_tr_f16x4 __attribute__((__vector_size__(4 * sizeof(__fp16))));");
                break;
            }

        // ---- signature: buffers then variables (c/mod.rs:138-172)
        std::vector<std::string> params;
        ProgramSpec spec;
        for (size_t i = 0; i < buffers.size(); i++) {
            const UOp* b = buffers[i];
            std::string nm = "data" + std::to_string(i);
            const bool is_out = out_slots.count(b->arg_i) != 0;
            params.push_back(std::string(is_out ? "" : "const ") + c_value_type(b->dtype) + "* __restrict__ " + nm);
            ctx.names[b->id] = nm;
            spec.globals.push_back(static_cast<size_t>(b->arg_i));
            if (is_out) spec.outs.push_back(static_cast<size_t>(b->arg_i));
            else if (in_slots.count(b->arg_i)) spec.ins.push_back(static_cast<size_t>(b->arg_i));
        }
        for (const UOp* v : variables) {
            if (v->str.empty()) return fail(kRenderError, "render: DEFINE_VAR without a name");
            const bool wide = v->dtype.scalar == Scalar::Int64 || v->dtype.scalar == Scalar::Index ||
                              v->dtype.scalar == Scalar::UInt64;
            params.push_back(std::string("const ") + c_scalar(v->dtype.scalar) + " " + v->str);
            ctx.names[v->id] = v->str;
            spec.var_names.push_back(v->str);
            spec.var_is_i64.push_back(wide ? 1 : 0);
            Variable var;
            var.name = v->str;
            if (v->extra.size() >= 2) {
                var.min = v->extra[0];
                var.max = v->extra[1];
            }
            spec.vars.push_back(var);
        }

        std::vector<std::string> decls;  // function-scope declarations
        for (const UOp& u : nodes) {
            if (u.op == Op::DefineLocal) {  // c/mod.rs:175-185, as LDS
                std::string nm = "local" + std::to_string(u.arg_i);
                int64_t n = u.dtype.ptr_size > 0 ? u.dtype.ptr_size : 1;
                decls.push_back(fmt("  __shared__ %s %s[%" PRId64 "];", c_value_type(u.dtype).c_str(), nm.c_str(), n));
                ctx.names[u.id] = nm;
            } else if (u.op == Op::Reduce && u.src.size() > 1) {  // c/mod.rs:190-203
                std::string nm = "acc" + std::to_string(u.id);
                decls.push_back("  " + c_dtype(u.dtype) + " " + nm + " = " +
                                reduce_identity(static_cast<ReduceOp>(u.sub), u.dtype) + ";");
                ctx.names[u.id] = nm;
            } else if (u.op == Op::Const) {
                ctx.names[u.id] = c_const(u);
            } else if (u.op == Op::Range) {
                ctx.names[u.id] = "ridx" + std::to_string(u.arg_i);
            }
        }

        // ---- body
        for (const UOp& u : nodes) {
            int rc = render_uop(u, node, ctx);
            if (rc != kOk) return rc;
        }
        if (ctx.depth != 1) return fail(kRenderError, "render: unbalanced RANGE/END or IF/ENDIF");

        std::ostringstream src;
        for (const std::string& l : pre) src << l << "\n";
        if (!pre.empty()) src << "\n";
        src << "extern \"C\" __global__ void __launch_bounds__(" << local[0] * local[1] * local[2] << ") "
            << (two_waves ? "__attribute__((amdgpu_waves_per_eu(2))) " : "") << kernel_name << "(";
        for (size_t i = 0; i < params.size(); i++) src << (i ? ", " : "") << params[i];
        src << ") {\n";
        for (const std::string& l : decls) src << l << "\n";
        for (const std::string& l : ctx.hoisted) src << l << "\n";
        for (const std::string& l : ctx.body) src << l << "\n";
        src << "}\n";

        spec.name = kernel_name;
        spec.src = src.str();
        spec.device_id = id_;
        spec.ast_hash = k.content_hash;
        spec.has_sizes = true;
        spec.global_size = global;
        spec.local_size = local;
        spec.buf_count = buffers.size();
        *out = std::move(spec);
        return kOk;
    }

  private:
    int id_;

    // c/mod.rs:282-333: values defined at a deeper scope than one of their uses get a
    // function-scope declaration.
    static std::unordered_set<uint32_t> scope_escaping(const std::vector<UOp>& nodes,
                                                       std::unordered_map<uint32_t, size_t>& refs) {
        size_t depth = 0;
        std::unordered_map<uint32_t, size_t> def_depth, min_use;
        auto use = [&](const UOp& u) {
            for (uint32_t s : u.src) {
                auto it = min_use.find(s);
                if (it == min_use.end()) min_use[s] = depth;
                else if (depth < it->second) it->second = depth;
            }
        };
        for (const UOp& u : nodes) {
            if (u.op == Op::Range || u.op == Op::If) {
                if (refs[u.id] > 1) def_depth.emplace(u.id, depth);
                use(u);
                depth++;
                continue;
            }
            if (u.op == Op::End) depth = depth >= u.src.size() ? depth - std::max<size_t>(u.src.size(), 1) : 0;
            if (u.op == Op::EndIf) depth = depth ? depth - 1 : 0;
            if (refs[u.id] > 1) def_depth.emplace(u.id, depth);
            use(u);
        }
        std::unordered_set<uint32_t> out;
        for (auto& kv : def_depth) {
            auto it = min_use.find(kv.first);
            if (it != min_use.end() && it->second < kv.second) out.insert(kv.first);
        }
        return out;
    }

    // the PARAM / DEFINE_LOCAL / DEFINE_REG a pointer expression is based on
    template <class NodeFn>
    static const UOp* base_buffer_of(uint32_t id, NodeFn& node) {
        for (;;) {
            const UOp& u = node(id);
            switch (u.op) {
                case Op::Param:
                case Op::DefineLocal:
                case Op::DefineReg: return &u;
                case Op::Index:
                case Op::Cast:
                case Op::BitCast:
                case Op::After:
                    if (u.src.empty()) return nullptr;
                    id = u.src[0];
                    break;
                default: return nullptr;
            }
        }
    }

    // Whether every lane of a wavefront computes the same value for this node: constants, kernel
    // variables, workgroup ids, loop counters, the y / z work-item ids of workgroups whose x extent
    // is a whole number of waves, and integer arithmetic over those.
    template <class NodeFn>
    bool wave_uniform(uint32_t id, NodeFn& node, Ctx& ctx) {
        auto it = ctx.uniform_memo.find(id);
        if (it != ctx.uniform_memo.end()) return it->second;
        const UOp& n = node(id);
        bool r = false;
        switch (n.op) {
            case Op::Const:
            case Op::DefineVar:
            case Op::Range: r = true; break;
            case Op::Special: r = n.str[0] == 'g' || (n.str[4] != '0' && ctx.wave_uniform_yz); break;
            case Op::Unary:
            case Op::Binary:
            case Op::Where:
            case Op::MulAcc:
            case Op::Cast:
                r = !n.src.empty() && n.dtype.vcount <= 1;
                for (uint32_t s : n.src) r = r && wave_uniform(s, node, ctx);
                break;
            default: break;
        }
        return ctx.uniform_memo[id] = r;
    }
    // The terms of an integer sum (a tree of ADDs), split into wave-uniform ones and the rest.
    template <class NodeFn>
    // A sum with per-lane terms is taken apart only where it is inlined into its consumer anyway
    // (single use); a wave-uniform sum (`whole_uniform`) always: its terms live in scalar registers
    // whether or not the sum itself has a name.
    void split_sum(uint32_t id, NodeFn& node, Ctx& ctx, std::vector<uint32_t>* uniform, std::vector<uint32_t>* varying, bool whole_uniform = false) {
        const UOp& n = node(id);
        if (n.op == Op::Binary && static_cast<BinaryOp>(n.sub) == BinaryOp::Add && n.src.size() == 2 && n.dtype.vcount <= 1 &&
            (whole_uniform || (!wave_uniform(id, node, ctx) && ctx.refs[id] <= 1))) {
            split_sum(n.src[0], node, ctx, uniform, varying, whole_uniform);
            split_sum(n.src[1], node, ctx, uniform, varying, whole_uniform);
            return;
        }
        (wave_uniform(id, node, ctx) ? uniform : varying)->push_back(id);
    }

    template <class NodeFn>
    int render_uop(const UOp& u, NodeFn& node, Ctx& ctx) {
        auto S = [&](size_t i) -> const std::string& { return ctx.get(u.src[i]); };
        auto need = [&](size_t n) -> int {
            if (u.src.size() < n)
                return failf(kRenderError, "render: node %u (op %u) needs %zu sources, has %zu", u.id,
                             static_cast<unsigned>(u.op), n, u.src.size());
            return kOk;
        };
        // 8-bit floats are storage and tensor-core operands; C arithmetic on their `unsigned char`
        // carrier would be integer arithmetic
        if (u.op == Op::Unary || u.op == Op::Binary || u.op == Op::Where || u.op == Op::MulAcc || u.op == Op::Cast || u.op == Op::Reduce ||
            u.op == Op::WaveReduce) {
            bool fp8 = u.dtype.is_fp8();
            for (uint32_t sid : u.src) fp8 = fp8 || node(sid).dtype.is_fp8();
            if (fp8) return fail(kRenderError, "render: 8-bit float values can be loaded, stored and fed to a tensor core, nothing else");
        }
        switch (u.op) {
            case Op::Param:
            case Op::DefineVar:
            case Op::DefineLocal:
            case Op::Const:
            case Op::Sink: return kOk;
            case Op::Noop:
                ctx.names[u.id] = "";
                return kOk;

            case Op::DefineReg: {  // ops.rs:144-157
                std::string nm = ctx.next("reg");
                int64_t n = u.dtype.ptr_size > 0 ? u.dtype.ptr_size : 1;
                ctx.body.push_back(ctx.indent() + fmt("%s %s[%" PRId64 "];", c_value_type(u.dtype).c_str(), nm.c_str(), n));
                ctx.names[u.id] = nm;
                return kOk;
            }
            case Op::Special: {
                const char* builtin = u.str[0] == 'g' ? "blockIdx" : "threadIdx";
                const char axis = "xyz"[u.str[4] - '0'];
                const int64_t extent = node(u.src[0]).arg_i;
                if (u.str[0] == 'l' && axis != 'x' && ctx.wave_uniform_yz)
                    ctx.body.push_back(ctx.indent() + fmt("const %s %s = __builtin_amdgcn_readfirstlane(%s.%c); /* %" PRId64 ", the same for a whole wave */",
                                                          c_scalar(u.dtype.scalar), u.str.c_str(), builtin, axis, extent));
                else
                    ctx.body.push_back(ctx.indent() + fmt("const %s %s = %s.%c; /* %" PRId64 " */", c_scalar(u.dtype.scalar),
                                                          u.str.c_str(), builtin, axis, extent));
                ctx.names[u.id] = u.str;
                return kOk;
            }
            case Op::Range: {  // ops.rs:303-316
                MRK_TRY(need(1));
                const std::string& var = ctx.get(u.id);
                // the accumulators' initial values have been written a few wait states back
                if (ctx.tied_wmma && ctx.range_depth == 0) ctx.settle_accumulators(8);
                ctx.range_depth++;
                ctx.body.push_back(ctx.indent() + fmt("for (%s %s = 0; %s < %s; %s++) {", c_scalar(u.dtype.scalar),
                                                      var.c_str(), var.c_str(), S(0).c_str(), var.c_str()));
                ctx.depth++;
                return kOk;
            }
            case Op::End: {  // ops.rs:318-340
                size_t closes = std::max<size_t>(u.src.size(), 1);
                for (size_t i = 0; i < closes; i++) {
                    if (ctx.depth <= 1) return fail(kRenderError, "render: END without an open RANGE");
                    ctx.depth--;
                    ctx.body.push_back(ctx.indent() + "}");
                    if (ctx.range_depth > 0) ctx.range_depth--;
                }
                ctx.pending_reduces.clear();
                // the last results have left the matrix pipe before anything else reads them
                if (ctx.tied_wmma && ctx.range_depth == 0) ctx.settle_accumulators(32);
                return kOk;
            }
            case Op::If:
                MRK_TRY(need(1));
                ctx.body.push_back(ctx.indent() + "if (" + S(0) + ") {");
                ctx.depth++;
                return kOk;
            case Op::EndIf:
                if (ctx.depth <= 1) return fail(kRenderError, "render: ENDIF without an open IF");
                ctx.depth--;
                ctx.body.push_back(ctx.indent() + "}");
                return kOk;
            case Op::Barrier:
                ctx.body.push_back(ctx.indent() + "__syncthreads();");
                if (!u.src.empty()) ctx.names[u.id] = S(0);
                return kOk;
            case Op::After:
                MRK_TRY(need(1));
                ctx.names[u.id] = S(0);
                return kOk;

            case Op::Index: {  // ops.rs:159-176,460-486
                MRK_TRY(need(1));
                size_t nidx = u.src.size() - 1 - (u.sub ? 1 : 0);
                if (nidx == 0) {
                    ctx.names[u.id] = S(0);
                    return kOk;
                }
                std::string idx;
                if (nidx == 1) {
                    idx = S(1);
                } else {
                    if (u.extra.size() != nidx)
                        return failf(kRenderError, "render: multi-index node %u needs %zu row-major strides", u.id, nidx);
                    for (size_t i = 0; i < nidx; i++) {
                        if (u.extra[i] == 0) continue;
                        std::string term = u.extra[i] == 1 ? S(1 + i) : fmt("(%s * %" PRId64 ")", S(1 + i).c_str(), u.extra[i]);
                        idx += (idx.empty() ? "" : " + ") + term;
                    }
                    idx = idx.empty() ? "0" : "(" + idx + ")";
                }
                ctx.emit(u, "(" + S(0) + " + " + idx + ")", "idx");
                return kOk;
            }
            case Op::Load: {  // ops.rs:186-215
                MRK_TRY(need(1));
                const UOp& ix = node(u.src[0]);
                if (ctx.tied_wmma && ctx.range_depth > 0 && ctx.acc_loads_with_other_users.count(u.id)) {
                    const UOp* base = base_buffer_of(u.src[0], node);
                    for (const auto& r : ctx.acc_regs)
                        if (base && base->id == r.first)
                            return fail(kRenderError, "render: inside a loop an accumulator of written-out tensor-core instructions may only "
                                                      "feed the next one (nothing waits for the matrix pipe there)");
                }
                std::string deref = u.dtype.vcount > 1 ? "*((" + c_value_type(u.dtype) + "*)(" + S(0) + "))" : "*(" + S(0) + ")";
                std::string expr = deref;
                if (ix.op == Op::Index && ix.sub) {
                    const std::string& gate = ctx.get(ix.src.back());
                    std::string alt;
                    if (u.src.size() > 1) alt = S(1);
                    else {
                        UOp z;
                        z.dtype = u.dtype;
                        z.dtype.is_ptr = false;
                        alt = c_const(z);
                    }
                    expr = "(" + gate + " ? " + deref + " : " + alt + ")";
                }
                ctx.emit(u, expr, "val", /*force_named=*/true);
                return kOk;
            }
            case Op::Store: {  // ops.rs:217-231
                MRK_TRY(need(2));
                const UOp& v = node(u.src[1]);
                if (v.dtype.vcount > 1)
                    ctx.body.push_back(ctx.indent() + "*((" + c_value_type(v.dtype) + "*)(" + S(0) + ")) = " + S(1) + ";");
                else
                    ctx.body.push_back(ctx.indent() + "*(" + S(0) + ") = " + S(1) + ";");
                return kOk;
            }
            case Op::Unary:
                MRK_TRY(need(1));
                if (u.sub > static_cast<uint16_t>(UnaryOp::Not)) return fail(kRenderError, "render: unknown unary op");
                ctx.emit(u, render_unary(static_cast<UnaryOp>(u.sub), S(0), node(u.src[0]).dtype), "alu");
                return kOk;
            case Op::Binary:
                MRK_TRY(need(2));
                if (u.sub > static_cast<uint16_t>(BinaryOp::Threefry)) return fail(kRenderError, "render: unknown binary op");
                ctx.emit(u, render_binary(static_cast<BinaryOp>(u.sub), S(0), S(1), node(u.src[0]).dtype), "alu");
                return kOk;
            case Op::Where:
                MRK_TRY(need(3));
                ctx.emit(u, "(" + S(0) + " ? " + S(1) + " : " + S(2) + ")", "alu");
                return kOk;
            case Op::MulAcc: {  // ops.rs:257-268
                MRK_TRY(need(3));
                const DType& d = node(u.src[0]).dtype;
                if (d.is_float() && d.vcount == 1)
                    ctx.emit(u, math_call("fma", d, as_float_arg(S(0), d) + ", " + as_float_arg(S(1), d) + ", " + as_float_arg(S(2), d)), "alu");
                else
                    ctx.emit(u, "((" + S(0) + " * " + S(1) + ") + " + S(2) + ")", "alu");
                return kOk;
            }
            case Op::Cast: {  // ops.rs:270-288
                MRK_TRY(need(1));
                const UOp& s = node(u.src[0]);
                if (u.dtype.is_ptr && (s.op == Op::Index || s.dtype.is_ptr)) {
                    ctx.emit(u, "((" + c_value_type(u.dtype) + "*)(" + S(0) + "))", "cast");
                    return kOk;
                }
                if (u.dtype.vcount > 1)
                    ctx.emit(u, "__builtin_convertvector(" + S(0) + ", " + c_value_type(u.dtype) + ")", "cast");
                else
                    ctx.emit(u, "((" + c_dtype(u.dtype) + ")" + S(0) + ")", "cast");
                return kOk;
            }
            case Op::BitCast: {  // ops.rs:290-301
                MRK_TRY(need(1));
                const std::string from = c_dtype(node(u.src[0]).dtype), to = c_dtype(u.dtype);
                if (from == to) ctx.names[u.id] = S(0);
                else ctx.emit(u, "__builtin_bit_cast(" + to + ", (" + from + ")(" + S(0) + "))", "cast");
                return kOk;
            }
            case Op::Gep: {  // ops.rs:363-377
                MRK_TRY(need(1));
                if (u.extra.empty()) return fail(kRenderError, "render: GEP without indices");
                if (u.extra.size() == 1) {
                    ctx.emit(u, fmt("(%s)[%" PRId64 "]", S(0).c_str(), u.extra[0]), "gep");
                } else {
                    std::string e = "(" + c_value_type(u.dtype) + "){";
                    for (size_t i = 0; i < u.extra.size(); i++)
                        e += (i ? ", " : "") + fmt("(%s)[%" PRId64 "]", S(0).c_str(), u.extra[i]);
                    ctx.emit(u, e + "}", "gep");
                }
                return kOk;
            }
            case Op::Vectorize: {  // ops.rs:379-391
                MRK_TRY(need(1));
                if (u.dtype.is_ptr) {
                    ctx.names[u.id] = S(0);
                    return kOk;
                }
                std::string e = "(" + c_value_type(u.dtype) + "){";
                // Arithmetic on 8- and 16-bit integers is carried out in int (the usual
                // promotions); a braced initialiser refuses the narrowing back, an explicit
                // cast of each element states it.
                const Scalar sc = u.dtype.scalar;
                const bool narrow = sc == Scalar::Int8 || sc == Scalar::UInt8 || sc == Scalar::Int16 || sc == Scalar::UInt16;
                DType elem = u.dtype;
                elem.vcount = 1;
                for (size_t i = 0; i < u.src.size(); i++)
                    e += (i ? ", " : "") + (narrow ? "((" + c_value_type(elem) + ")" + S(i) + ")" : S(i));
                ctx.emit(u, e + "}", "vec");
                return kOk;
            }
            case Op::Wmma:  // ops.rs:404-411
                MRK_TRY(need(3));
                ctx.emit(u, "__" + wmma_callee(u.str, node(u.src[0]).dtype.scalar) + "(" + S(0) + ", " + S(1) + ", " + S(2) + ")", "wmma", true);
                // written out, an instruction and what the kernel puts between it and the next one stay in that order
                if (ctx.tied_wmma) ctx.body.push_back(ctx.indent() + "__builtin_amdgcn_sched_barrier(0);");
                return kOk;
            case Op::Reduce: {  // ops.rs:342-361
                MRK_TRY(need(1));
                if (u.src.size() == 1) {
                    ctx.names[u.id] = S(0);
                    return kOk;
                }
                const std::string acc = ctx.get(u.id);
                ctx.body.push_back(ctx.indent() + reduce_accumulate(static_cast<ReduceOp>(u.sub), acc, S(0), u.dtype));
                return kOk;
            }
            case Op::LoadTr: {
                MRK_TRY(need(1));
                const char* bi = u.dtype.scalar == Scalar::BFloat16 ? "__builtin_amdgcn_ds_read_tr16_b64_v4bf16"
                                 : u.dtype.scalar == Scalar::Float16 ? "__builtin_amdgcn_ds_read_tr16_b64_v4f16"
                                                                     : nullptr;
                const UOp* base = base_buffer_of(u.src[0], node);
                if (!bi || u.dtype.vcount != 4 || !base || base->op != Op::DefineLocal)
                    return fail(kRenderError, "render: LOAD_TR reads 4 half / bfloat elements from local memory");
                const char* vt = u.dtype.scalar == Scalar::BFloat16 ? "mrk_tr_bf16x4" : "mrk_tr_f16x4";
                std::string call = fmt("%s((__attribute__((address_space(3))) %s*)(%s))", bi, vt, S(0).c_str());
                ctx.emit(u, "__builtin_bit_cast(" + c_value_type(u.dtype) + ", " + call + ")", "tr", true);
                return kOk;
            }
            case Op::AsyncCopy: {
                MRK_TRY(need(2));
                const UOp* g = base_buffer_of(u.src[0], node);
                const UOp* l = base_buffer_of(u.src[1], node);
                if (!g || g->op != Op::Param || !l || l->op != Op::DefineLocal)
                    return fail(kRenderError, "render: ASYNC_COPY copies from a PARAM to a DEFINE_LOCAL");
                // M0 holds the wave's local-memory destination; the copy itself is invisible to the
                // compiler's wait-count bookkeeping, WAIT_ASYNC is its only ordering.  The destination
                // is formed as the array's own local-memory offset plus an integer byte offset: cast
                // back from a generic pointer it would carry a null check per copy.
                auto sum_of = [&](const std::vector<uint32_t>& terms) {
                    std::string e;
                    for (uint32_t t : terms) e += (e.empty() ? "" : " + ") + ctx.get(t);
                    return e.empty() ? std::string("0") : "(" + e + ")";
                };
                const UOp& li = node(u.src[1]);
                const UOp& gi = node(u.src[0]);
                const int64_t lbytes = static_cast<int64_t>(scalar_bytes(l->dtype.scalar)) * l->dtype.vcount;
                const int64_t gbytes = static_cast<int64_t>(scalar_bytes(g->dtype.scalar)) * g->dtype.vcount;
                const bool plain_dst = li.op == Op::Index && li.src.size() == 2 && !li.sub && node(li.src[0]).op == Op::DefineLocal;
                const bool plain_src = gi.op == Op::Index && gi.src.size() == 2 && !gi.sub && node(gi.src[0]).op == Op::Param && g->dtype.ptr_size > 0 &&
                                       g->dtype.ptr_size * gbytes <= (int64_t(1) << 32);
                if (plain_dst && plain_src && wave_uniform(li.src[1], node, ctx)) {
                    // The form of the hand-written kernels: the destination is wave-uniform, so M0 is written
                    // by the one scalar addition that forms it (the array's base plus the terms that do not
                    // change from copy to copy on one side, the rest on the other); the source is the
                    // buffer's base advanced by the wave-uniform terms of the index in scalar registers
                    // plus the remaining per-lane terms as a 32-bit byte offset, which the compiler hoists
                    // out of the loop when they do not depend on it.
                    std::vector<uint32_t> du, dv, su, sv;
                    split_sum(li.src[1], node, ctx, &du, &dv, true);
                    split_sum(gi.src[1], node, ctx, &su, &sv);
                    std::vector<uint32_t> d_first(du.begin(), du.begin() + (du.size() + 1) / 2), d_rest(du.begin() + (du.size() + 1) / 2, du.end());
                    const std::string m0_a = "(unsigned)(unsigned long long)(__attribute__((address_space(3))) char*)(" + ctx.get(li.src[0]) + ") + (unsigned)" +
                                             sum_of(d_first) + " * " + std::to_string(lbytes) + "u";
                    const std::string m0_b = "(unsigned)" + sum_of(d_rest) + " * " + std::to_string(lbytes) + "u";
                    const std::string src_ops = "\"v\"((unsigned)" + sum_of(sv) + " * " + std::to_string(gbytes) + "u), \"s\"(" + ctx.get(gi.src[0]) + " + " +
                                                sum_of(su) + ")";
                    if (d_rest.empty())
                        ctx.body.push_back(ctx.indent() + "asm volatile(\"s_mov_b32 m0, %0\\n\\ts_nop 0\\n\\tglobal_load_lds_dwordx4 %1, %2\" : : \"s\"(" + m0_a +
                                           "), " + src_ops + " : \"m0\", \"memory\");");
                    else
                        ctx.body.push_back(ctx.indent() + "asm volatile(\"s_add_u32 m0, %0, %1\\n\\ts_nop 0\\n\\tglobal_load_lds_dwordx4 %2, %3\" : : \"s\"(" + m0_a +
                                           "), \"s\"(" + m0_b + "), " + src_ops + " : \"m0\", \"scc\", \"memory\");");
                } else {
                    std::string dst;
                    if (plain_dst)
                        dst = "(unsigned)(unsigned long long)(__attribute__((address_space(3))) char*)(" + ctx.get(li.src[0]) + ") + (unsigned)(" +
                              ctx.get(li.src[1]) + ") * " + std::to_string(lbytes) + "u";
                    else
                        dst = "(unsigned)(unsigned long long)(__attribute__((address_space(3))) char*)(" + S(1) + ")";
                    // source: the buffer's (scalar) base plus a 32-bit byte offset per lane where the buffer
                    // is known to be smaller than 4 GiB (two vector instructions fewer per copy than a
                    // 64-bit address per lane), else the full address
                    if (plain_src)
                        ctx.body.push_back(ctx.indent() + "asm volatile(\"s_mov_b32 m0, %0\\n\\ts_nop 0\\n\\tglobal_load_lds_dwordx4 %1, %2\" : : \"s\"(" +
                                           "__builtin_amdgcn_readfirstlane(" + dst + ")), \"v\"((unsigned)(" + ctx.get(gi.src[1]) + ") * " +
                                           std::to_string(gbytes) + "u), \"s\"(" + ctx.get(gi.src[0]) + ") : \"m0\", \"memory\");");
                    else
                        ctx.body.push_back(ctx.indent() + "asm volatile(\"s_mov_b32 m0, %0\\n\\ts_nop 0\\n\\tglobal_load_lds_dwordx4 %1, off\" : : \"s\"(" +
                                           "__builtin_amdgcn_readfirstlane(" + dst + ")), \"v\"((const char*)(" + S(0) + ")) : \"m0\", \"memory\");");
                }
                // next to written-out tensor-core instructions the copy stays where the kernel puts it
                // (a builder that spreads copies over a stretch of them means exactly that placement)
                if (ctx.tied_wmma) ctx.body.push_back(ctx.indent() + "__builtin_amdgcn_sched_barrier(0);");
                return kOk;
            }
            case Op::WaitAsync:
                if (u.arg_i < 0 || u.arg_i > 63) return fail(kRenderError, "render: WAIT_ASYNC takes a count of 0..63");
                ctx.body.push_back(ctx.indent() + fmt("asm volatile(\"s_waitcnt vmcnt(%d)\" ::: \"memory\");", static_cast<int>(u.arg_i)));
                return kOk;
            case Op::WaveReduce: {
                MRK_TRY(need(1));
                if (u.dtype.scalar != Scalar::Float32 || u.dtype.vcount != 1)
                    return fail(kRenderError, "render: WAVE_REDUCE is lowered for scalar float32 only");
                static const char* fn[] = {"mrk_wave_reduce_add", "mrk_wave_reduce_mul", "mrk_wave_reduce_max",
                                           "mrk_wave_reduce_min"};
                if (u.sub > 3) return fail(kRenderError, "render: unknown reduce op");
                ctx.emit(u, std::string(fn[u.sub]) + "(" + S(0) + ")", "red", true);
                return kOk;
            }
        }
        return failf(kRenderError, "render: unsupported op %u", static_cast<unsigned>(u.op));
    }
};

}  // namespace

std::shared_ptr<Renderer> make_hip_renderer(int device_id) { return std::make_shared<HipRenderer>(device_id); }

}  // namespace mrk
