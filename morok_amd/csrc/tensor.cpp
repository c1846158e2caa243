#include "tensor.h"
#include "kernels/kernels.h"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <mutex>
#include <set>
#include <tuple>
#include <unordered_map>

#include "builtin.h"
#include "device.h"
#include "error.h"
#include "runtime.h"
#include "schedule.h"

namespace mrk {

// ============================================================================ small helpers
size_t scalar_size(Scalar s) {
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
        case Scalar::Void: return 0;
        default: return 8;
    }
}

static bool is_float(Scalar s) {
    return s == Scalar::Float16 || s == Scalar::BFloat16 || s == Scalar::Float32 || s == Scalar::Float64;
}
static bool is_half(Scalar s) { return s == Scalar::Float16 || s == Scalar::BFloat16; }

// dtype/src/cast.rs:88: the smallest type both promote to (restricted to the types used here)
Scalar least_upper_dtype(Scalar a, Scalar b) {
    if (a == b) return a;
    auto frank = [](Scalar s) {
        switch (s) {
            case Scalar::Float16:
            case Scalar::BFloat16: return 1;
            case Scalar::Float32: return 2;
            case Scalar::Float64: return 3;
            default: return 0;
        }
    };
    if (is_float(a) && is_float(b)) {
        if (frank(a) == 1 && frank(b) == 1) return Scalar::Float32;  // half with bfloat16
        return frank(a) > frank(b) ? a : b;
    }
    if (is_float(a)) return a;
    if (is_float(b)) return b;
    auto irank = [](Scalar s) {
        switch (s) {
            case Scalar::Bool: return 0;
            case Scalar::Int8:
            case Scalar::UInt8: return 1;
            case Scalar::Int16:
            case Scalar::UInt16: return 2;
            case Scalar::Int32:
            case Scalar::UInt32: return 3;
            default: return 4;
        }
    };
    return irank(a) >= irank(b) ? a : b;
}

static thread_local bool g_fusion = true;
static thread_local RealizeStats g_stats;
void set_fusion_enabled(bool on) { g_fusion = on; }
bool fusion_enabled() { return g_fusion; }
const RealizeStats& last_realize_stats() { return g_stats; }

static Tensor bad(Status code, const std::string& msg) {
    fail(code, msg);
    return Tensor();
}
static std::string shape_str(const std::vector<int64_t>& s) {
    std::string r = "[";
    for (size_t i = 0; i < s.size(); i++) r += (i ? ", " : "") + std::to_string(s[i]);
    return r + "]";
}
static TensorRef mk(TKind kind, Scalar dt, std::vector<int64_t> shape, std::vector<TensorRef> src, int dev) {
    auto n = std::make_shared<TensorNode>();
    n->kind = kind;
    n->dtype = dt;
    n->shape = std::move(shape);
    n->src = std::move(src);
    n->device_id = dev;
    return n;
}
// nodes whose value always exists in memory before a consumer kernel reads it
static bool is_boundary_kind(const TensorNode* n) {
    return n->kind == TKind::Reduce || n->kind == TKind::Contiguous || n->kind == TKind::Copy;
}
static std::string device_name(int device_id) {
    return device_id == kCpuDevice ? std::string("CPU") : "HIP:" + std::to_string(device_id);
}
static bool norm_axis(int64_t* a, int64_t nd) {
    if (*a < 0) *a += nd;
    return *a >= 0 && *a < nd;
}

// ============================================================================ graph building
Tensor Tensor::from_raw_bytes(int device_id, const void* data, size_t nbytes, const std::vector<int64_t>& shape,
                              Scalar dtype) {
    int64_t numel = 1;
    for (int64_t d : shape) {
        if (d < 0) return bad(kInvalidArgument, "from_raw_bytes: negative dimension");
        numel *= d;
    }
    const size_t expected = static_cast<size_t>(numel) * scalar_size(dtype);
    if (nbytes != expected)  // data.rs:81-96
        return bad(kSizeMismatch, "from_raw_bytes: data length " + std::to_string(nbytes) + " != expected " +
                                      std::to_string(expected) + " (" + std::to_string(numel) + " elements * " +
                                      std::to_string(scalar_size(dtype)) + " bytes)");
    std::shared_ptr<Device> dev;
    if (DeviceFactoryRegistry::global().device("HIP", device_id, &dev) != kOk) return Tensor();
    BufferOptions opt;
    auto buf = std::make_shared<Buffer>(dev->allocator, expected, opt);
    if (expected && buf->copyin(data, expected) != kOk) return Tensor();  // data.rs:66-67: copied at creation
    return from_buffer(buf, shape, dtype);
}

Tensor Tensor::from_host_bytes(const void* data, size_t nbytes, const std::vector<int64_t>& shape, Scalar dtype) {
    int64_t numel = 1;
    for (int64_t d : shape) {
        if (d < 0) return bad(kInvalidArgument, "from_slice: negative dimension");
        numel *= d;
    }
    const size_t expected = static_cast<size_t>(numel) * scalar_size(dtype);
    if (nbytes != expected)  // data.rs:81-96
        return bad(kSizeMismatch, "from_raw_bytes: data length " + std::to_string(nbytes) + " != expected " +
                                      std::to_string(expected) + " (" + std::to_string(numel) + " elements * " +
                                      std::to_string(scalar_size(dtype)) + " bytes)");
    if (expected && !data) return bad(kInvalidArgument, "from_slice: null data");
    auto n = mk(TKind::Buffer, dtype, shape, {}, kCpuDevice);
    const uint8_t* p = static_cast<const uint8_t*>(data);
    n->host = std::make_shared<std::vector<uint8_t>>(p, p + expected);  // data.rs:66-67: copied at creation
    return Tensor(n);
}

Tensor Tensor::to(int device_id) const {
    if (!n_) return bad(kInvalidArgument, "to: invalid tensor");
    if (n_->device_id == device_id) return *this;  // lib.rs:480-482
    if (device_id != kCpuDevice) {
        int count = 0;
        if (ffi::device_count(&count) != 0 || device_id < 0 || device_id >= count)
            return bad(kInvalidDevice, "invalid device: HIP:" + std::to_string(device_id));
    }
    return Tensor(mk(TKind::Copy, n_->dtype, n_->shape, {n_}, device_id));
}

Tensor Tensor::from_buffer(std::shared_ptr<Buffer> buf, const std::vector<int64_t>& shape, Scalar dtype) {
    int64_t numel = 1;
    for (int64_t d : shape) numel *= d;
    if (static_cast<size_t>(numel) * scalar_size(dtype) != buf->size())
        return bad(kSizeMismatch, "from_buffer: buffer size does not match shape " + shape_str(shape));
    // kernels read and write 16 bytes per access: a view has to start on such a boundary
    if (buf->offset() % 16 != 0) return bad(kInvalidArgument, "from_buffer: a buffer view must start at a multiple of 16 bytes");
    auto n = mk(TKind::Buffer, dtype, shape, {}, buf->device_id());
    n->buffer = std::move(buf);
    return Tensor(n);
}

Tensor Tensor::const_(double value, Scalar dtype, int device_id) {
    auto n = mk(TKind::Const, dtype, {}, {}, device_id);
    n->cval = value;
    return Tensor(n);
}

Tensor Tensor::full(const std::vector<int64_t>& shape, double value, Scalar dtype, int device_id) {
    std::vector<int64_t> ones(shape.size(), 1);
    return const_(value, dtype, device_id).try_reshape(ones).try_expand(shape);
}

Tensor Tensor::try_reshape(const std::vector<int64_t>& shape_in) const {
    if (!n_) return Tensor();
    std::vector<int64_t> shape = shape_in;
    int64_t known = 1, infer = -1;
    for (size_t i = 0; i < shape.size(); i++) {
        if (shape[i] == -1) {
            if (infer >= 0) return bad(kInvalidArgument, "reshape: more than one -1");
            infer = static_cast<int64_t>(i);
        } else if (shape[i] < 0) {
            return bad(kInvalidArgument, "reshape: negative dimension");
        } else {
            known *= shape[i];
        }
    }
    const int64_t numel = n_->numel();
    if (infer >= 0) {
        if (known == 0 || numel % known) return bad(kInvalidArgument, "reshape: cannot infer dimension");
        shape[infer] = numel / known;
        known *= shape[infer];
    }
    if (known != numel)
        return bad(kInvalidArgument, "reshape: " + shape_str(n_->shape) + " -> " + shape_str(shape) + " changes the element count");
    if (shape == n_->shape) return *this;
    return Tensor(mk(TKind::Reshape, n_->dtype, shape, {n_}, n_->device_id));
}

Tensor Tensor::try_permute(const std::vector<int64_t>& perm_in) const {
    if (!n_) return Tensor();
    const int64_t nd = ndim();
    std::vector<int64_t> perm = perm_in, shape(perm.size());
    if (static_cast<int64_t>(perm.size()) != nd) return bad(kInvalidArgument, "permute: wrong number of axes");
    std::vector<bool> seen(nd, false);
    for (int64_t i = 0; i < nd; i++) {
        if (!norm_axis(&perm[i], nd) || seen[perm[i]]) return bad(kInvalidArgument, "permute: invalid permutation");
        seen[perm[i]] = true;
        shape[i] = n_->shape[perm[i]];
    }
    auto n = mk(TKind::Permute, n_->dtype, shape, {n_}, n_->device_id);
    n->arg = perm;
    return Tensor(n);
}

Tensor Tensor::try_transpose(int64_t a, int64_t b) const {
    if (!n_) return Tensor();
    const int64_t nd = ndim();
    if (!norm_axis(&a, nd) || !norm_axis(&b, nd)) return bad(kInvalidArgument, "transpose: axis out of range");
    std::vector<int64_t> perm(nd);
    for (int64_t i = 0; i < nd; i++) perm[i] = i;
    std::swap(perm[a], perm[b]);
    return try_permute(perm);
}

Tensor Tensor::try_expand(const std::vector<int64_t>& shape_in) const {
    if (!n_) return Tensor();
    if (shape_in.size() != n_->shape.size()) return bad(kInvalidArgument, "expand: rank mismatch");
    std::vector<int64_t> shape = shape_in;
    for (size_t i = 0; i < shape.size(); i++) {
        if (shape[i] == -1) shape[i] = n_->shape[i];
        if (shape[i] != n_->shape[i] && n_->shape[i] != 1)
            return bad(kInvalidArgument, "expand: " + shape_str(n_->shape) + " cannot broadcast to " + shape_str(shape));
    }
    if (shape == n_->shape) return *this;
    return Tensor(mk(TKind::Expand, n_->dtype, shape, {n_}, n_->device_id));
}

Tensor Tensor::try_shrink(const std::vector<int64_t>& begin, const std::vector<int64_t>& end) const {
    if (!n_) return Tensor();
    if (begin.size() != n_->shape.size() || end.size() != begin.size()) return bad(kInvalidArgument, "shrink: rank mismatch");
    std::vector<int64_t> shape(begin.size());
    for (size_t i = 0; i < begin.size(); i++) {
        if (begin[i] < 0 || end[i] > n_->shape[i] || begin[i] > end[i]) return bad(kInvalidArgument, "shrink: range out of bounds");
        shape[i] = end[i] - begin[i];
    }
    auto n = mk(TKind::Shrink, n_->dtype, shape, {n_}, n_->device_id);
    n->arg = begin;
    return Tensor(n);
}

Tensor Tensor::try_unsqueeze(int64_t axis) const {
    if (!n_) return Tensor();
    int64_t nd = ndim() + 1;
    if (!norm_axis(&axis, nd)) return bad(kInvalidArgument, "unsqueeze: axis out of range");
    std::vector<int64_t> shape = n_->shape;
    shape.insert(shape.begin() + axis, 1);
    return try_reshape(shape);
}

Tensor Tensor::try_squeeze(int64_t axis) const {
    if (!n_) return Tensor();
    if (!norm_axis(&axis, ndim()) || n_->shape[axis] != 1) return bad(kInvalidArgument, "squeeze: axis is not of size 1");
    std::vector<int64_t> shape = n_->shape;
    shape.erase(shape.begin() + axis);
    return try_reshape(shape);
}

Tensor Tensor::contiguous() const {
    if (!n_) return Tensor();
    if (n_->kind == TKind::Buffer || n_->kind == TKind::Contiguous) return *this;
    return Tensor(mk(TKind::Contiguous, n_->dtype, n_->shape, {n_}, n_->device_id));
}

Tensor Tensor::cat(const std::vector<Tensor>& parts, int64_t axis) {
    if (parts.empty()) return bad(kInvalidArgument, "cat: no tensors");
    for (const Tensor& p : parts)
        if (!p.valid()) return Tensor();
    const int64_t nd = parts[0].ndim();
    if (!norm_axis(&axis, nd)) return bad(kInvalidArgument, "cat: axis out of range");
    std::vector<int64_t> shape = parts[0].shape();
    std::vector<TensorRef> src;
    int64_t total = 0;
    for (const Tensor& p : parts) {
        if (p.ndim() != nd || p.dtype() != parts[0].dtype()) return bad(kInvalidArgument, "cat: rank or dtype mismatch");
        for (int64_t i = 0; i < nd; i++)
            if (i != axis && p.shape()[i] != shape[i]) return bad(kInvalidArgument, "cat: shape mismatch");
        total += p.shape()[axis];
        src.push_back(p.node());
    }
    shape[axis] = total;
    auto n = mk(TKind::Cat, parts[0].dtype(), shape, src, parts[0].node()->device_id);
    n->arg = {axis};
    return Tensor(n);
}

Tensor Tensor::cast(Scalar dtype) const {
    if (!n_) return Tensor();
    if (dtype == n_->dtype) return *this;
    return Tensor(mk(TKind::Cast, dtype, n_->shape, {n_}, n_->device_id));
}

Tensor Tensor::unary(UnaryOp op) const {
    if (!n_) return Tensor();
    auto n = mk(TKind::Unary, n_->dtype, n_->shape, {n_}, n_->device_id);
    n->sub = static_cast<uint16_t>(op);
    return Tensor(n);
}

// numpy-style broadcast of `t` to `shape` (explicit reshape + expand nodes, as the reference's
// binary ops insert them)
static Tensor broadcast_to(const Tensor& t, const std::vector<int64_t>& shape) {
    std::vector<int64_t> padded(shape.size() - t.shape().size(), 1);
    padded.insert(padded.end(), t.shape().begin(), t.shape().end());
    return t.try_reshape(padded).try_expand(shape);
}
static bool broadcast_shape(const std::vector<int64_t>& a, const std::vector<int64_t>& b, std::vector<int64_t>* out) {
    size_t n = std::max(a.size(), b.size());
    out->assign(n, 1);
    for (size_t i = 0; i < n; i++) {
        int64_t da = i < n - a.size() ? 1 : a[i - (n - a.size())];
        int64_t db = i < n - b.size() ? 1 : b[i - (n - b.size())];
        if (da != db && da != 1 && db != 1) return false;
        (*out)[i] = da == 1 ? db : da;
    }
    return true;
}

Tensor Tensor::binary(BinaryOp op, const Tensor& other) const {
    if (!n_ || !other.n_) return Tensor();
    std::vector<int64_t> shape;
    if (!broadcast_shape(n_->shape, other.n_->shape, &shape))
        return bad(kInvalidArgument, "binary op: shapes " + shape_str(n_->shape) + " and " + shape_str(other.n_->shape) + " do not broadcast");
    Scalar dt = least_upper_dtype(n_->dtype, other.n_->dtype);
    Tensor a = broadcast_to(cast(dt), shape), b = broadcast_to(other.cast(dt), shape);
    if (!a.valid() || !b.valid()) return Tensor();
    Scalar out = dt;
    switch (op) {
        case BinaryOp::Lt:
        case BinaryOp::Le:
        case BinaryOp::Gt:
        case BinaryOp::Ge:
        case BinaryOp::Eq:
        case BinaryOp::Ne: out = Scalar::Bool; break;
        default: break;
    }
    auto n = mk(TKind::Binary, out, shape, {a.n_, b.n_}, n_->device_id);
    n->sub = static_cast<uint16_t>(op);
    return Tensor(n);
}

Tensor Tensor::where_(const Tensor& cond, const Tensor& other) const {
    if (!n_ || !cond.n_ || !other.n_) return Tensor();
    std::vector<int64_t> s1, shape;
    if (!broadcast_shape(n_->shape, other.n_->shape, &s1) || !broadcast_shape(s1, cond.n_->shape, &shape))
        return bad(kInvalidArgument, "where: shapes do not broadcast");
    Scalar dt = least_upper_dtype(n_->dtype, other.n_->dtype);
    Tensor c = broadcast_to(cond.cast(Scalar::Bool), shape), t = broadcast_to(cast(dt), shape),
           f = broadcast_to(other.cast(dt), shape);
    if (!c.valid() || !t.valid() || !f.valid()) return Tensor();
    return Tensor(mk(TKind::Where, dt, shape, {c.n_, t.n_, f.n_}, n_->device_id));
}

Tensor Tensor::sigmoid() const {
    // sigmoid(x) = 1 / (1 + exp2(x * (-1/ln 2)))  (activation.rs:42-52)
    if (!n_) return Tensor();
    Tensor scaled = try_mul(const_(-1.0 / 0.6931471805599453, n_->dtype, n_->device_id));
    Tensor e = scaled.try_exp2();
    return const_(1.0, n_->dtype, n_->device_id).try_add(e).unary(UnaryOp::Reciprocal);
}
Tensor Tensor::swish() const {
    Tensor res = try_mul(sigmoid());
    if (res.valid()) {  // remembered so that silu(gate) * up over one packed product can run in that product's epilogue
        res.node()->hint = HintKind::Swish;
        res.node()->hint_inputs = {n_};
    }
    return res;
}
Tensor Tensor::tanh() const {
    // tanh(x) = 2 * sigmoid(2x) - 1  (activation.rs:64-74)
    if (!n_) return Tensor();
    Tensor two = const_(2.0, n_->dtype, n_->device_id);
    Tensor sig = try_mul(two).sigmoid();
    return two.try_mul(sig).try_sub(const_(1.0, n_->dtype, n_->device_id));
}

Tensor Tensor::reduce(ReduceOp op, std::vector<int64_t> axes, bool keepdim, bool promote) const {
    if (!n_) return Tensor();
    const int64_t nd = ndim();
    std::set<int64_t> ax;
    for (int64_t a : axes) {
        if (!norm_axis(&a, nd)) return bad(kInvalidArgument, "reduce: axis out of range");
        ax.insert(a);
    }
    // accumulation dtype (reduce.rs:101-117)
    Scalar acc = n_->dtype;
    if (promote) {
        switch (n_->dtype) {
            case Scalar::Bool:
            case Scalar::Int8:
            case Scalar::Int16: acc = Scalar::Int32; break;
            case Scalar::UInt8:
            case Scalar::UInt16: acc = Scalar::UInt32; break;
            case Scalar::Float16:
            case Scalar::BFloat16: acc = Scalar::Float32; break;
            default: break;
        }
    }
    Tensor work = cast(acc);
    std::vector<int64_t> kshape = n_->shape, oshape;
    for (int64_t i = 0; i < nd; i++) {
        if (ax.count(i)) kshape[i] = 1;
        else oshape.push_back(n_->shape[i]);
    }
    auto r = mk(TKind::Reduce, acc, kshape, {work.n_}, n_->device_id);
    r->sub = static_cast<uint16_t>(op);
    r->arg.assign(ax.begin(), ax.end());
    Tensor res(r);
    if (!keepdim) res = res.try_reshape(oshape);
    // cast back after a promoted sum of a half type (reduce.rs:665-691)
    if (promote && is_half(n_->dtype)) res = res.cast(n_->dtype);
    return res;
}

Tensor Tensor::mean(std::vector<int64_t> axes, bool keepdim) const {
    if (!n_) return Tensor();
    int64_t count = 1;
    for (int64_t a : axes) {
        if (!norm_axis(&a, ndim())) return bad(kInvalidArgument, "mean: axis out of range");
        count *= n_->shape[a];
    }
    Tensor s = reduce(ReduceOp::Add, axes, keepdim, true);
    if (!s.valid()) return s;
    // x / c is rewritten to x * (1/c) before rendering (schedule/src/optimizer/mod.rs:414-434)
    return s.try_mul(const_(1.0 / static_cast<double>(count), s.dtype(), n_->device_id));
}

Tensor Tensor::matmul(const Tensor& other, Scalar acc) const {
    if (!n_ || !other.n_) return Tensor();
    const int64_t dx = ndim(), dw = other.ndim();
    if (dx == 0 || dw == 0) return bad(kInvalidArgument, "matmul: 0-d operand");
    const int64_t k = n_->shape[dx - 1];
    const int64_t axis_w = dw >= 2 ? dw - 2 : 0;
    if (other.n_->shape[axis_w] != k)
        return bad(kInvalidArgument, "matmul: shapes " + shape_str(n_->shape) + " and " + shape_str(other.n_->shape) + " do not contract");
    // x[..., M, K] -> [..., M, 1, K];  w[..., K, N] -> [..., 1, N, K];  product.sum(-1)  (matmul.rs:96-109).
    // The broadcast axis is only inserted when both sides have one to pair it with: a vector
    // operand multiplies as it is ([K] * [N, K], [M, K] * [K], [K] * [K]).
    const int64_t bd = std::min<int64_t>({dx - 1, dw - 1, 1});
    std::vector<int64_t> xs = n_->shape;
    if (bd) xs.insert(xs.end() - 1, 1);
    Tensor wt = dw >= 2 ? other.try_transpose(-1, -2) : other;
    std::vector<int64_t> ws = wt.shape();
    if (bd) ws.insert(ws.end() - 2, 1);
    Tensor prod = try_reshape(xs).try_mul(wt.try_reshape(ws));
    if (acc != Scalar::Void) return prod.cast(acc).reduce(ReduceOp::Add, {-1}, false, false);  // sum_with().dtype(): reduce.rs:636-673
    Tensor res = prod.reduce(ReduceOp::Add, {-1}, false, true);
    if (!res.valid() || dx < 2 || dw < 2) return res;
    res.node()->hint = HintKind::Matmul;
    res.node()->hint_inputs = {n_, other.n_};
    return res;
}

Tensor Tensor::gemm(const Tensor& b, float alpha, float beta, bool trans_a, bool trans_b, const Tensor* c) const {
    if (!n_ || !b.valid()) return Tensor();
    Tensor a = trans_a ? try_transpose(0, 1) : *this;
    Tensor bb = trans_b ? b.try_transpose(0, 1) : b;
    Tensor res = a.matmul(bb);
    if (!res.valid()) return res;
    // the reference multiplies by f32 one-element tensors (matmul.rs:125-131): f32 promotion rules apply
    if (alpha != 1.0f) res = res.try_mul(full({1}, alpha, Scalar::Float32, n_->device_id));
    if (c) {
        if (!c->valid()) return Tensor();
        Tensor cc = beta != 1.0f ? c->try_mul(full({1}, beta, Scalar::Float32, n_->device_id)) : *c;
        res = res.try_add(cc);
    }
    return res;
}

Tensor Tensor::linear(const Tensor& weight, const Tensor* bias, Scalar acc) const {
    if (!n_ || !weight.valid()) return Tensor();
    Tensor res;
    if (weight.ndim() == 1) {
        res = acc != Scalar::Void ? cast(acc).try_mul(weight) : try_mul(weight);
    } else {
        res = matmul(weight.try_transpose(-1, -2), acc);
    }
    if (!res.valid() || !bias) return res;
    if (!bias->valid()) return Tensor();
    return res.try_add(*bias);  // broadcast to the result's shape
}

Tensor Tensor::softmax(int64_t axis) const {
    if (!n_) return Tensor();
    if (!norm_axis(&axis, ndim())) return bad(kInvalidArgument, "softmax: axis out of range");
    Tensor m = reduce(ReduceOp::Max, {axis}, true, false);
    Tensor e = try_sub(m).try_exp();
    Tensor s = e.reduce(ReduceOp::Add, {axis}, true, false);  // sum_with: no promotion (reduce.rs:197-205)
    Tensor res = e.try_div(s);
    if (!res.valid()) return res;
    res.node()->hint = HintKind::Softmax;
    res.node()->hint_inputs = {n_};
    res.node()->arg = {axis};
    return res;
}

Tensor Tensor::log_softmax(int64_t axis) const {
    // x - max(x) - log(sum(exp(x - max(x))))  (activation.rs:117-128)
    if (!n_) return Tensor();
    if (!norm_axis(&axis, ndim())) return bad(kInvalidArgument, "log_softmax: axis out of range");
    Tensor shifted = try_sub(reduce(ReduceOp::Max, {axis}, true, false));
    Tensor s = shifted.try_exp().reduce(ReduceOp::Add, {axis}, true, false);
    return shifted.try_sub(s.unary(UnaryOp::Log));
}

Tensor Tensor::logsumexp(int64_t axis) const {
    // max(x) + log(sum(exp(x - max(x)))), the kept axis dropped by a max over it  (activation.rs:143-157)
    if (!n_) return Tensor();
    if (!norm_axis(&axis, ndim())) return bad(kInvalidArgument, "logsumexp: axis out of range");
    Tensor m = reduce(ReduceOp::Max, {axis}, true, false);
    Tensor s = try_sub(m).try_exp().reduce(ReduceOp::Add, {axis}, true, false);
    return m.try_add(s.unary(UnaryOp::Log)).reduce(ReduceOp::Max, {axis}, false, false);
}

Tensor Tensor::rms_norm(int64_t axis, double eps) const {
    if (!n_) return Tensor();
    if (!norm_axis(&axis, ndim())) return bad(kInvalidArgument, "rms_norm: axis out of range");
    std::vector<int64_t> axes;
    for (int64_t a = axis; a < ndim(); a++) axes.push_back(a);
    Tensor x32 = cast(Scalar::Float32);
    Tensor norm = x32.square().mean(axes, true).try_add(const_(eps, Scalar::Float32, n_->device_id)).try_rsqrt();
    return try_mul(norm);  // bf16 * f32 promotes to f32 (dtype/src/cast.rs:88)
}

Tensor Tensor::embedding(const Tensor& indices) const {
    if (!n_ || !indices.n_) return Tensor();
    if (ndim() != 2) return bad(kInvalidArgument, "embedding: weight must be [vocab, dim]");
    std::vector<int64_t> shape = indices.shape();
    shape.push_back(n_->shape[1]);
    Tensor idx = indices.cast(Scalar::Int32);
    return Tensor(mk(TKind::Gather, n_->dtype, shape, {n_, idx.n_}, n_->device_id));
}

Tensor Tensor::apply_rotary_emb(const Tensor& cos, const Tensor& sin, bool interleaved) const {
    if (!n_ || !cos.valid() || !sin.valid()) return Tensor();
    const int64_t nd = ndim();
    if (nd == 0) return bad(kInvalidArgument, "apply_rotary_emb requires non-scalar input");
    const int64_t last = n_->shape[nd - 1], half = last / 2;
    if (last % 2) return bad(kInvalidArgument, "apply_rotary_emb: last dim must be even");
    Tensor x1, x2;
    std::vector<int64_t> b0(nd, 0), e0 = n_->shape;
    if (interleaved) {
        std::vector<int64_t> rs(n_->shape.begin(), n_->shape.end() - 1);
        rs.push_back(half);
        rs.push_back(2);
        Tensor r = try_reshape(rs);
        std::vector<int64_t> b(nd + 1, 0), e = rs;
        e[nd] = 1;
        x1 = r.try_shrink(b, e).try_squeeze(-1);
        b[nd] = 1;
        e[nd] = 2;
        x2 = r.try_shrink(b, e).try_squeeze(-1);
    } else {
        std::vector<int64_t> e = e0, b = b0;
        e[nd - 1] = half;
        x1 = try_shrink(b, e);
        b[nd - 1] = half;
        e[nd - 1] = last;
        x2 = try_shrink(b, e);
    }
    Tensor real = x1.try_mul(cos).try_sub(x2.try_mul(sin));
    Tensor imag = x1.try_mul(sin).try_add(x2.try_mul(cos));
    if (!real.valid() || !imag.valid()) return Tensor();
    if (interleaved) {
        Tensor st = cat({real.try_unsqueeze(-1), imag.try_unsqueeze(-1)}, -1);
        std::vector<int64_t> fs = real.shape();
        fs.back() = last;
        return st.try_reshape(fs);
    }
    Tensor out = cat({real, imag}, -1);
    if (out.valid()) {  // what this subgraph computes, for the scheduler (a product kernel can apply it in its epilogue)
        out.node()->hint = HintKind::Rope;
        out.node()->hint_inputs = {n_, cos.node(), sin.node()};
    }
    return out;
}

Tensor Tensor::scaled_dot_product_attention(const Tensor& key, const Tensor& value, double scale, bool is_causal,
                                            const Tensor* attn_mask, double softcap) const {
    if (!n_ || !key.valid() || !value.valid()) return Tensor();
    const int64_t nd = ndim();
    if (nd < 2 || key.ndim() != nd || value.ndim() != nd) return bad(kInvalidArgument, "sdpa: rank mismatch");
    const int64_t head_dim = n_->shape[nd - 1];
    const double scale_val = scale > 0.0 ? scale : 1.0 / std::sqrt(static_cast<double>(head_dim));  // transformer.rs:90-91
    const Scalar sdt = n_->dtype;
    // A head dim without a fused instantiation (80, 96, 192 ...) is padded with zero columns up to
    // the next one that has (64, 128, 256): zero columns add exact zeros to every score, the
    // padded columns of V give zero outputs that are cut off again, and the scale stays that of
    // the real head dim.  Three padded copies instead of a materialised [Sq, Sk] score matrix.
    if (nd == 4 && sdt == Scalar::BFloat16 && head_dim > 0 && head_dim < 256 && head_dim != 64 &&
        head_dim != 128 && key.shape()[3] == head_dim && value.shape()[3] == head_dim && key.dtype() == sdt && value.dtype() == sdt &&
        n_->numel() > 0 && key.node()->numel() > 0) {
        const int64_t padded = head_dim < 64 ? 64 : head_dim < 128 ? 128 : 256;
        auto pad = [&](const Tensor& t) {
            std::vector<int64_t> zs = t.shape();
            zs[3] = padded - head_dim;
            return Tensor::cat({t, Tensor::full(zs, 0.0, sdt, t.node()->device_id)}, 3);
        };
        Tensor out = pad(*this).scaled_dot_product_attention(pad(key), pad(value), scale_val, is_causal, attn_mask, softcap);
        if (!out.valid()) return out;
        std::vector<int64_t> b0(4, 0), e0 = out.shape();
        e0[3] = head_dim;
        return out.try_shrink(b0, e0);
    }
    Tensor scores = matmul(key.try_transpose(-1, -2));
    scores = scores.try_mul(const_(scale_val, sdt, n_->device_id));
    if (is_causal) {
        const int64_t ql = n_->shape[nd - 2], kl = key.shape()[nd - 2];
        // tril(0) over a [Sq, Sk] mask of ones: key j visible iff j <= i (transformer.rs:103-109)
        auto iota = [&](int64_t axis) {
            auto n = mk(TKind::Iota, Scalar::Int32, {ql, kl}, {}, n_->device_id);
            n->arg = {axis};
            return Tensor(n);
        };
        Tensor mask = iota(1).binary(BinaryOp::Le, iota(0));
        scores = scores.where_(mask, const_(-INFINITY, sdt, n_->device_id));
    }
    if (attn_mask) {  // transformer.rs:112-125
        if (!attn_mask->valid()) return Tensor();
        if (attn_mask->dtype() == Scalar::Bool) {
            // true = attend: 0 where the mask holds, -inf elsewhere, added to the scores
            Tensor additive = const_(0.0, sdt, n_->device_id).where_(*attn_mask, const_(-INFINITY, sdt, n_->device_id));
            scores = scores.try_add(additive);
        } else {
            scores = scores.try_add(*attn_mask);
        }
    }
    if (softcap > 0.0) {  // transformer.rs:128-132
        Tensor cap = const_(softcap, sdt, n_->device_id);
        scores = scores.try_div(cap).tanh().try_mul(cap);
    }
    Tensor out = scores.softmax(-1).matmul(value);
    if (!out.valid()) return out;
    // the fused kernel takes a Bool or an additive mask of the scores' own dtype; any other mask
    // dtype changes the dtype of the scores themselves and stays the composed graph
    if (attn_mask && attn_mask->dtype() != Scalar::Bool && attn_mask->dtype() != sdt) return out;
    out.node()->hint = HintKind::Sdpa;
    out.node()->hint_inputs = {n_, key.node(), value.node()};
    if (attn_mask) out.node()->hint_inputs.push_back(attn_mask->node());
    out.node()->hint_scale = scale_val;
    out.node()->hint_causal = is_causal;
    out.node()->hint_softcap = softcap > 0.0 ? softcap : 0.0;
    return out;
}

// ============================================================================ scheduling
namespace {

// A coordinate while an expression is emitted: value = node + off.  `off` is a compile-time
// constant, which lets the V elements one work-item produces (UPCAST of the innermost axis,
// schedule/src/optimizer/heuristics.rs:37-82) share all index arithmetic and lets a load of
// V consecutive elements become one vector load.  `aligned`: node is a multiple of the
// upcast width and off lies in [0, width).  `mult`: a known divisor of node (0 = nothing known),
// which survives a reshape that splits the upcast axis (node / 2 is still a multiple of
// width / 2) and decides whether a narrower group of elements can still be one vector load.
struct Cx {
    uint32_t node = 0;
    int64_t off = 0;
    bool aligned = false;
    int64_t mult = 0;
    bool operator<(const Cx& o) const { return std::tie(node, off, aligned, mult) < std::tie(o.node, o.off, o.aligned, o.mult); }
};
using Coords = std::vector<Cx>;

// One kernel under construction: the builder plus the device buffers it reads (slot 1..),
// discovered while the expression is emitted.
struct KernelGen {
    KernelGen() { b.enable_cse(); }
    KernelBuilder b;
    Scalar idx_t = Scalar::Int32;
    int64_t width = 1;  // upcast width of the innermost output axis
    std::vector<std::shared_ptr<Buffer>> inputs;
    std::vector<uint32_t> input_params;
    std::vector<Scalar> input_dtypes;
    // Condition under which the value being emitted is used at all (-1: always): the parts of
    // a cat are selected by position, so the loads of a part are predicated on the position
    // falling into it and the lanes of the other parts issue no memory request.
    int64_t gate = -1;
    std::map<std::tuple<const TensorNode*, Coords, int64_t>, uint32_t> memo;  // (node, coordinates, gate) -> value
    std::map<std::tuple<uint32_t, uint32_t, int64_t, int64_t>, uint32_t> vec_loads;  // (param, base index, group, gate) -> vector value
    // A cat that the kernel splits at its root: instead of evaluating every part and selecting,
    // the kernel runs one guarded region per part and this cat forwards to the part picked
    // (pick_part >= 0), or only reports its coordinate along the cat axis (pick_part == -2).
    // Nodes whose value this kernel has computed itself and holds in a register, whatever the
    // coordinates (a row's reduction inside the kernel that also consumes it).
    std::map<const TensorNode*, uint32_t> fixed;
    // Flat upcast: when the kernel's output is walked as one flat run (its innermost axis does not
    // divide into whole upcast groups, its element count does), the materialised tensors of the
    // output's own shape that are reached through elementwise nodes only are read at the flat
    // index itself: flat_base (a multiple of the width) + flat_off, one vector load per group.
    std::set<const TensorNode*> flat_leaves;
    uint32_t flat_base = 0;
    int64_t flat_off = 0;
    const TensorNode* pick_cat = nullptr;
    int pick_part = -1;
    Cx probed_pos;
    bool probed = false;

    uint32_t ci(int64_t v) { return b.ci(v, idx_t); }
    uint32_t value(const Cx& c) { return c.off ? b.iadd(c.node, ci(c.off)) : c.node; }
    Cx zero() { return Cx{ci(0), 0, true}; }
    uint32_t buffer_param(const std::shared_ptr<Buffer>& buf, Scalar dt, int64_t numel) {
        for (size_t i = 0; i < inputs.size(); i++)
            if (inputs[i].get() == buf.get() && input_dtypes[i] == dt) return input_params[i];
        inputs.push_back(buf);
        input_dtypes.push_back(dt);
        input_params.push_back(b.param(static_cast<int>(inputs.size()), dt, numel));
        return input_params.back();
    }
};

// half types are evaluated in f32
Scalar compute_dtype(Scalar s) { return is_half(s) ? Scalar::Float32 : s; }

uint32_t flatten_nodes(KernelGen& g, const std::vector<uint32_t>& coords, const std::vector<int64_t>& shape) {
    uint32_t flat = g.ci(0);
    int64_t stride = 1;
    for (size_t i = shape.size(); i-- > 0;) {
        if (shape[i] != 1) flat = g.b.iadd(flat, g.b.imul(coords[i], stride));
        stride *= shape[i];
    }
    return flat;
}
std::vector<uint32_t> unflatten(KernelGen& g, uint32_t flat, const std::vector<int64_t>& shape) {
    std::vector<uint32_t> coords(shape.size());
    int64_t inner = 1;
    for (size_t i = shape.size(); i-- > 0;) {
        if (shape[i] == 1) {
            coords[i] = g.ci(0);
        } else {
            uint32_t q = g.b.idiv(flat, inner);
            // the outermost non-unit dimension needs no modulo
            bool outermost = true;
            for (size_t j = 0; j < i; j++) outermost = outermost && shape[j] == 1;
            coords[i] = outermost ? q : g.b.imod(q, shape[i]);
        }
        inner *= shape[i];
    }
    return coords;
}

int64_t gcd64(int64_t a, int64_t b) {
    while (b) {
        int64_t t = a % b;
        a = b;
        b = t;
    }
    return a;
}

// Row-major flat index of `coords` in `shape` as (node, constant offset).  `aligned` in the
// result: the node part is known to be a multiple of the upcast width and the offset lies
// inside one group, i.e. the elements off = 0..width-1 are consecutive in memory.
Cx flatten(KernelGen& g, const Coords& coords, const std::vector<int64_t>& shape) {
    std::vector<uint32_t> nodes(coords.size());
    int64_t off = 0, stride = 1;
    // what the flat node is known to be a multiple of: per axis, what its node is a multiple
    // of times the axis stride (a constant-zero node contributes nothing)
    const uint32_t zero = g.ci(0);
    int64_t mult = 0;
    for (size_t i = shape.size(); i-- > 0;) {
        nodes[i] = coords[i].node;
        if (shape[i] != 1) {
            off += coords[i].off * stride;
            if (coords[i].node != zero) {
                const int64_t m = coords[i].aligned ? std::max<int64_t>(g.width, coords[i].mult) : std::max<int64_t>(1, coords[i].mult);
                mult = gcd64(mult, m * stride);
            }
        }
        stride *= shape[i];
    }
    if (mult == 0) mult = int64_t{1} << 40;  // every node is the constant zero
    // the group of `width` elements starts on a multiple of the width and this element lies in it
    const bool aligned = g.width > 1 && !shape.empty() && mult % g.width == 0 && off >= 0 && off < g.width;
    return Cx{flatten_nodes(g, nodes, shape), off, aligned, mult};
}

// Coordinates in `shape` of flat = node + off, where node is a multiple of the upcast width W
// and 0 <= off < W, when the trailing dimensions split W evenly: dimensions whose extent
// times everything inside them divides W see only the constant part of the index, the one
// dimension that straddles W gets node-part + constant without carry (its extent must be a
// multiple of what is left of W), everything further out sees only the node.  False when
// the dimensions do not line up that way.
bool split_group(KernelGen& g, const Cx& flat, const std::vector<int64_t>& shape, Coords* out) {
    const int64_t W = g.width;
    if (W <= 1 || shape.empty()) return false;
    std::vector<uint32_t> u = unflatten(g, flat.node, shape);
    out->assign(shape.size(), Cx{});
    int64_t inner = 1;
    bool done = false;  // past the straddling dimension
    for (size_t i = shape.size(); i-- > 0;) {
        const int64_t d = shape[i];
        if (d == 1) {
            (*out)[i] = g.zero();
        } else if (done) {
            (*out)[i] = Cx{u[i], 0, false, 0};
        } else if (W % (inner * d) == 0) {
            (*out)[i] = Cx{g.ci(0), (flat.off / inner) % d, false, 0};  // the node part is a multiple of inner * d
            done = inner * d == W;
        } else {
            if (W % inner || d % (W / inner)) return false;
            (*out)[i] = Cx{u[i], flat.off / inner, false, W / inner};
            done = true;
        }
        inner *= d;
    }
    return true;
}

uint32_t emit(KernelGen& g, const TensorNode* n, const Coords& coords);

uint32_t emit_load(KernelGen& g, const TensorNode* n, const Coords& coords) {
    KernelBuilder& b = g.b;
    uint32_t p = g.buffer_param(n->buffer, n->dtype, n->numel());
    Cx flat = g.flat_base && g.flat_leaves.count(n) ? Cx{g.flat_base, g.flat_off, true, g.width} : flatten(g, coords, n->shape);
    const int64_t per_load = std::min<int64_t>(g.width, 16 / std::max<int64_t>(1, static_cast<int64_t>(scalar_size(n->dtype))));
    // a group of per_load consecutive elements that starts on a multiple of per_load (and so lies
    // inside a buffer of a multiple of per_load elements) is one vector load
    const bool narrow = per_load > 1 && flat.mult > 0 && flat.mult % per_load == 0 && flat.off >= 0;
    if ((flat.aligned || narrow) && per_load > 1 && n->numel() % per_load == 0 && n->dtype != Scalar::Bool) {
        // one vector load per group of `per_load` consecutive elements, shared by the group
        const int64_t group = flat.off / per_load;
        auto key = std::make_tuple(p, flat.node, group, g.gate);
        auto it = g.vec_loads.find(key);
        uint32_t vec;
        if (it != g.vec_loads.end()) {
            vec = it->second;
        } else {
            uint32_t at = group ? b.iadd(flat.node, g.ci(group * per_load)) : flat.node;
            uint32_t ix = g.gate >= 0 ? b.index_gated(p, at, static_cast<uint32_t>(g.gate)) : b.index(p, at);
            vec = b.load(ix, static_cast<int>(per_load));
            g.vec_loads[key] = vec;
        }
        return b.gep(vec, static_cast<int>(flat.off % per_load));
    }
    if (g.gate >= 0) return b.load(b.index_gated(p, g.value(flat), static_cast<uint32_t>(g.gate)));
    return b.load(b.index(p, g.value(flat)));
}

uint32_t emit_uncached(KernelGen& g, const TensorNode* n, const Coords& coords) {
    KernelBuilder& b = g.b;
    const Scalar ct = compute_dtype(n->dtype);
    if (n->buffer) {  // materialised tensor: a load from its row-major buffer
        uint32_t v = emit_load(g, n, coords);
        return ct != n->dtype ? b.cast(v, ct) : v;
    }
    switch (n->kind) {
        case TKind::Const:
            return is_float(ct) ? b.cf(n->cval, ct) : b.ci(static_cast<int64_t>(n->cval), ct);
        case TKind::Unary: {
            uint32_t x = emit(g, n->src[0].get(), coords);
            return b.unary(static_cast<UnaryOp>(n->sub), x);
        }
        case TKind::Binary: {
            uint32_t x = emit(g, n->src[0].get(), coords), y = emit(g, n->src[1].get(), coords);
            return b.binary(static_cast<BinaryOp>(n->sub), x, y);
        }
        case TKind::Where: {
            uint32_t c = emit(g, n->src[0].get(), coords), t = emit(g, n->src[1].get(), coords),
                     f = emit(g, n->src[2].get(), coords);
            return b.where(c, t, f);
        }
        case TKind::Cast: {
            uint32_t x = emit(g, n->src[0].get(), coords);
            const Scalar from = compute_dtype(n->src[0]->dtype);
            if (is_half(n->dtype)) {  // an explicit cast to a half type rounds here
                uint32_t r = b.dtype(x).scalar == n->dtype ? x : b.cast(x, n->dtype);
                return b.cast(r, Scalar::Float32);
            }
            return from == ct ? x : b.cast(x, ct);
        }
        case TKind::Contiguous: return emit(g, n->src[0].get(), coords);
        case TKind::Reshape: {
            const TensorNode* s = n->src[0].get();
            // same sequence of non-unit dims: coordinates carry over
            std::vector<size_t> a, c;
            for (size_t i = 0; i < n->shape.size(); i++)
                if (n->shape[i] != 1) a.push_back(i);
            for (size_t i = 0; i < s->shape.size(); i++)
                if (s->shape[i] != 1) c.push_back(i);
            bool same = a.size() == c.size();
            for (size_t i = 0; same && i < a.size(); i++) same = n->shape[a[i]] == s->shape[c[i]];
            Coords sc(s->shape.size());
            if (same) {
                for (size_t i = 0; i < sc.size(); i++) sc[i] = g.zero();
                for (size_t i = 0; i < a.size(); i++) sc[c[i]] = coords[a[i]];
            } else {
                Cx flat = flatten(g, coords, n->shape);
                if (flat.aligned && !s->shape.empty() && s->shape.back() % g.width == 0) {
                    // the whole group stays inside the innermost source dimension
                    std::vector<uint32_t> u = unflatten(g, flat.node, s->shape);
                    for (size_t i = 0; i < sc.size(); i++) sc[i] = Cx{u[i], 0, false};
                    sc.back() = Cx{u.back(), flat.off, true};
                } else if (flat.aligned && split_group(g, flat, s->shape, &sc)) {
                    // the group is spread over several trailing source dimensions
                } else {
                    std::vector<uint32_t> u = unflatten(g, g.value(flat), s->shape);
                    for (size_t i = 0; i < sc.size(); i++) sc[i] = Cx{u[i], 0, false};
                }
            }
            return emit(g, s, sc);
        }
        case TKind::Permute: {
            Coords sc(coords.size());
            for (size_t i = 0; i < coords.size(); i++) sc[n->arg[i]] = coords[i];
            return emit(g, n->src[0].get(), sc);
        }
        case TKind::Expand: {
            const TensorNode* s = n->src[0].get();
            Coords sc = coords;
            for (size_t i = 0; i < sc.size(); i++)
                if (s->shape[i] == 1 && n->shape[i] != 1) sc[i] = g.zero();
            return emit(g, s, sc);
        }
        case TKind::Shrink: {
            Coords sc = coords;
            for (size_t i = 0; i < sc.size(); i++) {
                if (!n->arg[i]) continue;
                if (sc[i].aligned && n->arg[i] % g.width == 0) sc[i].node = b.iadd(sc[i].node, g.ci(n->arg[i]));
                else sc[i].off += n->arg[i], sc[i].aligned = false;
            }
            return emit(g, n->src[0].get(), sc);
        }
        case TKind::Iota: {
            uint32_t c = g.value(coords[n->arg[0]]);
            return b.dtype(c).scalar == ct ? c : b.cast(c, ct);
        }
        case TKind::Cat: {
            const size_t axis = static_cast<size_t>(n->arg[0]);
            // every part is evaluated at a clamped coordinate; the right one is selected
            bool groups = coords[axis].aligned;  // a whole upcast group falls into one part
            for (const TensorRef& p : n->src) groups = groups && p->shape[axis] % g.width == 0;
            if (n->numel() == 0) return is_float(ct) ? b.cf(0.0, ct) : b.ci(0, ct);
            if (n == g.pick_cat && g.pick_part == -2) {
                g.probed_pos = coords[axis];
                g.probed = true;
                return is_float(ct) ? b.cf(0.0, ct) : b.ci(0, ct);
            }
            if (n == g.pick_cat && g.pick_part >= 0) {  // inside the guarded region of one part
                int64_t start = 0;
                for (int i = 0; i < g.pick_part; i++) start += n->src[i]->shape[axis];
                Coords sc = coords;
                sc[axis] = Cx{start ? b.iadd(coords[axis].node, g.ci(-start)) : coords[axis].node, coords[axis].off, coords[axis].aligned};
                return emit(g, n->src[g.pick_part].get(), sc);
            }
            if (!groups && coords[axis].node == g.ci(0)) {
                // the position along the cat axis is a compile-time constant: no selection at all
                int64_t start = 0;
                for (const TensorRef& p : n->src) {
                    const int64_t len = p->shape[axis];
                    if (coords[axis].off >= start && coords[axis].off < start + len) {
                        Coords sc = coords;
                        sc[axis] = Cx{g.ci(0), coords[axis].off - start, false, 0};
                        return emit(g, p.get(), sc);
                    }
                    start += len;
                }
            }
            const uint32_t pos = groups ? coords[axis].node : g.value(coords[axis]);
            const int64_t span = groups ? g.width : 1;
            int64_t start = 0;
            std::vector<uint32_t> vals;
            std::vector<int64_t> ends;
            for (const TensorRef& p : n->src) {
                const int64_t len = p->shape[axis];
                if (len == 0) continue;  // an empty part contributes no element (and has no valid coordinate)
                Coords sc = coords;
                uint32_t rel = b.iadd(pos, g.ci(-start));
                uint32_t lo = b.where(b.binary(BinaryOp::Lt, rel, g.ci(0)), g.ci(0), rel);
                uint32_t cl = b.where(b.binary(BinaryOp::Gt, lo, g.ci(len - span)), g.ci(len - span), lo);
                sc[axis] = groups ? Cx{cl, coords[axis].off, true} : Cx{cl, 0, false};
                // this part is live where start <= pos < start + len (and the enclosing gate holds)
                const int64_t outer = g.gate;
                uint32_t live = b.binary(BinaryOp::And, b.binary(BinaryOp::Ge, pos, g.ci(start)),
                                         b.binary(BinaryOp::Lt, pos, g.ci(start + len)));
                if (outer >= 0) live = b.binary(BinaryOp::And, static_cast<uint32_t>(outer), live);
                g.gate = live;
                vals.push_back(emit(g, p.get(), sc));
                g.gate = outer;
                start += len;
                ends.push_back(start);
            }
            uint32_t res = vals.back();
            for (size_t i = vals.size() - 1; i-- > 0;)
                res = b.where(b.binary(BinaryOp::Lt, pos, g.ci(ends[i])), vals[i], res);
            return res;
        }
        case TKind::Gather: {
            const TensorNode* w = n->src[0].get();
            Coords ic(coords.begin(), coords.end() - 1);
            uint32_t row = emit(g, n->src[1].get(), ic);
            if (b.dtype(row).scalar != g.idx_t) row = b.cast(row, g.idx_t);
            // An index outside [0, rows) selects nothing: the reference gathers through a
            // comparison against arange(rows) (tensor/src/transformer.rs:12-25), which yields
            // zeros there.  The row is clamped for the load and the value masked afterwards.
            const int64_t rows = w->shape[0];
            uint32_t below = b.binary(BinaryOp::Lt, row, g.ci(0)), above = b.binary(BinaryOp::Gt, row, g.ci(rows - 1));
            uint32_t clamped = b.where(below, g.ci(0), b.where(above, g.ci(rows - 1), row));
            uint32_t v = emit(g, w, {Cx{clamped, 0, false}, coords.back()});
            uint32_t zero = is_float(ct) ? b.cf(0.0, ct) : b.ci(0, ct);
            return b.where(b.binary(BinaryOp::Or, below, above), zero, v);
        }
        case TKind::Reduce:
        case TKind::Buffer: break;  // always materialised before being read
    }
    return 0;
}

uint32_t emit(KernelGen& g, const TensorNode* n, const Coords& coords) {
    auto fx = g.fixed.find(n);
    if (fx != g.fixed.end()) return fx->second;
    auto key = std::make_tuple(n, coords, g.gate);
    auto it = g.memo.find(key);
    if (it != g.memo.end()) return it->second;
    uint32_t v = emit_uncached(g, n, coords);
    g.memo[key] = v;
    return v;
}

Coords plain(const std::vector<uint32_t>& nodes) {
    Coords c(nodes.size());
    for (size_t i = 0; i < nodes.size(); i++) c[i] = Cx{nodes[i], 0, false};
    return c;
}

// ---- strided views.  A chain of movement ops over data in memory is an offset plus one
// stride per axis whenever no reshape in it splits or merges axes that are not contiguous
// with each other; the hand-written attention kernel reads and writes such views in place.
static std::vector<int64_t> dense_strides(const std::vector<int64_t>& shape) {
    std::vector<int64_t> st(shape.size(), 1);
    for (size_t i = shape.size(); i-- > 1;) st[i - 1] = st[i] * shape[i];
    return st;
}

// Strides of the same memory seen through `to` instead of `from` (equal element counts, no
// zero extents); false when the reshape would need a copy.
static bool reshape_strides(const std::vector<int64_t>& from, const std::vector<int64_t>& from_st, const std::vector<int64_t>& to,
                            std::vector<int64_t>* to_st) {
    std::vector<int64_t> od, os;  // extents of 1 carry no stride
    for (size_t i = 0; i < from.size(); i++)
        if (from[i] != 1) od.push_back(from[i]), os.push_back(from_st[i]);
    to_st->assign(to.size(), 0);
    size_t oi = 0, ni = 0;
    while (ni < to.size()) {
        if (to[ni] == 1) {
            ni++;
            continue;
        }
        if (oi >= od.size()) return false;
        // smallest groups of axes on both sides with equal products
        size_t oj = oi + 1, nj = ni + 1;
        int64_t op = od[oi], np = to[ni];
        while (op != np) {
            if (np < op) {
                if (nj >= to.size()) return false;
                np *= to[nj++];
            } else {
                if (oj >= od.size()) return false;
                op *= od[oj++];
            }
        }
        for (size_t k = oi; k + 1 < oj; k++)
            if (os[k] != od[k + 1] * os[k + 1]) return false;  // the old group is not one run of memory
        int64_t st = os[oj - 1];
        for (size_t k = nj; k-- > ni;) {
            (*to_st)[k] = to[k] == 1 ? 0 : st;
            st *= to[k];
        }
        oi = oj;
        ni = nj;
    }
    return oi == od.size();
}

struct StridedView {
    TensorNode* base = nullptr;  // in memory, or to be materialised
    int64_t offset = 0;          // elements
    std::vector<int64_t> strides;
};

static bool strided_view(TensorNode* n, StridedView* v) {
    const bool movement = n->kind == TKind::Reshape || n->kind == TKind::Permute || n->kind == TKind::Expand || n->kind == TKind::Shrink;
    // a node carrying a fused-kernel hint is a unit: its inner graph is not looked into
    if (n->buffer || !movement || n->hint != HintKind::None) {
        v->base = n;
        v->offset = 0;
        v->strides = dense_strides(n->shape);
        return true;
    }
    StridedView c;
    TensorNode* s = n->src[0].get();
    if (n->numel() == 0 || !strided_view(s, &c)) return false;
    v->base = c.base;
    v->offset = c.offset;
    v->strides.assign(n->shape.size(), 0);
    switch (n->kind) {
        case TKind::Permute:
            for (size_t i = 0; i < n->shape.size(); i++) v->strides[i] = c.strides[n->arg[i]];
            return true;
        case TKind::Expand:
            for (size_t i = 0; i < n->shape.size(); i++) v->strides[i] = s->shape[i] == n->shape[i] ? c.strides[i] : 0;
            return true;
        case TKind::Shrink:
            for (size_t i = 0; i < n->shape.size(); i++) {
                v->offset += n->arg[i] * c.strides[i];
                v->strides[i] = c.strides[i];
            }
            return true;
        default: return reshape_strides(s->shape, c.strides, n->shape, &v->strides);
    }
}

struct Scheduler {
    std::shared_ptr<Device> dev;
    std::unique_ptr<ExecutionPlan> plan;
    RealizeStats stats;
    std::vector<TensorNode*> produced;  // nodes this realization gave a buffer
    std::vector<TensorNode*> produced_host;  // CPU nodes this realization gave host memory (device -> CPU copies)
    std::unordered_map<const TensorNode*, int> uses;  // consumers of a node within the realised graph

    std::unordered_map<const TensorNode*, std::vector<TensorNode*>> matmul_readers;  // who reads each product node
    void count_uses(const TensorNode* root) {
        std::vector<const TensorNode*> stack{root};
        std::set<const TensorNode*> seen{root};
        while (!stack.empty()) {
            const TensorNode* n = stack.back();
            stack.pop_back();
            for (const TensorRef& c : n->src) {
                uses[c.get()]++;
                if (c->hint == HintKind::Matmul) matmul_readers[c.get()].push_back(const_cast<TensorNode*>(n));
                if (seen.insert(c.get()).second) stack.push_back(c.get());
            }
        }
    }

    int add_kernel(const std::shared_ptr<CachedKernel>& k, const std::vector<std::shared_ptr<Buffer>>& bufs, bool cached) {
        std::vector<size_t> idx;
        for (auto& bptr : bufs) idx.push_back(plan->add_buffer(bptr));
        MRK_TRY(plan->add_kernel(k, idx, {}));
        stats.kernel_names.push_back(k->entry_point);
        stats.kernel_sources.push_back(k->code);
        if (cached) stats.cached_kernels++;
        return kOk;
    }
    std::shared_ptr<Buffer> new_buffer(const TensorNode* n) {
        BufferOptions o;
        size_t bytes = static_cast<size_t>(n->numel()) * scalar_size(n->dtype);
        return std::make_shared<Buffer>(dev->allocator, bytes ? bytes : 1, o);
    }
    // Kernels this schedule needs that the cache does not hold yet.  With `deferred` set they are
    // not compiled here (the caller holds the graph lock): the schedule goes on with a placeholder
    // and is thrown away, the caller compiles them with the lock released and schedules again.
    // `fresh` names the kernels compiled that way, so that the second pass still reports them as
    // newly compiled.
    struct PendingKernel {
        LinearKernel k;
        std::string name;
    };
    std::vector<PendingKernel>* deferred = nullptr;
    const std::set<uint64_t>* fresh = nullptr;
    int compile_kernel(const LinearKernel& k, const char* name, std::shared_ptr<CachedKernel>* ck, bool* cached) {
        if (deferred && !lookup_linear_kernel(*dev, k, ck)) {
            deferred->push_back({k, name});
            *ck = std::make_shared<CachedKernel>();
            (*ck)->entry_point = name;
            *cached = false;
            return kOk;
        }
        MRK_TRY(get_or_compile_linear_kernel(*dev, k, name, ck, cached));
        if (fresh && fresh->count(k.content_hash)) *cached = false;
        return kOk;
    }
    int builtin(const char* kind, const std::vector<int64_t>& params, const std::vector<std::shared_ptr<Buffer>>& bufs) {
        std::string key = std::string("builtin:") + kind;
        for (int64_t p : params) key += ":" + std::to_string(p);
        const std::string device = "HIP:" + std::to_string(dev->device_id);
        std::shared_ptr<CachedKernel> ck;
        bool cached = false;
        MRK_TRY(KernelCache::global().get_or_compile(
            fnv1a64(reinterpret_cast<const uint8_t*>(key.data()), key.size()), device,
            [&](std::shared_ptr<CachedKernel>* fresh) -> int {
                std::unique_ptr<Program> p;
                MRK_TRY(create_builtin_program(dev->device_id, dev->allocator->stream(), kind, params.data(), params.size(), &p));
                auto k = std::make_shared<CachedKernel>();
                k->entry_point = p->name();
                k->program = std::move(p);
                k->device = device;
                *fresh = std::move(k);
                return kOk;
            },
            &ck, &cached));
        return add_kernel(ck, bufs, cached);
    }

    // nodes that must exist in memory before the kernel rooted at `root` can read them
    void boundaries(const TensorNode* n, const TensorNode* root, std::set<const TensorNode*>& seen,
                    std::vector<TensorNode*>& out, int64_t* max_numel) {
        if (!seen.insert(n).second) return;
        *max_numel = std::max(*max_numel, n->numel());
        if (n->buffer) return;
        TensorNode* other = nullptr;
        if (n != root && !side_inline.count(n) &&
            (is_boundary_kind(n) || fusable(n) || generated_tc(n) || residual_matmul(const_cast<TensorNode*>(n), &other) || swiglu_matmul(n))) {
            out.push_back(const_cast<TensorNode*>(n));
            return;
        }
        for (const TensorRef& s : n->src) boundaries(s.get(), root, seen, out, max_numel);
    }
    // Tensors the row-resident kernel being generated computes in passing and also writes out
    // (its side outputs): boundaries() looks through them, emit() evaluates them in place.
    std::set<const TensorNode*> side_inline;

    // An input of a row-resident kernel rooted at `n` that this kernel can produce itself: an
    // elementwise expression the caller wants in memory (`contiguous()`) that nobody has computed
    // yet, of the kernel's own shape and element size, so that every work-item holds exactly the
    // elements it would otherwise load (an embedding lookup in front of the first normalisation
    // of a decoder block: the looked-up rows are written for the residual and normalised without
    // being read back).  Anything with a kernel of its own kind (a product, an attention, a copy
    // between devices, a reshape of data in memory) keeps it.
    bool side_output_candidate(const TensorNode* d, const TensorNode* n) {
        if (d->buffer || d->kind != TKind::Contiguous || d->hint != HintKind::None || d->shape != n->shape || d->numel() == 0) return false;
        if (d->dtype == Scalar::Bool || scalar_size(d->dtype) != scalar_size(n->dtype)) return false;
        const TensorNode* s = d->src[0].get();
        TensorNode* other = nullptr;
        if (s->buffer || is_boundary_kind(s) || fusable(s) || generated_tc(s) || residual_matmul(const_cast<TensorNode*>(s), &other) || swiglu_matmul(s)) return false;
        {
            TensorNode* rest = nullptr;
            int64_t split = 0, seq = 0;
            std::vector<int64_t> out_strides;
            if (rope_matmul(const_cast<TensorNode*>(d), &rest, &split, &seq) || attention_under(const_cast<TensorNode*>(d), &out_strides)) return false;
        }
        // no reduction of the row's own may hide under it (it would have to be fused as well)
        std::set<const TensorNode*> seen;
        std::vector<TensorNode*> deps;
        int64_t ignore = 0;
        boundaries(d, d, seen, deps, &ignore);
        for (const TensorNode* x : deps)
            if (!x->buffer && x->kind == TKind::Reduce) return false;
        return true;
    }

    bool fusable(const TensorNode* n) const {
        if (!g_fusion || n->hint == HintKind::None) return false;
        switch (n->hint) {
            case HintKind::Swish: return false;  // no kernel of its own: only matched as part of swiglu_matmul
            case HintKind::Rope: return false;   // likewise: only matched as the epilogue of a packed projection (rope_matmul)
            case HintKind::Softmax:
                return n->dtype == Scalar::Float32 && !n->shape.empty() &&
                       n->arg[0] == static_cast<int64_t>(n->shape.size()) - 1 && n->numel() > 0;
            case HintKind::Matmul: {
                const TensorNode *a = n->hint_inputs[0].get(), *w = n->hint_inputs[1].get();
                if (a->dtype != w->dtype) return false;
                if (a->dtype == Scalar::BFloat16 || a->dtype == Scalar::Float16) {  // the hand-written 16-bit products
                    // [..., M, K] x [K, N] is one product over the flattened leading axes;
                    // equal leading axes on both sides are that many products in one launch
                    if (n->dtype != a->dtype || n->numel() == 0 || a->shape.size() < 2) return false;
                    if (w->shape.size() == 2) return true;
                    if (w->shape.size() != a->shape.size()) return false;
                    int64_t batch = 1;
                    for (size_t i = 0; i + 2 < a->shape.size(); i++) {
                        if (a->shape[i] != w->shape[i]) return false;
                        batch *= a->shape[i];
                    }
                    return batch <= 65535;
                }
                if (a->shape.size() != 2 || w->shape.size() != 2) return false;
                if (a->dtype == Scalar::Float32)
                    return a->shape[0] % 64 == 0 && w->shape[1] % 64 == 0 && a->shape[0] > 0 && w->shape[1] > 0;
                return false;
            }
            case HintKind::Sdpa: {
                const TensorNode* q = n->hint_inputs[0].get();
                const TensorNode* k = n->hint_inputs[1].get();
                const TensorNode* v = n->hint_inputs[2].get();
                if (!(q->dtype == Scalar::BFloat16 && k->dtype == q->dtype && v->dtype == q->dtype &&
                      q->shape.size() == 4 && (q->shape[3] == 256 || q->shape[3] == 128 || q->shape[3] == 64) && v->shape[3] == q->shape[3] && k->shape[2] > 0 &&
                      k->shape[0] == q->shape[0] && k->shape[1] == q->shape[1] && q->numel() > 0))
                    return false;
                if (n->hint_inputs.size() > 3) {
                    // attn_mask inside the kernel: Bool or bf16, broadcastable to [B, H, Sq, Sk] with the
                    // key axis in full, read in groups of four keys
                    const TensorNode* m = n->hint_inputs[3].get();
                    const int64_t full[4] = {q->shape[0], q->shape[1], q->shape[2], k->shape[2]};
                    if ((m->dtype != Scalar::Bool && m->dtype != Scalar::BFloat16) || m->shape.empty() || m->shape.size() > 4 ||
                        m->shape.back() != full[3] || full[3] % 4)
                        return false;
                    for (size_t i = 0; i < m->shape.size(); i++) {
                        const int64_t want = full[4 - m->shape.size() + i];
                        if (m->shape[i] != want && m->shape[i] != 1) return false;
                    }
                }
                return true;
            }
            default: return false;
        }
    }

    // With the hand-written kernels switched off, a bf16 matmul whose shape fits still takes the
    // tensor-core route of the optimizer (schedule/src/optimizer/tc.rs:36-94): the generated
    // WMMA kernel staged through local memory instead of the generic reduce kernel.
    // The fixed heuristic for the register-staged variant (any shape whose N and K are multiples
    // of 8): the largest of a few workgroup tiles that gives every CU a workgroup
    // (16 waves on 256 x 256 measured 1.05 PF at 4096^3 against 0.74 for 4 waves on 128 x 128)
    // and pads the output by at most an eighth; a shape too small for that takes the tile with
    // the least padding, the smaller one among equals.  MOROK_BEAM searches the whole space.
    static bool default_tc_opts(const TensorCore& tc, int64_t M, int64_t N, int64_t K, WmmaLdsOpts* o) {
        // shapes that whole tiles and 64-deep K steps divide take the variant with direct
        // global -> local copies (faster at every shape measured: 4096^3 1.26 against 1.08 PF,
        // 2048^3 0.76 against 0.49, 1024^3 0.30 against 0.23): the largest tile that still fills
        // the chip (one 256 x 256 workgroup or two smaller ones per CU), else the smallest
        static const int direct[][5] = {{2, 2, 8, 8, 256}, {2, 4, 8, 4, 256}, {2, 2, 4, 4, 512}, {2, 2, 4, 2, 512}, {2, 2, 2, 2, 0}};
        for (auto& c : direct) {
            // (stages = 3, a third stage of the second operand with the copies spread over the whole step,
            // measured the same or 1 % slower at 4096^3: the beam search tries it, the heuristic does not)
            WmmaLdsOpts t{c[0], c[1], c[2], c[3], 0, 2};
            if (!wmma_lds_opts_valid(tc, t, M, N, K)) continue;
            int bm, bn, bk;
            wmma_lds_tile(tc, t, K, &bm, &bn, &bk);
            if ((M / bm) * (N / bn) >= c[4]) {
                *o = t;
                return true;
            }
        }
        static const int choices[][4] = {{4, 4, 4, 4}, {2, 2, 4, 4}, {2, 2, 2, 2}, {2, 2, 1, 1}, {1, 1, 1, 1}};
        bool found = false;
        int64_t least = 0;
        for (auto& c : choices) {
            WmmaLdsOpts t{c[0], c[1], c[2], c[3], 0};
            if (!wmma_lds_opts_valid(tc, t, M, N, K)) continue;
            int bm, bn, bk;
            wmma_lds_tile(tc, t, K, &bm, &bn, &bk);
            const int64_t tm = (M + bm - 1) / bm, tn = (N + bn - 1) / bn, padded = tm * bm * tn * bn;
            if (padded * 8 <= M * N * 9 && tm * tn >= 256) {
                *o = t;
                return true;
            }
            if (!found || padded <= least) {
                *o = t;
                least = padded;
                found = true;
            }
        }
        return found;
    }
    bool generated_tc(const TensorNode* n) const {
        if (n->hint != HintKind::Matmul || n->numel() == 0) return false;
        const TensorNode *a = n->hint_inputs[0].get(), *w = n->hint_inputs[1].get();
        const Scalar dt = n->dtype;
        // both 16-bit float types have hand-written kernels, taken while those are switched on
        if ((dt != Scalar::BFloat16 && dt != Scalar::Float16) || g_fusion) return false;
        if (a->dtype != dt || w->dtype != dt) return false;
        if (a->shape.size() != 2 || w->shape.size() != 2) return false;
        const auto tcs = cdna4_tensor_cores();
        const int tc = select_tensor_core(tcs, dt, dt, Scalar::Float32);
        WmmaLdsOpts o;
        return tc >= 0 && default_tc_opts(tcs[tc], a->shape[0], w->shape[1], a->shape[1], &o);
    }
    int materialize_generated_tc(TensorNode* n) {
        for (const TensorRef& in : n->hint_inputs) MRK_TRY(materialize(in.get()));
        const TensorNode *a = n->hint_inputs[0].get(), *w = n->hint_inputs[1].get();
        const int64_t M = a->shape[0], K = a->shape[1], N = w->shape[1];
        const auto tcs = cdna4_tensor_cores();
        const int tc = select_tensor_core(tcs, n->dtype, n->dtype, Scalar::Float32);
        if (tc < 0) return fail(kRuntime, "no tensor core for this dtype in the CDNA table");
        WmmaLdsOpts opts;
        if (!default_tc_opts(tcs[tc], M, N, K, &opts)) return fail(kRuntime, "tensor-core matmul: no workgroup tile divides the shape");
        int beam = 0;
        if (const char* e = std::getenv("MOROK_BEAM")) beam = std::atoi(e);
        if (beam > 0) MRK_TRY(beam_search_wmma_matmul(*dev, tcs[tc], tc, M, N, K, beam, &opts, nullptr, nullptr, nullptr));
        LinearKernel k;
        MRK_TRY(build_wmma_matmul_lds_kernel(tcs[tc], M, N, K, n->dtype, opts, &k));
        std::shared_ptr<CachedKernel> ck;
        bool cached = false;
        const std::string name = "r_tc_" + std::to_string(M) + "_" + std::to_string(N) + "_" + std::to_string(K);
        MRK_TRY(compile_kernel(k, name.c_str(), &ck, &cached));
        auto out = new_buffer(n);
        MRK_TRY(add_kernel(ck, {out, a->buffer, w->buffer}, cached));
        n->buffer = out;
        produced.push_back(n);
        return kOk;
    }

    // A product with so few rows that it is not run as one pass of output tiles: the K loop spread over the chip
    // (scratch and a second kernel), or the weight streamed for a handful of rows.  The tiled kernels' fused
    // epilogues would hold such a product on the few workgroups its tiles make (measured at 4 x 22016 x 4096 with
    // the gate: 70 us against 30 us for the streamed product plus an elementwise kernel), so they are not matched.
    bool spread_or_streamed(const TensorNode* mm, int64_t M, int64_t N, int64_t K, int64_t batch) const {
        long splits = 0, per = 0;
        if (gemm_bf16_workspace_bytes(M, N, K, batch) || gemm_kn_rows_plan(M, N, K, batch, &splits, &per)) return true;
        return transposed_weight(mm) && (gemm_nt_skinny_supported(M, N, K, batch) || gemm_nt_rows_supported(M, N, K, batch));
    }
    // x + (a @ w) in bf16 where nothing else reads the product: the product kernel adds x in its
    // epilogue (same bits as the product followed by the add).  Returns the product node and the
    // other operand.
    TensorNode* residual_matmul(TensorNode* n, TensorNode** other, bool* is_row = nullptr) const {
        if (is_row) *is_row = false;
        if (!g_fusion || n->kind != TKind::Binary || static_cast<BinaryOp>(n->sub) != BinaryOp::Add || n->dtype != Scalar::BFloat16 ||
            n->numel() == 0 || n->src.size() != 2)
            return nullptr;
        for (int side = 0; side < 2; side++) {
            TensorNode* mm = n->src[side].get();
            TensorNode* r = n->src[1 - side].get();
            if (mm->buffer || mm->hint != HintKind::Matmul || !fusable(mm) || mm->dtype != Scalar::BFloat16) continue;
            auto u = uses.find(mm);
            if (u == uses.end() || u->second != 1) continue;
            if (r->dtype != Scalar::BFloat16 || r->shape != n->shape || mm->shape != n->shape) continue;
            int64_t M, N, K, batch;
            matmul_extents(mm, &M, &N, &K, &batch);
            // a bias (x @ w + b, tensor/src/nn/linear.rs:39-41): one row [N] that is in memory, broadcast over the
            // rows (reshape to [1, .., 1, N], expand); the kernel adds it with a row pitch of zero
            // (with a single row the expand is the identity and there is no such node)
            if (!r->buffer && (r->kind == TKind::Expand || (M * batch == 1 && r->kind == TKind::Reshape))) {
                TensorNode* b = r->kind == TKind::Expand ? r->src[0].get() : r;
                while (!b->buffer && b->kind == TKind::Reshape) b = b->src[0].get();
                if (!b->buffer || b->dtype != Scalar::BFloat16 || b->numel() != N || n->shape.back() != N || b->buffer->offset() % 16) continue;
                if (!gemm_bf16_bias_supported(M, N, K, batch, transposed_weight(mm) != nullptr)) continue;
                *other = b;
                if (is_row) *is_row = true;
                return mm;
            }
            // only an operand that is in memory anyway: a lazy expression (x * 2)
            // is cheaper evaluated inside the add than written out first
            const TensorNode* rb = r;
            while (!rb->buffer && rb->kind == TKind::Reshape) rb = rb->src[0].get();
            if (!(rb->buffer || is_boundary_kind(rb) || fusable(rb))) continue;
            // (whichever kernel writes the product adds the operand: a tiled kernel's epilogue, the sum of a product spread
            // along K, a streaming kernel for a handful of rows)
            if (!gemm_bf16_bias_supported(M, N, K, batch, transposed_weight(mm) != nullptr)) continue;
            *other = r;
            return mm;
        }
        return nullptr;
    }
    // silu(p[:, :F]) * p[:, F:] in bf16 over one packed product p = a @ [Wg | Wu] that nothing else
    // reads: the product kernel applies the gate in its epilogue and writes [M, F] directly.
    // Returns the product node.
    TensorNode* swiglu_matmul(const TensorNode* n) const {
        if (!g_fusion || n->kind != TKind::Binary || static_cast<BinaryOp>(n->sub) != BinaryOp::Mul || n->dtype != Scalar::BFloat16 ||
            n->numel() == 0 || n->src.size() != 2 || n->shape.size() != 2)
            return nullptr;
        for (int side = 0; side < 2; side++) {
            const TensorNode* sw = n->src[side].get();
            const TensorNode* up = n->src[1 - side].get();
            if (sw->buffer || sw->hint != HintKind::Swish || sw->hint_inputs.size() != 1) continue;
            const TensorNode* gate = sw->hint_inputs[0].get();
            if (gate->buffer || up->buffer || gate->kind != TKind::Shrink || up->kind != TKind::Shrink) continue;
            TensorNode* mm = gate->src[0].get();
            if (up->src[0].get() != mm || mm->buffer || mm->hint != HintKind::Matmul || !fusable(mm) || mm->dtype != Scalar::BFloat16) continue;
            if (mm->shape.size() != 2 || mm->hint_inputs[1]->shape.size() != 2) continue;
            const int64_t M = mm->shape[0], F = n->shape[1];
            if (mm->shape[1] != 2 * F || n->shape[0] != M || gate->shape != n->shape || up->shape != n->shape) continue;
            if (gate->arg.size() != 2 || up->arg.size() != 2 || gate->arg[0] != 0 || gate->arg[1] != 0 || up->arg[0] != 0 || up->arg[1] != F) continue;
            // nobody else may read the packed product, its halves or the gate's activation
            auto used = [&](const TensorNode* t, int times) {
                auto u = uses.find(t);
                return u != uses.end() && u->second == times;
            };
            if (!used(mm, 2) || !used(gate, 2) || !used(up, 1) || !used(sw, 1)) continue;
            int64_t Mx, N2, K, batch;
            matmul_extents(mm, &Mx, &N2, &K, &batch);
            if (batch != 1 || Mx != M || N2 != 2 * F || !gemm_bf16_swiglu_supported(M, F, K)) continue;
            // (a handful of rows against a [2F, K] weight: the streaming kernel has a gated form of its own)
            if (spread_or_streamed(mm, M, N2, K, 1) && !(transposed_weight(mm) && gemm_nt_swiglu_streamed(M, F, K))) continue;
            return mm;
        }
        return nullptr;
    }
    // The second operand of a bf16 product given as the transpose of data that is in memory anyway
    // (x @ w.T with w [N, K]: how a Linear layer multiplies, tensor/src/nn/linear.rs:39-41): the
    // [N, K] node, which the "_nt" product kernels read in place; nullptr otherwise.
    TensorNode* transposed_weight(const TensorNode* mm) const {
        if (!g_fusion) return nullptr;
        TensorNode* w = mm->hint_inputs[1].get();
        if (w->buffer || w->kind != TKind::Permute || (w->dtype != Scalar::BFloat16 && w->dtype != Scalar::Float16) || w->shape.size() != 2 ||
            w->arg.size() != 2 ||
            w->arg[0] != 1 || w->arg[1] != 0)
            return nullptr;
        TensorNode* wt = w->src[0].get();
        const TensorNode* rb = wt;
        while (!rb->buffer && rb->kind == TKind::Reshape) rb = rb->src[0].get();
        return rb->buffer || is_boundary_kind(rb) || fusable(rb) ? wt : nullptr;
    }
    // Materialises a product's second operand and tells the layout the kernel will read it in:
    // [K, N], or (where nt_ok says the shape has a kernel for it) the [N, K] data behind a transpose.
    int weight_operand(TensorNode* mm, bool nt_ok, std::shared_ptr<Buffer>* buf, bool* nt) {
        *nt = false;
        // the B^T kernels have no any-alignment fallback: the first operand (materialised by the
        // caller; the output is always a fresh buffer) must start on a 16-byte boundary as well
        const std::shared_ptr<Buffer>& ab = mm->hint_inputs[0]->buffer;
        TensorNode* wt = nt_ok && ab && ab->offset() % 16 == 0 ? transposed_weight(mm) : nullptr;
        if (wt) {
            MRK_TRY(materialize(wt));
            if (wt->buffer->offset() % 16 == 0) {
                *buf = wt->buffer;
                *nt = true;
                return kOk;
            }
        }
        TensorNode* w = mm->hint_inputs[1].get();
        MRK_TRY(materialize(w));
        *buf = w->buffer;
        return kOk;
    }
    int materialize_swiglu_matmul(TensorNode* n, TensorNode* mm) {
        int64_t M, N2, K, batch;
        matmul_extents(mm, &M, &N2, &K, &batch);
        MRK_TRY(materialize(mm->hint_inputs[0].get()));
        std::shared_ptr<Buffer> wbuf;
        bool nt = false;
        MRK_TRY(weight_operand(mm, gemm_bf16_swiglu_supported(M, N2 / 2, K, true), &wbuf, &nt));
        auto out = new_buffer(n);
        MRK_TRY(builtin(nt ? "gemm_bf16_nt_swiglu" : "gemm_bf16_swiglu", {M, N2 / 2, K}, {out, mm->hint_inputs[0]->buffer, wbuf}));
        n->buffer = out;
        produced.push_back(n);
        return kOk;
    }
    static void matmul_extents(const TensorNode* mm, int64_t* M, int64_t* N, int64_t* K, int64_t* batch) {
        const TensorNode *a = mm->hint_inputs[0].get(), *w = mm->hint_inputs[1].get();
        *K = a->shape.back();
        *N = w->shape.back();
        *M = a->shape[a->shape.size() - 2];
        *batch = 1;
        for (size_t i = 0; i + 2 < a->shape.size(); i++) (w->shape.size() == 2 ? *M : *batch) *= a->shape[i];
    }
    int materialize_residual_matmul(TensorNode* n, TensorNode* mm, TensorNode* r, bool is_row) {
        int64_t M, N, K, batch;
        matmul_extents(mm, &M, &N, &K, &batch);
        MRK_TRY(materialize(mm->hint_inputs[0].get()));
        std::shared_ptr<Buffer> wbuf;
        bool nt = false;
        MRK_TRY(weight_operand(mm, true, &wbuf, &nt));  // (the residual epilogue exists for exactly the shapes the B^T kernels take)
        MRK_TRY(materialize(r));
        auto out = new_buffer(n);
        const std::string kind = std::string(nt ? "gemm_bf16_nt_" : "gemm_bf16_") + (is_row ? "bias" : "residual");
        // few output tiles against a long K: scratch for the partial results, an intermediate of the plan like any other
        const size_t ws = nt ? gemm_bf16_nt_workspace_bytes(M, N, K, batch) : gemm_bf16_workspace_bytes(M, N, K, batch);
        if (ws) {
            auto scratch = std::make_shared<Buffer>(dev->allocator, ws, BufferOptions());
            MRK_TRY(builtin(kind.c_str(), {M, N, K, batch, static_cast<int64_t>(ws)}, {out, mm->hint_inputs[0]->buffer, wbuf, r->buffer, scratch}));
        } else {
            const std::vector<int64_t> params = batch == 1 ? std::vector<int64_t>{M, N, K} : std::vector<int64_t>{M, N, K, batch};
            MRK_TRY(builtin(kind.c_str(), params, {out, mm->hint_inputs[0]->buffer, wbuf, r->buffer}));
        }
        n->buffer = out;
        produced.push_back(n);
        return kOk;
    }

    // Everything a realization computes runs on a HIP device.  Host-resident data may enter a
    // graph only through a COPY node (Tensor::to), and a copy back to the CPU only as the root.
    int check_placement(const TensorNode* root) {
        if (root->device_id == kCpuDevice && root->kind != TKind::Copy)
            return fail(kUnsupportedDevice, "this backend computes on HIP devices only: the tensor lives on the CPU device; "
                                            "move its inputs with to(\"HIP:0\") first");
        std::vector<const TensorNode*> stack{root};
        std::set<const TensorNode*> seen{root};
        while (!stack.empty()) {
            const TensorNode* n = stack.back();
            stack.pop_back();
            if (n->buffer) continue;
            if (n->kind == TKind::Copy && n->device_id != kCpuDevice) continue;  // checked when it is materialised
            if (n->kind == TKind::Copy && n != root)
                return fail(kUnsupportedDevice, "a copy to the CPU device can only be the last step of a realization");
            if (n->kind == TKind::Buffer && n->host)
                return fail(kUnsupportedDevice, "an operand lives on the CPU device: move it with to(\"HIP:0\") before computing "
                                                "with it (this backend does not compute on the CPU)");
            for (const TensorRef& c : n->src)
                if (seen.insert(c.get()).second) stack.push_back(c.get());
        }
        return kOk;
    }

    int add_copy_item(bool to_device, std::shared_ptr<std::vector<uint8_t>> host, const std::shared_ptr<Buffer>& device_side) {
        std::unique_ptr<Program> p;
        MRK_TRY(create_copy_program(dev->device_id, dev->allocator->stream(), to_device, std::move(host), &p));
        auto k = std::make_shared<CachedKernel>();
        k->entry_point = p->name();
        k->program = std::move(p);
        k->device = "HIP:" + std::to_string(dev->device_id);
        return add_kernel(k, {device_side}, false);
    }

    // COPY nodes become copy items of the plan, executed in order with its kernels
    // (tensor/src/realize.rs:1002-1011): nothing is transferred while scheduling.
    int materialize_copy(TensorNode* n) {
        TensorNode* s = n->src[0].get();
        const size_t bytes = static_cast<size_t>(n->numel()) * scalar_size(n->dtype);
        if (n->device_id == kCpuDevice) {  // device -> CPU
            if (s->device_id == kCpuDevice) return fail(kRuntime, "runtime error: copy between two CPU tensors");
            MRK_TRY(materialize(s));
            auto host = std::make_shared<std::vector<uint8_t>>(bytes);
            if (bytes) MRK_TRY(add_copy_item(false, host, s->buffer));
            n->host = host;
            n->host_from = dev->device_id;
            produced_host.push_back(n);
            return kOk;
        }
        if (s->device_id != kCpuDevice)
            return failf(kCopyFailed, "copy operation failed: cross-device copy %s -> %s is not supported", device_name(s->device_id).c_str(),
                         device_name(n->device_id).c_str());
        // CPU -> device: the source must be stored bytes (a reshape of stored bytes is the same bytes)
        const TensorNode* h = s;
        while (!h->host && h->kind == TKind::Reshape) h = h->src[0].get();
        if (!h->host)
            return fail(kUnsupportedDevice, "to(): the source is an unrealised expression on the CPU device; this backend does not "
                                            "compute on the CPU - move the stored operands to the device first and compute there");
        if (h->host_from != kCpuDevice) {  // bytes that a device is still writing (an earlier copy to the CPU)
            std::shared_ptr<Allocator> a;
            MRK_TRY(AllocatorRegistry::global().get(h->host_from, &a));
            MRK_TRY(a->synchronize());
        }
        auto out = new_buffer(n);
        if (bytes) MRK_TRY(add_copy_item(true, h->host, out));
        n->buffer = out;
        produced.push_back(n);
        return kOk;
    }

    // contiguous(cast_bf16(apply_rotary_emb(reshape(p[:, :split], [B, S, heads, 128]), cos, sin))) over a packed
    // bf16 projection p = a @ w whose only other reader is the slice p[:, split:] (q | k and v of a fused
    // QKV product): the product kernel rotates the heads in its epilogue and writes the two parts to
    // buffers of their own, so the packed product is never written and read again.  Returns the
    // product node and the node of the unrotated slice (nullptr when split == N).
    TensorNode* rope_matmul(TensorNode* n, TensorNode** rest, int64_t* split_out, int64_t* seq_out) const {
        if (!g_fusion || n->kind != TKind::Contiguous || n->dtype != Scalar::BFloat16 || n->numel() == 0) return nullptr;
        auto used_once = [&](const TensorNode* t) {
            auto u = uses.find(t);
            return u != uses.end() && u->second == 1;
        };
        const TensorNode* c = n->src[0].get();
        if (c->buffer || c->kind != TKind::Cast || !used_once(c)) return nullptr;
        const TensorNode* rp = c->src[0].get();
        if (rp->buffer || rp->hint != HintKind::Rope || rp->hint_inputs.size() != 3 || !used_once(rp)) return nullptr;
        const TensorNode* x = rp->hint_inputs[0].get();  // [B, S, heads, 128], read by the two half slices only
        const TensorNode *cs = rp->hint_inputs[1].get(), *sn = rp->hint_inputs[2].get();
        if (x->buffer || x->kind != TKind::Reshape || x->shape.size() != 4 || x->shape[3] != 128 || x->dtype != Scalar::BFloat16) return nullptr;
        auto ux = uses.find(x);
        if (ux == uses.end() || ux->second != 2) return nullptr;
        const int64_t S = x->shape[1];
        for (const TensorNode* t : {cs, sn})  // tables [1, S, 1, 64] f32, in memory
            if (!t->buffer || t->dtype != Scalar::Float32 || t->shape != std::vector<int64_t>{1, S, 1, 64} || t->buffer->offset() % 32) return nullptr;
        const TensorNode* sl = x->src[0].get();  // p[:, :split]
        if (sl->buffer || sl->kind != TKind::Shrink || !used_once(sl) || sl->shape.size() != 2) return nullptr;
        TensorNode* mm = sl->src[0].get();
        if (mm->buffer || mm->hint != HintKind::Matmul || !fusable(mm) || mm->dtype != Scalar::BFloat16 || mm->shape.size() != 2) return nullptr;
        if (mm->hint_inputs[0]->shape.size() != 2 || mm->hint_inputs[1]->shape.size() != 2) return nullptr;
        const int64_t M = mm->shape[0], N = mm->shape[1], K = mm->hint_inputs[0]->shape[1], split = sl->shape[1];
        if (sl->shape[0] != M || sl->arg.size() != 2 || sl->arg[0] != 0 || sl->arg[1] != 0) return nullptr;
        if (x->shape[0] * S != M || x->shape[2] * 128 != split || !gemm_bf16_rope_supported(M, N, K, split, S) || spread_or_streamed(mm, M, N, K, 1))
            return nullptr;
        // the product's readers: this slice and, when there are columns left, exactly the slice of all of them
        auto readers = matmul_readers.find(mm);
        if (readers == matmul_readers.end()) return nullptr;
        TensorNode* other = nullptr;
        for (TensorNode* r : readers->second)
            if (r != sl) {
                if (other && other != r) return nullptr;
                other = r;
            }
        if (split == N) {
            if (other) return nullptr;
        } else {
            if (!other || other->buffer || other->kind != TKind::Shrink || other->shape != std::vector<int64_t>{M, N - split} || other->arg.size() != 2 ||
                other->arg[0] != 0 || other->arg[1] != split)
                return nullptr;
        }
        *rest = other;
        *split_out = split;
        *seq_out = S;
        return mm;
    }
    int materialize_rope_matmul(TensorNode* n, TensorNode* mm, TensorNode* rest, int64_t split, int64_t seq) {
        const TensorNode* rp = n->src[0]->src[0].get();
        int64_t M, N, K, batch;
        matmul_extents(mm, &M, &N, &K, &batch);
        MRK_TRY(materialize(mm->hint_inputs[0].get()));
        const std::shared_ptr<Buffer>& a = mm->hint_inputs[0]->buffer;
        std::shared_ptr<Buffer> w;
        bool nt = false;
        MRK_TRY(weight_operand(mm, true, &w, &nt));  // (a weight stored [N, K] is read in place)
        if (a->offset() % 16 || w->offset() % 16) return fail(kRuntime, "rope_matmul: unaligned operand");  // (views of whole tensors start aligned)
        auto out = new_buffer(n);
        std::shared_ptr<Buffer> rest_buf = rest ? new_buffer(rest) : out;
        MRK_TRY(builtin(nt ? "gemm_bf16_nt_rope" : "gemm_bf16_rope", {M, N, K, split, seq},
                        {out, a, w, rest_buf, rp->hint_inputs[1]->buffer, rp->hint_inputs[2]->buffer}));
        n->buffer = out;
        produced.push_back(n);
        if (rest) {
            rest->buffer = rest_buf;
            produced.push_back(rest);
        }
        return kOk;
    }

    int materialize(TensorNode* n) {
        if (n->buffer) return kOk;
        if (n->kind == TKind::Copy) return materialize_copy(n);
        if (n->numel() > 0 && fusable(n)) return materialize_fused(n);
        {
            TensorNode* other = nullptr;
            bool is_row = false;
            if (TensorNode* mm = residual_matmul(n, &other, &is_row)) return materialize_residual_matmul(n, mm, other, is_row);
            if (TensorNode* mm = swiglu_matmul(n)) return materialize_swiglu_matmul(n, mm);
            int64_t split = 0, seq = 0;
            if (TensorNode* mm = rope_matmul(n, &other, &split, &seq)) return materialize_rope_matmul(n, mm, other, split, seq);
        }
        {
            std::vector<int64_t> out_strides;
            if (TensorNode* att = attention_under(n, &out_strides)) return materialize_attention(att, n, out_strides);
        }
        if (generated_tc(n)) return materialize_generated_tc(n);
        // a reshape of materialised data is the same bytes, and so is making it contiguous
        if (n->kind == TKind::Reshape || n->kind == TKind::Contiguous) {
            TensorNode* s = n->src[0].get();
            TensorNode* other = nullptr;
            if (s->buffer || is_boundary_kind(s) || fusable(s) || generated_tc(s) || residual_matmul(s, &other) || swiglu_matmul(s)) {
                MRK_TRY(materialize(s));
                n->buffer = s->buffer;
                produced.push_back(n);
                return kOk;
            }
        }
        if (n->numel() == 0) {
            n->buffer = new_buffer(n);
            produced.push_back(n);
            return kOk;
        }
        std::set<const TensorNode*> seen;
        std::vector<TensorNode*> deps;
        int64_t max_numel = 0;
        boundaries(n, n, seen, deps, &max_numel);
        int64_t row_block = 0;
        const std::vector<TensorNode*> Rs = row_reduce_deps(n, deps, &row_block);
        if (!Rs.empty()) {
            std::vector<TensorNode*> sides;
            {
                const char* off = std::getenv("MOROK_NO_SIDE_OUTPUTS");  // measurement switch
                const bool enabled = !(off && off[0] && off[0] != '0');
                for (TensorNode* d : deps)
                    if (enabled && sides.size() < 2 && side_output_candidate(d, n)) sides.push_back(d);
                for (TensorNode* R : Rs) {  // the reductions' expressions may read such a tensor as well
                    if (!enabled) break;
                    std::set<const TensorNode*> seen_r;
                    std::vector<TensorNode*> deps_r;
                    int64_t ignore = 0;
                    boundaries(R, R, seen_r, deps_r, &ignore);
                    for (TensorNode* d : deps_r)
                        if (sides.size() < 2 && std::find(sides.begin(), sides.end(), d) == sides.end() && side_output_candidate(d, n)) sides.push_back(d);
                }
            }
            struct ClearSides {
                std::set<const TensorNode*>& s;
                ~ClearSides() { s.clear(); }
            } clear_sides{side_inline};
            if (!sides.empty()) {
                side_inline.insert(sides.begin(), sides.end());
                seen.clear();
                deps.clear();
                boundaries(n, n, seen, deps, &max_numel);
            }
            // everything any part of the kernel reads has to exist: the other inputs of the elementwise
            // part and the inputs of the reductions' own expressions
            auto fused = [&](const TensorNode* d) { return std::find(Rs.begin(), Rs.end(), d) != Rs.end(); };
            auto input = [&](TensorNode* d) {  // the kernels of this kernel's inputs are scheduled on their own terms
                std::set<const TensorNode*> mine;
                mine.swap(side_inline);
                const int rc = materialize(d);
                mine.swap(side_inline);
                return rc;
            };
            for (TensorNode* d : deps)
                if (!fused(d)) MRK_TRY(input(d));
            for (TensorNode* R : Rs) {
                std::set<const TensorNode*> seen_r;
                std::vector<TensorNode*> deps_r;
                boundaries(R, R, seen_r, deps_r, &max_numel);
                for (TensorNode* d : deps_r)
                    if (!fused(d)) MRK_TRY(input(d));
            }
            if (const char* e = std::getenv("MOROK_BEAM")) {
                const int beam = std::atoi(e);
                if (beam > 0 && !dry) return beam_generated(n, max_numel, beam, &Rs, row_block, &sides);
            }
            return gen_row_fused(n, Rs, row_block, max_numel, sides);
        }
        for (TensorNode* d : deps) MRK_TRY(materialize(d));
        if (const char* e = std::getenv("MOROK_BEAM")) {
            const int beam = std::atoi(e);
            if (beam > 0 && !dry) return beam_generated(n, max_numel, beam);
        }
        return n->kind == TKind::Reduce ? gen_reduce(n, max_numel) : gen_elementwise(n, max_numel);
    }

    // Beam search over the choices of one generated elementwise / reduce kernel
    // (tensor/src/realize.rs:1190-1242, schedule/src/optimizer/beam.rs:36-120): every candidate is
    // built as the real kernel would be, compiled and timed on buffers of the real sizes (inputs
    // that already hold data are read in place, everything else is zero-filled scratch), staged
    // like the matmul searches: UPCAST then LOCAL for an elementwise kernel, GROUP (waves per
    // output and segments) then LOCAL (outputs per workgroup) for a wave reduction.  The winner
    // is cached on disk under the hash of the kernel the fixed heuristics produce.
    int beam_generated(TensorNode* n, int64_t max_numel, int width, const std::vector<TensorNode*>* row_reduce = nullptr, int64_t row_block = 0,
                       const std::vector<TensorNode*>* sides = nullptr) {
        const bool red = n->kind == TKind::Reduce && !row_reduce;
        auto generate = [&]() -> int {
            if (row_reduce) return gen_row_fused(n, *row_reduce, row_block, max_numel, sides ? *sides : std::vector<TensorNode*>());
            return red ? gen_reduce(n, max_numel) : gen_elementwise(n, max_numel);
        };
        auto build = [&](const GenOpts& o, std::vector<DryKernel>* out) -> int {
            dry = true;
            gen_opts = o;
            dry_kernels.clear();
            const int rc = generate();
            dry = false;
            gen_opts = GenOpts();
            *out = std::move(dry_kernels);
            dry_kernels.clear();
            return rc;
        };
        auto for_real = [&](const GenOpts& o) -> int {
            gen_opts = o;
            const int rc = generate();
            gen_opts = GenOpts();
            return rc;
        };
        std::vector<DryKernel> base;
        MRK_TRY(build(GenOpts(), &base));
        int64_t work = n->numel();
        if (red) for (int64_t a : n->arg) work *= n->src[0]->shape[a];
        if (base.empty() || work < (1 << 16)) return for_real(GenOpts());  // too small to be worth a search
        uint64_t h = 1469598103934665603ull;
        for (const DryKernel& d : base) h = (h ^ d.k.content_hash) * 1099511628211ull;
        const std::string device = "HIP:" + std::to_string(dev->device_id);
        struct Record {
            int32_t opts[5];
            double ms;
        };
        auto to_opts = [](const Record& r) {
            GenOpts o;
            o.upcast_bytes = r.opts[0], o.local = r.opts[1], o.group = r.opts[2], o.split = r.opts[3], o.outs = r.opts[4];
            return o;
        };
        std::vector<uint8_t> cached;
        if (BeamCache::get(h, width, device, &cached) && cached.size() == sizeof(Record)) {
            Record r;
            std::memcpy(&r, cached.data(), sizeof r);
            const GenOpts o = to_opts(r);
            std::vector<DryKernel> probe;
            if (build(o, &probe) == kOk && !probe.empty()) {
                stats.beam_cache_hits++;
                return for_real(o);
            }
            clear_error();
        }
        double best_so_far = 1e300;
        std::set<std::string> tried;
        auto time_one = [&](const GenOpts& o, double* ms) -> bool {
            std::vector<DryKernel> ks;
            if (build(o, &ks) != kOk || ks.empty()) {
                clear_error();
                return false;
            }
            std::string sig;
            for (const DryKernel& d : ks) sig += std::to_string(d.k.content_hash) + ":";
            if (!tried.insert(sig).second) return false;  // the choice changed nothing
            double total = 0;
            for (const DryKernel& d : ks) {
                std::vector<std::unique_ptr<Buffer>> scratch;
                std::vector<void*> ptrs;
                for (const auto& bp : d.bufs) {
                    const Buffer* use = bp.get();
                    if (!bp->is_allocated() || bp.get() == d.bufs[0].get()) {
                        BufferOptions bo;
                        bo.zero_init = true;
                        scratch.push_back(std::make_unique<Buffer>(dev->allocator, bp->size(), bo));
                        if (scratch.back()->ensure_allocated() != kOk) return false;
                        use = scratch.back().get();
                    }
                    void* ptr = nullptr;
                    if (use->as_raw_ptr(&ptr) != kOk) return false;
                    ptrs.push_back(ptr);
                }
                BenchmarkResult r;
                bool skipped = false;
                if (compile_and_time(*dev, d.k, "beam_candidate", ptrs.data(), ptrs.size(), nullptr, 0, 2, 5, &r,
                                     best_so_far < 1e300 ? 3.0 * best_so_far : 0.0, &skipped) != kOk) {
                    clear_error();
                    return false;
                }
                if (skipped) return false;
                total += r.min_ms;
            }
            stats.beam_candidates++;
            *ms = total;
            best_so_far = std::min(best_so_far, total);
            return true;
        };
        using Cand = std::pair<double, GenOpts>;
        auto keep_best = [&](std::vector<Cand>& v) {
            std::sort(v.begin(), v.end(), [](const Cand& x, const Cand& y) { return x.first < y.first; });
            if (static_cast<int>(v.size()) > width) v.resize(width);
        };
        std::vector<Cand> beam;
        {
            double ms;
            if (!time_one(GenOpts(), &ms)) return for_real(GenOpts());
            beam.emplace_back(ms, GenOpts());
        }
        if (row_reduce) {
            // LOCAL: the work-items that share a row (the row stays in their registers)
            for (int local : {64, 128, 256, 512, 1024}) {
                GenOpts o;
                o.local = local;
                double ms;
                if (time_one(o, &ms)) beam.emplace_back(ms, o);
            }
            keep_best(beam);
        } else if (!red) {
            for (int up : {8, 4, 32}) {
                GenOpts o;
                o.upcast_bytes = up;
                double ms;
                if (time_one(o, &ms)) beam.emplace_back(ms, o);
            }
            keep_best(beam);
            std::vector<Cand> next = beam;
            for (const Cand& c : beam)
                for (int local : {64, 128, 512, 1024}) {
                    GenOpts o = c.second;
                    o.local = local;
                    double ms;
                    if (time_one(o, &ms)) next.emplace_back(ms, o);
                }
            beam = next;
            keep_best(beam);
        } else {
            int64_t R = 1;
            for (int64_t a : n->arg) R *= n->src[0]->shape[a];
            const int64_t Nout = n->numel();
            for (int grp : {1, 2, 4, 8, 16})
                for (int split : {1, 4, 16, 64, 256}) {
                    if (R / split < 64LL * grp || Nout * split > (1LL << 22) || (split > 1 && R / split < 1024)) continue;
                    GenOpts o;
                    o.group = grp, o.split = split;
                    double ms;
                    if (time_one(o, &ms)) beam.emplace_back(ms, o);
                }
            keep_best(beam);
            std::vector<Cand> next = beam;
            for (const Cand& c : beam) {
                if (c.second.group > 1) continue;  // a shared output owns its workgroup
                for (int outs : {1, 2, 8, 16}) {
                    GenOpts o = c.second;
                    if (o.group == 0) o.group = 1, o.split = 0;
                    o.outs = outs;
                    double ms;
                    if (time_one(o, &ms)) next.emplace_back(ms, o);
                }
            }
            beam = next;
            keep_best(beam);
        }
        const GenOpts& w = beam[0].second;
        Record r{{w.upcast_bytes, w.local, w.group, w.split, w.outs}, beam[0].first};
        (void)BeamCache::put(h, width, device, &r, sizeof r);  // a read-only cache directory is not an error
        clear_error();
        return for_real(w);
    }

    // A reshape / permute chain whose only source is a fusable attention node nobody else
    // reads: the kernel can write that layout itself.  Returns the attention node and the
    // strides of its [B, H, Sq, D] output inside the chain end's dense buffer.
    TensorNode* attention_under(TensorNode* n, std::vector<int64_t>* out_strides) const {
        if (!g_fusion || n->numel() == 0 || n->hint != HintKind::None || (n->kind != TKind::Reshape && n->kind != TKind::Permute)) return nullptr;
        std::vector<int64_t> st = dense_strides(n->shape);
        TensorNode* m = n;
        while (m->hint == HintKind::None && (m->kind == TKind::Reshape || m->kind == TKind::Permute)) {
            TensorNode* c = m->src[0].get();
            if (c->buffer) return nullptr;
            auto u = uses.find(c);
            if (u == uses.end() || u->second != 1) return nullptr;
            std::vector<int64_t> cst(c->shape.size(), 0);
            if (m->kind == TKind::Permute) {
                for (size_t i = 0; i < m->shape.size(); i++) cst[m->arg[i]] = st[i];
            } else if (!reshape_strides(m->shape, st, c->shape, &cst)) {
                return nullptr;
            }
            st = cst;
            m = c;
        }
        if (m->hint != HintKind::Sdpa || !fusable(m)) return nullptr;
        if (st.size() != 4 || st[3] != 1 || st[0] % 8 || st[1] % 8 || st[2] % 8) return nullptr;
        if (st[2] > (1LL << 30) || (m->shape[2] - 1) * st[2] * 2 + m->shape[3] * 2 > 0xffffffffLL) return nullptr;
        *out_strides = st;
        return m;
    }

    // The attention kernel over whatever views its operands are: an operand that is a strided
    // view of data in memory (rows of head-dim contiguous elements, 16-byte aligned) is read in
    // place, anything else is materialised first.  `dst` is the node that receives the buffer,
    // `out_strides` the layout of the [B, H, Sq, D] result inside it.
    int materialize_attention(TensorNode* att, TensorNode* dst, const std::vector<int64_t>& out_strides) {
        const TensorNode* q = att->hint_inputs[0].get();
        const TensorNode* k = att->hint_inputs[1].get();
        const int64_t B = q->shape[0], H = q->shape[1], Sq = q->shape[2], Sk = k->shape[2], D = q->shape[3];
        std::vector<int64_t> params;
        std::vector<std::shared_ptr<Buffer>> bufs(4);
        int64_t offsets[4] = {0, 0, 0, 0};
        std::vector<int64_t> strides;
        bool dense = true;
        for (int i = 0; i < 3; i++) {
            TensorNode* in = att->hint_inputs[i].get();
            StridedView v;
            bool ok = !in->buffer && strided_view(in, &v) && v.base != in && v.strides.size() == 4 && v.offset % 8 == 0;
            // only data that is (or will be) in memory anyway: a view of an unrealised
            // elementwise expression is cheaper computed over the view alone
            ok = ok && (v.base->buffer || is_boundary_kind(v.base) || fusable(v.base));
            if (ok) {
                for (int a = 0; a < 4; a++)
                    if (in->shape[a] == 1) v.strides[a] = 0;
                const int64_t rows = in->shape[2];
                ok = (D == 1 || v.strides[3] == 1) && v.strides[0] >= 0 && v.strides[1] >= 0 && v.strides[2] >= 0 &&
                     v.strides[0] % 8 == 0 && v.strides[1] % 8 == 0 && v.strides[2] % 8 == 0 && v.strides[2] <= (1LL << 30) &&
                     (rows - 1) * v.strides[2] * 2 + D * 2 <= 0xffffffffLL;
            }
            if (ok) {
                MRK_TRY(materialize(v.base));
                bufs[i + 1] = v.base->buffer;
                offsets[i] = v.offset;
                strides.insert(strides.end(), v.strides.begin(), v.strides.begin() + 3);
                dense = false;
            } else {
                MRK_TRY(materialize(in));
                bufs[i + 1] = in->buffer;
                const std::vector<int64_t> ds = dense_strides(in->shape);
                strides.insert(strides.end(), ds.begin(), ds.begin() + 3);
            }
        }
        strides.insert(strides.end(), out_strides.begin(), out_strides.begin() + 3);
        dense = dense && out_strides == dense_strides(att->shape);
        // attn_mask: read in place where it is a view of data in memory with contiguous keys whose
        // offset and strides are multiples of four elements; else materialised in its own shape
        const bool has_mask = att->hint_inputs.size() > 3;
        int64_t mask_offset = 0, mask_strides[3] = {0, 0, 0};
        std::shared_ptr<Buffer> mask_buf;
        if (has_mask) {
            TensorNode* m = att->hint_inputs[3].get();
            const size_t mr = m->shape.size();
            std::vector<int64_t> mst;
            StridedView v;
            bool ok = !m->buffer && strided_view(m, &v) && v.base != m && v.strides.size() == mr && v.offset % 4 == 0 &&
                      (v.base->buffer || is_boundary_kind(v.base) || fusable(v.base)) && (m->shape.back() == 1 || v.strides.back() == 1);
            if (ok)
                for (size_t a = 0; a + 1 < mr; a++) ok = ok && (m->shape[a] == 1 || (v.strides[a] >= 0 && v.strides[a] % 4 == 0));
            if (ok) {
                MRK_TRY(materialize(v.base));
                mask_buf = v.base->buffer;
                mask_offset = v.offset;
                mst = v.strides;
            } else {
                MRK_TRY(materialize(m));
                mask_buf = m->buffer;
                mst = dense_strides(m->shape);
            }
            for (size_t a = 0; a + 1 < mr; a++) mask_strides[4 - mr + a] = m->shape[a] == 1 ? 0 : mst[a];
        }
        auto out = new_buffer(dst);
        bufs[0] = out;
        float scale = static_cast<float>(att->hint_scale);
        uint32_t bits;
        std::memcpy(&bits, &scale, 4);
        if (has_mask || att->hint_softcap > 0.0) {
            float cap = static_cast<float>(att->hint_softcap);
            uint32_t cap_bits;
            std::memcpy(&cap_bits, &cap, 4);
            const int64_t kind = !has_mask ? 0 : att->hint_inputs[3]->dtype == Scalar::Bool ? 1 : 2;
            params = {B, H, Sq, Sk, D, att->hint_causal ? 1 : 0, static_cast<int64_t>(bits), att->hint_softcap > 0.0 ? static_cast<int64_t>(cap_bits) : 0,
                      kind, offsets[0], offsets[1], offsets[2], 0, mask_offset};
            params.insert(params.end(), strides.begin(), strides.end());
            params.insert(params.end(), mask_strides, mask_strides + 3);
            bufs.push_back(has_mask ? mask_buf : bufs[1]);
            // a handful of queries without the causal rule: the kernel that splits the keys, with its scratch
            const size_t ws = flash_fwd_workspace_bytes(B * H, Sq, Sk, D, att->hint_causal ? 1 : 0);
            if (ws) {
                bufs.push_back(std::make_shared<Buffer>(dev->allocator, ws, BufferOptions()));
                params.push_back(static_cast<int64_t>(ws));
            }
            MRK_TRY(builtin("flash_fwd_bf16_ext", params, bufs));
        } else {
            // a handful of queries against a long key sequence: the keys are split over workgroups and the ranges'
            // partial results go through scratch, an intermediate of the plan like any other
            const size_t ws = flash_fwd_workspace_bytes(B * H, Sq, Sk, D, att->hint_causal ? 1 : 0);
            if (ws) bufs.push_back(std::make_shared<Buffer>(dev->allocator, ws, BufferOptions()));
            if (dense) {
                params = {B * H, Sq, Sk, D, att->hint_causal ? 1 : 0, static_cast<int64_t>(bits)};
            } else {
                params = {B, H, Sq, Sk, D, att->hint_causal ? 1 : 0, static_cast<int64_t>(bits), offsets[0], offsets[1], offsets[2], 0};
                params.insert(params.end(), strides.begin(), strides.end());
            }
            if (ws) params.push_back(static_cast<int64_t>(ws));
            MRK_TRY(builtin(dense ? "flash_fwd_bf16" : "flash_fwd_bf16_strided", params, bufs));
        }
        dst->buffer = out;
        produced.push_back(dst);
        return kOk;
    }

    int materialize_fused(TensorNode* n) {
        if (n->hint == HintKind::Sdpa) return materialize_attention(n, n, dense_strides(n->shape));
        std::shared_ptr<Buffer> wbuf;  // a bf16 product's second operand, and its layout
        bool nt = false;
        if (n->hint == HintKind::Matmul && (n->hint_inputs[0]->dtype == Scalar::BFloat16 || n->hint_inputs[0]->dtype == Scalar::Float16)) {
            int64_t M, N, K, batch;
            matmul_extents(n, &M, &N, &K, &batch);
            MRK_TRY(materialize(n->hint_inputs[0].get()));
            MRK_TRY(weight_operand(n, gemm_bf16_nt_supported(M, N, K, batch), &wbuf, &nt));
        } else {
            for (const TensorRef& in : n->hint_inputs) MRK_TRY(materialize(in.get()));
        }
        auto out = new_buffer(n);
        int rc = kOk;
        if (n->hint == HintKind::Softmax) {
            const int64_t cols = n->shape.back(), rows = n->numel() / cols;
            rc = builtin("softmax_f32", {rows, cols}, {out, n->hint_inputs[0]->buffer});
        } else if (n->hint == HintKind::Matmul) {
            const TensorNode *a = n->hint_inputs[0].get(), *w = n->hint_inputs[1].get();
            const int64_t K = a->shape.back(), N = w->shape.back();
            int64_t M = a->shape[a->shape.size() - 2], batch = 1;
            for (size_t i = 0; i + 2 < a->shape.size(); i++) (w->shape.size() == 2 ? M : batch) *= a->shape[i];
            if (a->dtype == Scalar::BFloat16 || a->dtype == Scalar::Float16) {
                // few output tiles against a long K: scratch for split-K partials, an intermediate
                // of the plan like any other (lazily allocated, placed by the memory planner)
                // (up to 64 rows against an [N, K] weight stream it in one pass and need no scratch)
                const size_t ws = nt ? gemm_bf16_nt_workspace_bytes(M, N, K, batch) : gemm_bf16_workspace_bytes(M, N, K, batch);
                const std::string kind = a->dtype == Scalar::Float16 ? "gemm_f16" : "gemm_bf16";
                if (nt && ws) {
                    auto scratch = std::make_shared<Buffer>(dev->allocator, ws, BufferOptions());
                    rc = builtin((kind + "_nt").c_str(), {M, N, K, 1, static_cast<int64_t>(ws)}, {out, a->buffer, wbuf, scratch});
                } else if (nt) {
                    rc = builtin((kind + "_nt").c_str(), {M, N, K}, {out, a->buffer, wbuf});
                } else if (ws) {
                    auto scratch = std::make_shared<Buffer>(dev->allocator, ws, BufferOptions());
                    rc = builtin(kind.c_str(), {M, N, K, batch, static_cast<int64_t>(ws)}, {out, a->buffer, wbuf, scratch});
                } else {
                    rc = batch == 1 ? builtin(kind.c_str(), {M, N, K}, {out, a->buffer, wbuf}) : builtin(kind.c_str(), {M, N, K, batch}, {out, a->buffer, wbuf});
                }
            } else {
                // MOROK_BEAM=<width> selects the LOCAL/UPCAST/UNROLL choices by timed search
                // (cached on disk) instead of the fixed heuristic (tensor/src/realize.rs:1160-1250)
                // fixed heuristic: the operand tiles go through local memory, with the largest of three
                // workgroup tiles (128 x 128, 64 x 64, 64 rows x 32 columns) that still leaves at least
                // 512 workgroups (two per compute unit), else the smallest that divides the shape;
                // shapes none of them divides read their operands straight from global memory
                MatmulF32Opts opts;
                const MatmulF32Opts tiles[3] = {{32, 16, 4, 8, 1, 16}, {16, 16, 4, 4, 1, 16}, {8, 16, 4, 4, 1, 16}};
                for (const MatmulF32Opts& c : tiles) {
                    if (!matmul_f32_opts_valid(c, M, N, K)) continue;
                    opts = c;
                    if ((M / (c.local_y * c.up_m)) * (N / (c.local_x * c.up_n)) >= 512) break;
                }
                int beam = 0;
                if (const char* e = std::getenv("MOROK_BEAM")) beam = std::atoi(e);
                if (beam > 0) MRK_TRY(beam_search_matmul_f32(*dev, M, N, K, beam, &opts, nullptr, nullptr, nullptr));
                LinearKernel k = build_matmul_f32_kernel(M, N, K, opts);
                std::shared_ptr<CachedKernel> ck;
                bool cached = false;
                const std::string name = "r_" + std::to_string(M) + "_" + std::to_string(N) + "_" + std::to_string(K);
                MRK_TRY(compile_kernel(k, name.c_str(), &ck, &cached));
                rc = add_kernel(ck, {out, a->buffer, w->buffer}, cached);
            }
        }
        MRK_TRY(rc);
        n->buffer = out;
        produced.push_back(n);
        return kOk;
    }

    // Choices a search may make for a generated kernel in place of the fixed heuristics
    // (the optimizer's actions on an elementwise / reduce kernel, schedule/src/optimizer/beam.rs:36-120);
    // 0 leaves a choice to the heuristic.
    struct GenOpts {
        int upcast_bytes = 0;  // UPCAST: bytes of consecutive outputs per work-item (elementwise; heuristic 16)
        int local = 0;         // LOCAL: work-items per workgroup (elementwise; heuristic 256)
        int group = 0;         // GROUP: waves that share one output through local memory (wave reductions)
        int split = 0;         // with group: segments per output folded by a second kernel (1 = none)
        int outs = 0;          // LOCAL: outputs (one wave each) per workgroup when group == 1 (heuristic 4)
    };
    GenOpts gen_opts;
    // dry run: kernels are built and collected here instead of being compiled and queued, and
    // no node is marked as produced (a search builds every candidate this way)
    struct DryKernel {
        LinearKernel k;
        std::vector<std::shared_ptr<Buffer>> bufs;
    };
    bool dry = false;
    std::vector<DryKernel> dry_kernels;

    int queue_kernel(KernelGen& g, const std::shared_ptr<Buffer>& out, const std::string& name) {
        LinearKernel k = g.b.finish();
        if (dry) {
            DryKernel d;
            d.k = std::move(k);
            d.bufs.push_back(out);
            d.bufs.insert(d.bufs.end(), g.inputs.begin(), g.inputs.end());
            dry_kernels.push_back(std::move(d));
            return kOk;
        }
        std::shared_ptr<CachedKernel> ck;
        bool cached = false;
        MRK_TRY(compile_kernel(k, name.c_str(), &ck, &cached));
        std::vector<std::shared_ptr<Buffer>> bufs{out};
        bufs.insert(bufs.end(), g.inputs.begin(), g.inputs.end());
        return add_kernel(ck, bufs, cached);
    }
    int finish_kernel(KernelGen& g, TensorNode* n, const std::shared_ptr<Buffer>& out, const std::string& name) {
        MRK_TRY(queue_kernel(g, out, name));
        if (dry) return kOk;
        n->buffer = out;
        produced.push_back(n);
        return kOk;
    }

    // The cat a kernel rooted at `n` may split on: reached from the root through single-source
    // nodes that neither reduce nor reorder within the innermost axis in ways the caller cannot
    // check (the caller verifies the coordinate correspondence by probing), with at least two
    // parts of equal extent along the cat's last axis, each a whole number of upcast groups,
    // and at least one part that is not already in memory (else selecting costs nothing).
    static const TensorNode* root_cat(const TensorNode* n, int64_t width) {
        if (width <= 1 || n->shape.empty()) return nullptr;
        const TensorNode* m = n;
        while (!m->buffer && m->hint == HintKind::None &&
               (m->kind == TKind::Contiguous || m->kind == TKind::Cast || m->kind == TKind::Permute || m->kind == TKind::Reshape) && m != nullptr) {
            if (m->src.empty()) return nullptr;
            m = m->src[0].get();
        }
        if (m->buffer || m->kind != TKind::Cat || m->src.size() < 2 || m->src.size() > 4 || m->shape.empty()) return nullptr;
        const size_t axis = static_cast<size_t>(m->arg[0]);
        if (axis + 1 != m->shape.size() || m->shape[axis] != n->shape.back()) return nullptr;
        bool computed = false;
        for (const TensorRef& p : m->src) {
            if (p->shape[axis] != m->src[0]->shape[axis] || p->shape[axis] % width) return nullptr;
            computed = computed || !p->buffer;
        }
        return computed ? m : nullptr;
    }

    // Workgroup index of a generated kernel.  `gdims` are the kernel's global axes counted in
    // workgroups, outermost first (the order of the GLOBAL ranges of the reference's kernels).
    // Their launch extents (gidx0..2) and the index of every axis come from get_grouped_dims
    // under this device's limits (schedule/src/gpudims.rs:60-196,331-382): the innermost axis
    // lands on gidx0, axes beyond three or beyond 65535 in y / z are regrouped and recovered
    // with mod / div.  Returns the row-major flat workgroup index (0 on failure, error set).
    uint32_t workgroup_index(KernelBuilder& b, Scalar idx_t, const std::vector<int64_t>& gdims) {
        static const RendererCaps caps = amd_cdna4_caps();
        std::vector<size_t> d(gdims.begin(), gdims.end());
        const GroupedDims gd = get_grouped_dims(d, &caps.global_max, DimOrder::kReverseDims);
        for (size_t i = 0; i < gd.launch.size(); i++)
            if (i >= caps.global_max.size() || gd.launch[i] > caps.global_max[i]) {
                fail(kInvalidArgument, "realize: tensor too large for one launch");
                return 0;
            }
        std::vector<uint32_t> raw;
        for (size_t i = 0; i < gd.launch.size(); i++) {
            uint32_t sp = b.special("gidx" + std::to_string(i), static_cast<int64_t>(gd.launch[i]));
            raw.push_back(idx_t != Scalar::Int32 ? b.cast(sp, idx_t) : sp);
        }
        const std::vector<uint32_t> ax = gd.map_nodes(b, raw);
        uint32_t flat = ax[0];
        for (size_t i = 1; i < ax.size(); i++) flat = b.iadd(b.imul(flat, gdims[i]), ax[i]);
        return flat;
    }
    // Global axes of a kernel over `rows` rows of `per_row` work-items each with `block` work-items
    // per workgroup: [rows, workgroups per row] when workgroups tile a row exactly, else the flat
    // workgroup count.
    static std::vector<int64_t> workgroup_axes(int64_t items, int64_t per_row, int64_t block) {
        if (per_row > 0 && per_row % block == 0 && items % per_row == 0 && items / per_row > 1)
            return {items / per_row, per_row / block};
        return {(items + block - 1) / block};
    }

    // Row-resident fusion: an elementwise kernel whose one unrealised reduce input folds the last
    // axis of a tensor of the output's own shape (keepdim), as rms_norm's x * rsqrt(mean(x^2) + eps)
    // does.  One workgroup then owns a row: it folds the row (wave reduction + local memory),
    // keeps the total in a register and produces the row's outputs from the values it already
    // loaded, so the row is read once and the reduction needs no kernel and no buffer of its own.
    // Returns the reduce nodes, or nothing when the shape does not fit (the separate kernels remain).
    // Up to three such reductions may feed the kernel, one building on another (softmax: the row
    // maximum, then the sum of exp(x - max); layer norm: the mean, then the variance of the centred
    // row): they are returned in an order in which each one's own expression only needs earlier ones.
    std::vector<TensorNode*> row_reduce_deps(const TensorNode* n, const std::vector<TensorNode*>& deps, int64_t* block_out) {
        const char* off = std::getenv("MOROK_NO_ROW_FUSION");
        if (off && off[0] && off[0] != '0') return {};
        if (n->kind == TKind::Reduce || n->shape.empty() || n->dtype == Scalar::Bool || n->numel() == 0) return {};
        const int64_t last = static_cast<int64_t>(n->shape.size()) - 1;
        auto qualifies = [&](const TensorNode* R) {
            if (R->buffer || R->kind != TKind::Reduce || R->src.size() != 1 || R->arg.size() != 1) return false;
            if (R->src[0]->shape != n->shape || R->arg[0] != last) return false;
            const ReduceOp op = static_cast<ReduceOp>(R->sub);
            if (compute_dtype(R->dtype) != Scalar::Float32 || (op != ReduceOp::Add && op != ReduceOp::Max)) return false;
            auto u = uses.find(R);
            return u != uses.end() && u->second == 1;  // else somebody wants the reduction in memory
        };
        // the reductions directly under n, and the ones under those
        std::vector<TensorNode*> found;
        std::map<TensorNode*, std::vector<TensorNode*>> needs;  // reduction -> qualifying reductions its expression reads
        std::vector<TensorNode*> todo;
        for (TensorNode* d : deps)
            if (!d->buffer && d->kind == TKind::Reduce) todo.push_back(d);
        while (!todo.empty()) {
            TensorNode* R = todo.back();
            todo.pop_back();
            if (std::find(found.begin(), found.end(), R) != found.end()) continue;
            if (!qualifies(R)) {
                // a reduction of another shape directly under n rules the fusion out; further down it is
                // simply computed first, like any other input
                if (std::find(deps.begin(), deps.end(), R) != deps.end()) return {};
                continue;
            }
            found.push_back(R);
            if (found.size() > 3) return {};
            std::set<const TensorNode*> seen_r;
            std::vector<TensorNode*> deps_r;
            int64_t ignore = 0;
            boundaries(R, R, seen_r, deps_r, &ignore);
            for (TensorNode* d : deps_r)
                if (!d->buffer && d->kind == TKind::Reduce && qualifies(d)) {
                    needs[R].push_back(d);
                    todo.push_back(d);
                }
        }
        if (found.empty()) return {};
        std::vector<TensorNode*> ordered;
        while (ordered.size() < found.size()) {
            bool progress = false;
            for (TensorNode* R : found) {
                if (std::find(ordered.begin(), ordered.end(), R) != ordered.end()) continue;
                bool ready = true;
                for (TensorNode* d : needs[R]) ready = ready && std::find(ordered.begin(), ordered.end(), d) != ordered.end();
                if (ready) {
                    ordered.push_back(R);
                    progress = true;
                }
            }
            if (!progress) return {};
        }
        // The kernel hands a reduction's consumer the total of the workgroup's own row whatever
        // coordinates the consumer asks for, so every path from the output (and from a later
        // reduction's expression) down to a fused reduction must keep the row: elementwise nodes
        // of the output's shape, one expand of the keepdim shape, and below it elementwise nodes
        // and reshapes that only add or drop axes of extent 1.  A transpose, shrink, cat, gather
        // or any other expand on such a path (x + rowsum.T) keeps the separate reduce kernel.
        std::vector<int64_t> kshape = n->shape;
        kshape.back() = 1;
        auto strip1 = [](const std::vector<int64_t>& s) {
            std::vector<int64_t> r;
            for (int64_t d : s)
                if (d != 1) r.push_back(d);
            return r;
        };
        const std::vector<int64_t> kstripped = strip1(kshape);
        std::map<const TensorNode*, bool> reach_memo;
        std::function<bool(const TensorNode*)> reaches = [&](const TensorNode* m) -> bool {
            if (std::find(found.begin(), found.end(), m) != found.end()) return true;
            if (m->buffer || m->kind == TKind::Reduce) return false;
            auto it = reach_memo.find(m);
            if (it != reach_memo.end()) return it->second;
            bool r = false;
            for (const TensorRef& c : m->src) r = r || reaches(c.get());
            return reach_memo[m] = r;
        };
        std::map<std::pair<const TensorNode*, bool>, bool> ok_memo;
        std::function<bool(const TensorNode*, bool)> keeps_row = [&](const TensorNode* m, bool full) -> bool {
            if (std::find(found.begin(), found.end(), m) != found.end()) return !full && m->shape == kshape;
            if (!reaches(m)) return true;  // read at the coordinates it is asked for, like any operand
            auto it = ok_memo.find({m, full});
            if (it != ok_memo.end()) return it->second;
            bool ok = false;
            switch (m->kind) {
                case TKind::Unary:
                case TKind::Binary:
                case TKind::Where:
                case TKind::Cast:
                case TKind::Contiguous:
                    ok = true;
                    for (const TensorRef& c : m->src) ok = ok && c->shape == m->shape && keeps_row(c.get(), full);
                    break;
                case TKind::Expand: ok = full && m->shape == n->shape && m->src[0]->shape == kshape && keeps_row(m->src[0].get(), false); break;
                case TKind::Reshape:
                    ok = !full && strip1(m->shape) == kstripped && strip1(m->src[0]->shape) == kstripped && keeps_row(m->src[0].get(), false);
                    break;
                default: break;
            }
            return ok_memo[{m, full}] = ok;
        };
        if (!keeps_row(n, true)) return {};
        for (TensorNode* R : ordered)
            if (!keeps_row(R->src[0].get(), true)) return {};
        const int64_t C = n->shape.back(), rows = n->numel() / C;
        int64_t width = 1;
        for (int64_t w = 16 / static_cast<int64_t>(scalar_size(n->dtype)); w > 1; w /= 2)
            if (C % w == 0) {
                width = w;
                break;
            }
        const int64_t V = C / width;
        int64_t block = 0;
        for (int64_t c : {256, 128, 64})
            if (V % c == 0) {
                block = c;
                break;
            }
        // whole waves, at most 8 vectors per work-item (the row stays in registers), enough rows to fill the chip; a
        // handful of short rows (a decode step's activations: up to 1 MiB in all) is bound by launches, not by the
        // chip, and one kernel instead of a reduction and an elementwise kernel is the faster form there
        const bool tiny = n->numel() * static_cast<int64_t>(scalar_size(n->dtype)) <= (1 << 20);
        if (!block || V / block > 8 || (rows < 128 && !tiny)) return {};
        *block_out = block;
        return ordered;
    }

    int gen_row_fused(TensorNode* n, const std::vector<TensorNode*>& Rs, int64_t block, int64_t max_numel, const std::vector<TensorNode*>& sides = {}) {
        const int64_t N = n->numel(), C = n->shape.back(), rows = N / C;
        KernelGen g;
        g.idx_t = max_numel >= (1LL << 31) ? Scalar::Int64 : Scalar::Int32;
        KernelBuilder& b = g.b;
        auto out = new_buffer(n);
        uint32_t po = b.param(0, n->dtype, N);
        int64_t width = 1;
        for (int64_t w = 16 / static_cast<int64_t>(scalar_size(n->dtype)); w > 1; w /= 2)
            if (C % w == 0) {
                width = w;
                break;
            }
        g.width = width;
        if (gen_opts.local > 0) {  // a search's explicit choice; rows that do not split that way keep the heuristic
            const int64_t cand = gen_opts.local, Vt = C / width;
            if (cand % 64 || cand > 1024 || Vt % cand || Vt / cand > 8) return fail(kInvalidArgument, "row-resident kernel: the row does not split over that many work-items");
            block = cand;
        }
        const int64_t V = C / width, per_item = V / block, waves = block / 64;
        uint32_t row = workgroup_index(b, g.idx_t, {rows});
        if (!row) return last_status();
        uint32_t lx = b.special("lidx0", block);
        if (g.idx_t != Scalar::Int32) lx = b.cast(lx, g.idx_t);
        // vector i of this work-item: lx + i * block, so that a wave reads consecutive 16-byte pieces
        std::vector<uint32_t> base(per_item);
        std::vector<Coords> coords(per_item);
        for (int64_t i = 0; i < per_item; i++) {
            base[i] = b.imul(b.iadd(b.iadd(b.imul(row, V), lx), g.ci(i * block)), width);
            coords[i] = plain(unflatten(g, base[i], n->shape));
            if (width > 1) coords[i].back().aligned = true;
        }
        // ---- the row's reductions, in dependency order: per work-item, per wave, then across the
        // waves through local memory (an array of its own per reduction: no barrier is needed to
        // reuse one).  A later reduction's expression finds the earlier totals in g.fixed and the
        // values already computed for this row in the memo.
        for (size_t ri = 0; ri < Rs.size(); ri++) {
            TensorNode* R = Rs[ri];
            const TensorNode* src = R->src[0].get();
            const ReduceOp op = static_cast<ReduceOp>(R->sub);
            uint32_t acc = 0;
            for (int64_t i = 0; i < per_item; i++)
                for (int64_t e = 0; e < width; e++) {
                    Coords ce = coords[i];
                    ce.back().off = e;
                    uint32_t v = emit(g, src, ce);
                    if (b.dtype(v).scalar != Scalar::Float32) v = b.cast(v, Scalar::Float32);
                    acc = acc ? b.binary(op == ReduceOp::Add ? BinaryOp::Add : BinaryOp::Max, acc, v) : v;
                }
            uint32_t total = b.wave_reduce(op, acc);
            if (waves > 1) {
                uint32_t lds = b.define_local(static_cast<int>(ri), Scalar::Float32, waves);
                uint32_t lane = b.imod(lx, 64), wave = b.idiv(lx, 64);
                b.if_(b.binary(BinaryOp::Eq, lane, g.ci(0)));
                b.store(b.index(lds, wave), total);
                b.endif();
                b.barrier();
                total = b.load(b.index(lds, g.ci(0)));
                for (int64_t w = 1; w < waves; w++)
                    total = b.binary(op == ReduceOp::Add ? BinaryOp::Add : BinaryOp::Max, total, b.load(b.index(lds, g.ci(w))));
            }
            g.fixed[R] = R->dtype != Scalar::Float32 ? b.cast(total, compute_dtype(R->dtype)) : total;
        }
        // ---- the row's outputs, from the loads the reduction already made
        for (int64_t i = 0; i < per_item; i++) {
            std::vector<uint32_t> vals;
            for (int64_t e = 0; e < width; e++) {
                Coords ce = coords[i];
                ce.back().off = e;
                uint32_t v = n->kind == TKind::Contiguous ? emit(g, n->src[0].get(), ce) : emit_uncached(g, n, ce);
                if (b.dtype(v).scalar != n->dtype) v = b.cast(v, n->dtype);
                vals.push_back(v);
            }
            if (width > 1) b.store(b.index(po, base[i]), b.vectorize(vals));
            else b.store(b.index(po, base[i]), vals[0]);
        }
        // ---- side outputs: inputs of the row that this kernel computed in passing (the values are
        // the ones the reductions and the outputs used: same memo entries), written where a kernel of
        // their own would have put them
        std::vector<std::pair<TensorNode*, std::shared_ptr<Buffer>>> side_bufs;
        for (TensorNode* d : sides) {
            if (d->buffer) continue;  // another input of this kernel needed it first: it is in memory, and was read from there
            side_bufs.emplace_back(d, new_buffer(d));
            uint32_t ps = g.buffer_param(side_bufs.back().second, d->dtype, N);
            for (int64_t i = 0; i < per_item; i++) {
                std::vector<uint32_t> vals;
                for (int64_t e = 0; e < width; e++) {
                    Coords ce = coords[i];
                    ce.back().off = e;
                    uint32_t v = emit(g, d, ce);
                    if (b.dtype(v).scalar != d->dtype) v = b.cast(v, d->dtype);
                    vals.push_back(v);
                }
                if (width > 1) b.store(b.index(ps, base[i]), b.vectorize(vals));
                else b.store(b.index(ps, base[i]), vals[0]);
            }
        }
        MRK_TRY(finish_kernel(g, n, out, "rE_" + std::to_string(rows) + "_g" + std::to_string(C) + (width > 1 ? "_" + std::to_string(width) : "") +
                                             (Rs.size() > 1 ? "_x" + std::to_string(Rs.size()) : "") + (side_bufs.empty() ? "" : "_s" + std::to_string(side_bufs.size()))));
        if (!dry)
            for (auto& sb : side_bufs) {
                sb.first->buffer = sb.second;
                produced.push_back(sb.first);
            }
        return kOk;
    }

    // Materialised tensors under `n` of shape `shape`: reached through elementwise nodes only
    // (`direct`), or through at least one node that moves coordinates (`indirect`).
    static void flat_candidates(const TensorNode* n, const std::vector<int64_t>& shape, bool pure, std::set<const TensorNode*>* direct,
                                std::set<const TensorNode*>* indirect) {
        if (n->buffer) {
            (pure && n->shape == shape ? direct : indirect)->insert(n);
            return;
        }
        const bool elementwise = n->kind == TKind::Unary || n->kind == TKind::Binary || n->kind == TKind::Where || n->kind == TKind::Cast ||
                                 n->kind == TKind::Contiguous;
        for (const TensorRef& c : n->src) flat_candidates(c.get(), shape, pure && elementwise && c->shape == shape, direct, indirect);
    }

    int gen_elementwise(TensorNode* n, int64_t max_numel) {
        const int64_t N = n->numel();
        KernelGen g;
        g.idx_t = max_numel >= (1LL << 31) ? Scalar::Int64 : Scalar::Int32;
        KernelBuilder& b = g.b;
        auto out = new_buffer(n);
        uint32_t po = b.param(0, n->dtype, N);
        // UPCAST of the innermost axis: one work-item produces `width` consecutive outputs
        // (16 bytes of them) when the axis divides evenly
        int64_t width = 1;
        const int64_t up_bytes = gen_opts.upcast_bytes > 0 ? gen_opts.upcast_bytes : 16;
        if (!n->shape.empty() && n->dtype != Scalar::Bool)
            for (int64_t w = up_bytes / static_cast<int64_t>(scalar_size(n->dtype)); w > 1; w /= 2)
                if (n->shape.back() % w == 0) {
                    width = w;
                    break;
                }
        // flat upcast: the innermost axis gives no (or a narrower) group but the element count does
        // and some operand can be read flat (an odd vocabulary, [N, 3] points, a column vector)
        bool flat = false;
        const char* no_flat = std::getenv("MOROK_NO_FLAT_UPCAST");  // measurement switch
        if (n->dtype != Scalar::Bool && N > 0 && !(no_flat && no_flat[0] && no_flat[0] != '0')) {
            int64_t fw = 1;
            for (int64_t w = up_bytes / static_cast<int64_t>(scalar_size(n->dtype)); w > 1; w /= 2)
                if (N % w == 0) {
                    fw = w;
                    break;
                }
            if (fw > width) {
                std::set<const TensorNode*> direct, indirect;
                flat_candidates(n, n->shape, true, &direct, &indirect);
                for (const TensorNode* d : direct)
                    if (!indirect.count(d)) g.flat_leaves.insert(d);
                if (!g.flat_leaves.empty()) {
                    flat = true;
                    width = fw;
                }
            }
        }
        g.width = width;
        const int64_t items = N / width, block = gen_opts.local > 0 ? gen_opts.local : 256;
        uint32_t gx = workgroup_index(b, g.idx_t, workgroup_axes(items, n->shape.empty() ? 0 : n->shape.back() / width, block));
        if (!gx) return last_status();
        uint32_t lx = b.special("lidx0", block);
        if (g.idx_t != Scalar::Int32) lx = b.cast(lx, g.idx_t);
        uint32_t item = b.iadd(b.imul(gx, block), lx);
        b.if_(b.binary(BinaryOp::Lt, item, g.ci(items)));
        auto emit_group = [&](const Coords& coords, uint32_t base) {
            std::vector<uint32_t> vals;
            for (int64_t e = 0; e < width; e++) {
                Coords ce = coords;
                if (!ce.empty()) ce.back().off = e;
                uint32_t v = n->kind == TKind::Contiguous ? emit(g, n->src[0].get(), ce) : emit_uncached(g, n, ce);
                if (b.dtype(v).scalar != n->dtype) v = b.cast(v, n->dtype);
                vals.push_back(v);
            }
            if (width > 1) b.store(b.index(po, base), b.vectorize(vals));
            else b.store(b.index(po, base), vals[0]);
        };
        // A cat of computed parts along the innermost output axis (rotary embedding: cat(real,
        // imag)).  Evaluating every part for every output and selecting costs the arithmetic of
        // all parts; instead the work-items are renumbered so that the 64 of a wave produce
        // outputs of one part only (R rows x the part's vectors), and each part gets its own
        // guarded region, which a wave of the other part skips altogether.
        const TensorNode* cat = flat ? nullptr : root_cat(n, width);
        bool split = false;
        if (cat) {
            const int64_t P = static_cast<int64_t>(cat->src.size()), V = n->shape.back() / width, Vp = V / P;
            const size_t axis = static_cast<size_t>(cat->arg[0]);
            if (Vp >= 1 && V % P == 0 && 64 % Vp == 0 && block % (64 * P) == 0 && items % (64 * P) == 0) {
                const int64_t R = 64 / Vp;
                uint32_t grp = b.idiv(item, 64 * P), part = b.imod(b.idiv(item, 64), P), k = b.imod(item, 64);
                uint32_t row = b.iadd(b.imul(grp, R), b.idiv(k, Vp));
                uint32_t vec = b.iadd(b.imul(part, Vp), b.imod(k, Vp));
                uint32_t base = b.imul(b.iadd(b.imul(row, V), vec), width);
                Coords coords = plain(unflatten(g, base, n->shape));
                coords.back().aligned = true;
                // where along the cat axis this group lies: it has to be the innermost output
                // coordinate itself for the renumbering to make waves uniform
                g.pick_cat = cat;
                g.pick_part = -2;
                g.probed = false;
                (void)(n->kind == TKind::Contiguous ? emit(g, n->src[0].get(), coords) : emit_uncached(g, n, coords));
                g.memo.clear();
                g.vec_loads.clear();
                if (g.probed && g.probed_pos.aligned && g.probed_pos.off == 0 && g.probed_pos.node == coords.back().node) {
                    split = true;
                    int64_t start = 0;
                    for (int64_t pi = 0; pi < P; pi++) {
                        const int64_t len = cat->src[pi]->shape[axis];
                        uint32_t live = b.binary(BinaryOp::And, b.binary(BinaryOp::Ge, g.probed_pos.node, g.ci(start)),
                                                 b.binary(BinaryOp::Lt, g.probed_pos.node, g.ci(start + len)));
                        b.if_(live);
                        g.pick_part = static_cast<int>(pi);
                        emit_group(coords, base);
                        b.endif();
                        // values named inside a guarded region are not visible after it
                        g.memo.clear();
                        g.vec_loads.clear();
                        start += len;
                    }
                }
                g.pick_cat = nullptr;
                g.pick_part = -1;
            }
        }
        if (flat) {
            // every element gets its own coordinates (for what cannot be read flat); operands of the
            // output's shape ignore them and share one vector load per group
            uint32_t base = b.imul(item, width);
            g.flat_base = base;
            std::vector<uint32_t> vals;
            for (int64_t e = 0; e < width; e++) {
                g.flat_off = e;
                Coords ce = plain(unflatten(g, b.iadd(base, g.ci(e)), n->shape));
                uint32_t v = n->kind == TKind::Contiguous ? emit(g, n->src[0].get(), ce) : emit_uncached(g, n, ce);
                if (b.dtype(v).scalar != n->dtype) v = b.cast(v, n->dtype);
                vals.push_back(v);
            }
            b.store(b.index(po, base), b.vectorize(vals));
        } else if (!split) {
            uint32_t base = b.imul(item, width);
            Coords coords = plain(unflatten(g, base, n->shape));
            if (width > 1) coords.back().aligned = true;
            emit_group(coords, base);
        }
        b.endif();
        return finish_kernel(g, n, out, "E_" + std::to_string(N) + (width > 1 ? "_" + std::to_string(width) : "") + (flat ? "f" : ""));
    }

    int gen_reduce(TensorNode* n, int64_t max_numel) {
        const TensorNode* s = n->src[0].get();
        const ReduceOp op = static_cast<ReduceOp>(n->sub);
        const int64_t Nout = n->numel();
        std::vector<int64_t> rdims;
        int64_t R = 1;
        for (int64_t a : n->arg) {
            rdims.push_back(s->shape[a]);
            R *= s->shape[a];
        }
        KernelGen g;
        g.idx_t = max_numel >= (1LL << 31) ? Scalar::Int64 : Scalar::Int32;
        KernelBuilder& b = g.b;
        auto out = new_buffer(n);
        const Scalar ct = compute_dtype(n->dtype);
        // A reduction that keeps the innermost (contiguous) axis of its input - column sums, a fold
        // over a middle axis - puts the lanes along that kept axis: a work-item per output walks
        // the reduce range, so every load of a wave is one contiguous row piece.  (Lanes along the
        // reduce range, as for row reductions, would stride the input by whole rows.)
        const bool reduces_last = std::find(n->arg.begin(), n->arg.end(), static_cast<int64_t>(s->shape.size()) - 1) != n->arg.end();
        const bool columns = !reduces_last && !s->shape.empty() && s->shape.back() >= 16;
        const bool wave = R >= 128 && ct == Scalar::Float32 && (op == ReduceOp::Add || op == ReduceOp::Max) && !columns;
        // ... and when that leaves too few work-items to fill the chip, the outermost reduce axis is
        // cut into Pt segments (split_reduceop again): Pt times the work-items, partials laid out
        // [segment][output] so both kernels stay coalesced
        int64_t Pt = 1;
        if (!wave && columns && R >= 128)
            while (Pt * 2 * Nout <= (1 << 18) && rdims[0] % (Pt * 2) == 0 && R / (Pt * 2) >= 32) Pt *= 2;
        // Two-stage reduction (split_reduceop, schedule/src/rangeify/kernel.rs:44-61): when one
        // output folds at least 32768 inputs, the reduce range is cut into P segments (8 <= P <=
        // 256, partial buffer of at most 2^22 elements) reduced by P times as many waves, and
        // a second small kernel folds the P partials.
        int64_t P = 1;
        if (wave && R >= 32768) {
            for (int64_t d = 256; d >= 8; d /= 2)
                if (R / d >= 1024 && Nout * d <= (1LL << 22)) {
                    P = d;
                    break;
                }
        }
        // GROUP through local memory (GROUPTOP, schedule/src/optimizer/heuristics.rs:370-392: kernels
        // with at most 2048 outputs let several work-items share an output).  Here the sharing unit
        // is the wavefront: G waves of one workgroup fold interleaved 64-element blocks of the same
        // output (or of the same segment of it), leave their partial in local memory and, behind a
        // barrier, the first folds the G partials in order.  A split reduction keeps its number of
        // waves and folds G times fewer partials in the second kernel; an unsplit one with few
        // outputs gets up to 16 times the waves without a second launch.
        int64_t G = 1;
        const char* no_group = std::getenv("MOROK_NO_GROUP_REDUCE");  // measurement switch: every wave on its own
        const bool grouping = wave && Nout <= 2048 && !(no_group && no_group[0] && no_group[0] != '0');
        if (grouping && R >= 32768) {
            // waves per output: each folds at least 4096 inputs, about 4096 waves over the whole chip;
            // up to 16 of them form a workgroup, the rest are segments for the second kernel
            int64_t wpo = 1;
            while (wpo * 2 <= R / 4096 && wpo * 2 * Nout <= 4096) wpo *= 2;
            G = wpo < 16 ? wpo : 16;
            P = wpo / G;
            if (P > 256) P = 256;
        } else if (grouping) {  // more waves per output while each keeps at least 512 inputs
            for (int64_t c = 16; c > 1; c /= 2)
                if (R / c >= 512 && Nout * c <= 2048) {
                    G = c;
                    break;
                }
        }
        if (wave && gen_opts.group > 0) {  // a search's explicit choice
            G = gen_opts.group;
            P = gen_opts.split > 0 ? gen_opts.split : 1;
        }
        const int64_t chunk = (R + P - 1) / P;
        std::shared_ptr<Buffer> partial;
        if (P > 1) {
            BufferOptions bo;
            partial = std::make_shared<Buffer>(dev->allocator, static_cast<size_t>(Nout * P) * 4, bo);
        }
        uint32_t po = P > 1 ? b.param(0, Scalar::Float32, Nout * P) : Pt > 1 ? b.param(0, ct, Nout * Pt) : b.param(0, n->dtype, Nout);
        auto identity = [&]() -> uint32_t {
            if (is_float(ct)) return b.cf(op == ReduceOp::Add ? 0.0 : op == ReduceOp::Mul ? 1.0 : op == ReduceOp::Max ? -INFINITY : INFINITY, ct);
            return b.ci(op == ReduceOp::Mul ? 1 : 0, ct);
        };
        if (!wave) {
            // one work-item per output element (per segment of one), the reduced axes as nested sequential loops
            const int64_t block = 64, Wt = Nout * Pt, seg_len = rdims[0] / Pt;
            uint32_t gx = workgroup_index(b, g.idx_t, workgroup_axes(Wt, Pt > 1 || n->shape.empty() ? 0 : n->shape.back(), block));
            if (!gx) return last_status();
            uint32_t lx = b.special("lidx0", block);
            if (g.idx_t != Scalar::Int32) lx = b.cast(lx, g.idx_t);
            uint32_t o = b.iadd(b.imul(gx, block), lx);
            uint32_t gate = b.binary(BinaryOp::Lt, o, g.ci(Wt));
            uint32_t oc = b.where(gate, o, g.ci(Wt - 1));  // clamp: masked lanes recompute the last element
            uint32_t seg = Pt > 1 ? b.idiv(oc, Nout) : 0, oo = Pt > 1 ? b.imod(oc, Nout) : oc;
            Coords coords = plain(unflatten(g, oo, n->shape));
            std::vector<uint32_t> ranges;
            for (size_t r = 0; r < n->arg.size(); r++) {
                uint32_t rg = b.add(Op::Range, KernelBuilder::scalar(g.idx_t), {g.ci(r == 0 ? seg_len : rdims[r])}, static_cast<int64_t>(r), 0,
                                    static_cast<uint16_t>(AxisType::Reduce));
                ranges.push_back(rg);
                coords[n->arg[r]] = Cx{r == 0 && Pt > 1 ? b.iadd(b.imul(seg, seg_len), rg) : rg, 0, false};
            }
            uint32_t v = emit(g, s, coords);
            uint32_t red = b.reduce(op, v, ranges);
            std::vector<uint32_t> rev(ranges.rbegin(), ranges.rend());
            b.end(rev);
            b.if_(gate);
            uint32_t res = red;
            const Scalar store_t = Pt > 1 ? ct : n->dtype;
            if (b.dtype(res).scalar != store_t) res = b.cast(res, store_t);
            b.store(b.index(po, o), res);
            b.endif();
            if (Pt == 1) return finish_kernel(g, n, out, "r_" + std::to_string(Nout) + "_" + std::to_string(R));
            BufferOptions bo;
            auto part = std::make_shared<Buffer>(dev->allocator, static_cast<size_t>(Wt) * scalar_size(ct), bo);
            MRK_TRY(queue_kernel(g, part, "r_" + std::to_string(Nout) + "x" + std::to_string(Pt) + "_" + std::to_string(R / Pt)));
            // second stage: a work-item per output folds its Pt partials, one coalesced row of them per step
            KernelGen g2;
            KernelBuilder& b2 = g2.b;
            uint32_t po2 = b2.param(0, n->dtype, Nout);
            uint32_t pin = g2.buffer_param(part, ct, Wt);
            uint32_t gx2 = workgroup_index(b2, Scalar::Int32, workgroup_axes(Nout, 0, block));
            if (!gx2) return last_status();
            uint32_t o2 = b2.iadd(b2.imul(gx2, block), b2.special("lidx0", block));
            uint32_t gate2 = b2.binary(BinaryOp::Lt, o2, b2.ci(Nout));
            uint32_t oc2 = b2.where(gate2, o2, b2.ci(Nout - 1));
            uint32_t r2 = b2.range(Pt, 0, AxisType::Reduce);
            uint32_t pv = b2.load(b2.index(pin, b2.iadd(b2.imul(r2, Nout), oc2)));
            uint32_t red2 = b2.reduce(op, pv, {r2});
            b2.end({r2});
            b2.if_(gate2);
            uint32_t res2 = red2;
            if (b2.dtype(res2).scalar != n->dtype) res2 = b2.cast(res2, n->dtype);
            b2.store(b2.index(po2, o2), res2);
            b2.endif();
            return finish_kernel(g2, n, out, "r_" + std::to_string(Nout) + "_" + std::to_string(Pt));
        }
        // one wavefront per output element: lanes stride the flattened reduce space, partial
        // results are combined with the wave64 cross-lane reduction (the GROUP_REDUCE idea of
        // schedule/src/optimizer/heuristics.rs:370-392 without the LDS round trip)
        const int64_t W = Nout * P;  // wave-sized (G == 1) or workgroup-sized outputs of this kernel
        const int64_t per_block = G > 1 ? 1 : gen_opts.outs > 0 ? gen_opts.outs : 4;
        uint32_t gx = workgroup_index(b, g.idx_t, workgroup_axes(W, 0, per_block));
        if (!gx) return last_status();
        uint32_t lane = b.special("lidx0", 64), ly = b.special("lidx1", G > 1 ? G : per_block);
        if (g.idx_t != Scalar::Int32) {
            lane = b.cast(lane, g.idx_t);
            ly = b.cast(ly, g.idx_t);
        }
        // G == 1: wave ly of the workgroup owns output w; G > 1: the whole workgroup owns w = gx
        uint32_t w = G > 1 ? gx : b.iadd(b.imul(gx, per_block), ly);
        uint32_t wgate = b.binary(BinaryOp::Lt, w, g.ci(W));
        uint32_t wc = G > 1 ? w : b.where(wgate, w, g.ci(W - 1));
        uint32_t oc = P > 1 ? b.idiv(wc, P) : wc;
        uint32_t seg0 = P > 1 ? b.imul(b.imod(wc, P), chunk) : g.ci(0);  // first reduce index of the segment
        Coords coords = plain(unflatten(g, oc, n->shape));
        const int64_t steps = (chunk + 64 * G - 1) / (64 * G);
        uint32_t rg = b.add(Op::Range, KernelBuilder::scalar(g.idx_t), {g.ci(steps)}, 0, 0, static_cast<uint16_t>(AxisType::Reduce));
        // block rg * G + ly of the segment: the G waves read neighbouring 256-byte blocks
        uint32_t blk = G > 1 ? b.iadd(b.imul(rg, G), ly) : rg;
        uint32_t in_seg = b.iadd(b.imul(blk, 64), lane);
        uint32_t f = b.iadd(seg0, in_seg);
        const bool exact = chunk % (64 * G) == 0 && chunk * P == R;
        uint32_t fgate = b.binary(BinaryOp::And, b.binary(BinaryOp::Lt, in_seg, g.ci(chunk)), b.binary(BinaryOp::Lt, f, g.ci(R)));
        uint32_t fc = exact ? f : b.where(fgate, f, g.ci(R - 1));
        std::vector<uint32_t> rc = unflatten(g, fc, rdims);
        for (size_t r = 0; r < n->arg.size(); r++) coords[n->arg[r]] = Cx{rc[r], 0, false};
        uint32_t v = emit(g, s, coords);
        if (!exact) v = b.where(fgate, v, identity());
        uint32_t red = b.reduce(op, v, {rg});
        b.end({rg});
        uint32_t total = b.wave_reduce(op, red);
        uint32_t first = b.binary(BinaryOp::Eq, lane, g.ci(0));
        if (G > 1) {
            uint32_t lds = b.define_local(0, ct, G);
            b.if_(first);
            b.store(b.index(lds, ly), total);
            b.endif();
            b.barrier();
            b.if_(b.binary(BinaryOp::And, first, b.binary(BinaryOp::Eq, ly, g.ci(0))));
            uint32_t r2 = b.add(Op::Range, KernelBuilder::scalar(g.idx_t), {g.ci(G)}, 1, 0, static_cast<uint16_t>(AxisType::Reduce));
            uint32_t folded = b.reduce(op, b.load(b.index(lds, r2)), {r2});
            b.end({r2});
            uint32_t res = folded;
            if (P == 1 && b.dtype(res).scalar != n->dtype) res = b.cast(res, n->dtype);
            b.store(b.index(po, w), res);
            b.endif();
        } else {
            b.if_(b.binary(BinaryOp::And, first, wgate));
            uint32_t res = total;
            if (P == 1 && b.dtype(res).scalar != n->dtype) res = b.cast(res, n->dtype);
            b.store(b.index(po, w), res);
            b.endif();
        }
        const std::string grp = G > 1 ? "_l" + std::to_string(G) : "";  // waves sharing an output through local memory
        if (P == 1) return finish_kernel(g, n, out, "r_" + std::to_string(Nout) + "_g" + std::to_string(R) + grp);
        MRK_TRY(queue_kernel(g, partial, "r_" + std::to_string(Nout) + "x" + std::to_string(P) + "_g" + std::to_string(chunk) + grp));
        // second stage: one work-item per output folds its P partials
        KernelGen g2;
        KernelBuilder& b2 = g2.b;
        uint32_t po2 = b2.param(0, n->dtype, Nout);
        uint32_t pin = g2.buffer_param(partial, Scalar::Float32, Nout * P);
        const int64_t block2 = 64;
        uint32_t gx2 = workgroup_index(b2, Scalar::Int32, workgroup_axes(Nout, 0, block2));
        if (!gx2) return last_status();
        uint32_t o2 = b2.iadd(b2.imul(gx2, block2), b2.special("lidx0", block2));
        uint32_t gate2 = b2.binary(BinaryOp::Lt, o2, b2.ci(Nout));
        uint32_t oc2 = b2.where(gate2, o2, b2.ci(Nout - 1));
        uint32_t r2 = b2.range(P, 0, AxisType::Reduce);
        uint32_t pv = b2.load(b2.index(pin, b2.iadd(b2.imul(oc2, P), r2)));
        uint32_t red2 = b2.reduce(op, pv, {r2});
        b2.end({r2});
        b2.if_(gate2);
        uint32_t res2 = red2;
        if (b2.dtype(res2).scalar != n->dtype) res2 = b2.cast(res2, n->dtype);
        b2.store(b2.index(po2, o2), res2);
        b2.endif();
        return finish_kernel(g2, n, out, "r_" + std::to_string(Nout) + "_" + std::to_string(P));
    }
};

}  // namespace

// Scheduling writes provisional buffers onto graph nodes, and graphs of different roots may
// share nodes, so every path that reads or writes TensorNode::buffer runs under this lock:
// concurrent realizations of tensors over a common lazy subgraph are serialised for the
// (host-side) scheduling and for the enqueue of the plan, not for the GPU work itself.
static std::recursive_mutex g_graph_mutex;

namespace {
// Schedules `root`.  On success `kept` lists the nodes (root included) that keep a buffer whose
// contents exist only after the plan has run; on failure no node keeps one.
constexpr int kCompileFirst = -77001;  // internal: the schedule found kernels to compile; nothing was kept
int prepare_locked(const TensorRef& root, std::unique_ptr<ExecutionPlan>* out, std::vector<TensorNode*>* kept,
                   std::vector<Scheduler::PendingKernel>* deferred = nullptr, const std::set<uint64_t>* fresh = nullptr) {
    g_stats = RealizeStats();
    auto t0 = std::chrono::steady_clock::now();
    Scheduler s;
    s.deferred = deferred;
    s.fresh = fresh;
    // every exit that is not the successful one returns the touched nodes to their lazy state
    struct Rollback {
        Scheduler& s;
        bool armed = true;
        ~Rollback() {
            if (!armed) return;
            for (TensorNode* t : s.produced) t->buffer = nullptr;
            for (TensorNode* t : s.produced_host) t->host = nullptr;
        }
    } rollback{s};
    // a copy to the CPU is scheduled on the device its source lives on
    const bool to_cpu = root->device_id == kCpuDevice && root->kind == TKind::Copy;
    const int device_id = to_cpu ? root->src[0]->device_id : root->device_id;
    MRK_TRY(s.check_placement(root.get()));
    MRK_TRY(DeviceFactoryRegistry::global().device("HIP", device_id, &s.dev));
    s.plan.reset(new ExecutionPlan(device_id));
    s.count_uses(root.get());
    if (to_cpu) {
        if (!root->host) MRK_TRY(s.materialize(root.get()));
        s.plan->set_outputs({s.plan->add_buffer(root->src[0]->buffer)});  // the device side of the copy stays whole
    } else {
        if (!root->buffer) MRK_TRY(s.materialize(root.get()));
        s.plan->set_outputs({s.plan->add_buffer(root->buffer)});
    }
    if (deferred && !deferred->empty()) return kCompileFirst;  // (the rollback returns every touched node to its lazy state)
    // Intermediates share blocks by liveness (tensor/src/memory_planner.rs); their contents do
    // not outlive the plan's execution, so their nodes go back to being lazy: only the root
    // keeps its buffer.  MOROK_NO_MEMORY_PLANNER=1 keeps every intermediate resident.
    const char* no_planner = std::getenv("MOROK_NO_MEMORY_PLANNER");
    const bool planner = !(no_planner && no_planner[0] && no_planner[0] != '0');
    if (planner) s.plan->enable_memory_planner();
    MRK_TRY(s.plan->build());
    rollback.armed = false;
    for (TensorNode* t : s.produced) {
        if (planner && t != root.get()) t->buffer = nullptr;
        else if (kept) kept->push_back(t);
    }
    if (kept) kept->insert(kept->end(), s.produced_host.begin(), s.produced_host.end());
    s.stats.buffers_reused = s.plan->memory_plan().buffers_reused;
    s.stats.memory_saved = s.plan->memory_plan().memory_saved;
    s.stats.intermediate_bytes = s.plan->memory_plan().memory_planned;
    s.stats.elapsed_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    g_stats = s.stats;
    *out = std::move(s.plan);
    return kOk;
}
// Schedules `root` with the graph lock held by `lock` on entry and on return, but released while
// kernels are compiled: a first pass under the lock only collects what the kernel cache lacks and
// rolls the graph back, the compiles (the slow part: hiprtc) run unlocked, so realizations of
// other tensors proceed meanwhile (as the reference's get_or_compile_kernel lets compiles race,
// runtime/src/kernel_cache.rs:95-117), and a second pass under the lock builds the plan from the
// cache.  A graph that needs no new kernel takes one pass.  Under MOROK_BEAM the search times its
// candidates on the device and everything stays under the lock.
int prepare_compiling_unlocked(const TensorRef& root, std::unique_lock<std::recursive_mutex>& lock, std::unique_ptr<ExecutionPlan>* out,
                               std::vector<TensorNode*>* kept) {
    int beam = 0;
    if (const char* e = std::getenv("MOROK_BEAM")) beam = std::atoi(e);
    if (beam > 0) return prepare_locked(root, out, kept);
    std::vector<Scheduler::PendingKernel> pending;
    int rc = prepare_locked(root, out, kept, &pending);
    if (rc != kCompileFirst) return rc;
    const bool to_cpu = root->device_id == kCpuDevice && root->kind == TKind::Copy;
    const int device_id = to_cpu ? root->src[0]->device_id : root->device_id;
    std::shared_ptr<Device> dev;
    MRK_TRY(DeviceFactoryRegistry::global().device("HIP", device_id, &dev));
    std::set<uint64_t> fresh;
    lock.unlock();
    rc = kOk;
    for (const Scheduler::PendingKernel& p : pending) {
        std::shared_ptr<CachedKernel> ck;
        bool cached = false;
        rc = get_or_compile_linear_kernel(*dev, p.k, p.name.c_str(), &ck, &cached);
        if (rc != kOk) break;
        if (!cached) fresh.insert(p.k.content_hash);
    }
    lock.lock();
    if (rc != kOk) return rc;
    if (kept) kept->clear();
    return prepare_locked(root, out, kept, nullptr, &fresh);
}
}  // namespace

int Tensor::prepare(std::unique_ptr<ExecutionPlan>* out) const {
    if (!n_) return fail(kInvalidArgument, "prepare: invalid tensor");
    std::unique_lock<std::recursive_mutex> lock(g_graph_mutex);
    return prepare_compiling_unlocked(n_, lock, out, nullptr);
}

int Tensor::realize() const {
    if (!n_) return fail(kInvalidArgument, "realize: invalid tensor");
    std::unique_lock<std::recursive_mutex> lock(g_graph_mutex);
    if (n_->buffer || (n_->device_id == kCpuDevice && n_->host)) {
        g_stats = RealizeStats();
        return kOk;
    }
    auto t0 = std::chrono::steady_clock::now();
    std::unique_ptr<ExecutionPlan> plan;
    std::vector<TensorNode*> kept;
    MRK_TRY(prepare_compiling_unlocked(n_, lock, &plan, &kept));
    // The plan is enqueued before the lock is released: whoever sees the root's buffer next
    // queues its reads behind these kernels on the device's in-order stream.
    int rc = plan->execute();
    if (rc != kOk) {
        for (TensorNode* t : kept) {  // nothing was computed into them
            t->buffer = nullptr;
            if (t->kind == TKind::Copy && t->device_id == kCpuDevice) t->host = nullptr;
        }
        return rc;
    }
    g_stats.elapsed_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    return kOk;
}

std::shared_ptr<Buffer> Tensor::buffer() const {
    if (!n_) return nullptr;
    std::lock_guard<std::recursive_mutex> lock(g_graph_mutex);
    return n_->buffer;
}

int Tensor::to_bytes(void* dst, size_t nbytes) const {
    if (!n_) return fail(kInvalidArgument, "to_vec: invalid tensor");
    std::shared_ptr<Buffer> buf;
    std::shared_ptr<std::vector<uint8_t>> host;
    int host_from = kCpuDevice;
    for (int attempt = 0; attempt < 2 && !buf && !host; attempt++) {
        {
            std::lock_guard<std::recursive_mutex> lock(g_graph_mutex);
            if (n_->device_id == kCpuDevice) {
                host = n_->host;
                host_from = n_->host_from;
            } else {
                buf = n_->buffer;
            }
        }
        // realize takes the lock itself (and lets go of it while kernels compile)
        if (!buf && !host && attempt == 0) MRK_TRY(realize());
    }
    if (!buf && !host) return fail(kRuntime, "to_vec: the tensor has no data after realize");
    const size_t expect = static_cast<size_t>(n_->numel()) * scalar_size(n_->dtype);
    if (nbytes != expect) return failf(kSizeMismatch, "size mismatch: expected %zu, got %zu", expect, nbytes);
    if (expect == 0) return kOk;
    if (host) {
        if (host_from != kCpuDevice) {  // the copy that fills these bytes was queued on that device's stream
            std::shared_ptr<Allocator> a;
            MRK_TRY(AllocatorRegistry::global().get(host_from, &a));
            MRK_TRY(a->synchronize());
        }
        std::memcpy(dst, host->data(), expect);
        return kOk;
    }
    return buf->copyout(dst, nbytes);
}

}  // namespace mrk
