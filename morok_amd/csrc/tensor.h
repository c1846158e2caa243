// Lazy tensor API over the HIP device: the caller side of the boundary
// (tensor/src/realize.rs:83-127,299-357,937-1117; tensor/src/schedule.rs:238-501) and the op
// library the hot-path configs use (tensor/src/matmul.rs:82-110, tensor/src/activation.rs:42-52,
// 90-101,309-318, tensor/src/reduce.rs:101-117,620-692, tensor/src/nn/norm.rs:92-111,
// tensor/src/transformer.rs:12-137).
//
// Ops build a lazy graph; nothing runs until realize().  realize() splits the graph into
// kernels, obtains each kernel through the kernel cache (render -> compile -> load, or a
// hand-written kernel), assembles an ExecutionPlan and executes it on the device stream.
//
// Scheduling rules (a reduced restatement of rangeify + kernel split):
//   - a reduce is a kernel boundary; the elementwise expression feeding it is fused into it;
//   - everything else is recomputed inside its consumers (softmax = 3 kernels, as upstream,
//     tensor/src/test/unit/fusion.rs:83-88), except tensors explicitly made contiguous;
//   - movement ops (reshape / permute / expand / shrink) never copy: they become index
//     arithmetic in the consuming kernel;
//   - with fusion enabled, the composed graphs of softmax, matmul and scaled-dot-product
//     attention are recognised by the hint their builder attached and replaced by the
//     hand-written gfx950 kernels when dtype and layout qualify.
// Numerics: half / bfloat16 elementwise chains are evaluated in f32 and rounded once at the
// kernel output (or at an explicit cast); reductions of half types accumulate in f32
// (reduce.rs:101-117).
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "buffer.h"
#include "uop.h"

namespace mrk {

enum class TKind : uint8_t {
    Buffer, Const, Unary, Binary, Where, Cast, Reduce, Reshape, Permute, Expand, Shrink, Iota, Cat, Gather, Contiguous, Copy,
};

// Device id of data that lives in host memory (DeviceSpec::Cpu); HIP devices are 0, 1, ...
constexpr int kCpuDevice = -1;

enum class HintKind : uint8_t { None, Softmax, Matmul, Sdpa, Swish, Rope };

struct TensorNode;
using TensorRef = std::shared_ptr<TensorNode>;

struct TensorNode {
    TKind kind = TKind::Buffer;
    Scalar dtype = Scalar::Float32;
    std::vector<int64_t> shape;
    std::vector<TensorRef> src;
    uint16_t sub = 0;           // UnaryOp / BinaryOp / ReduceOp
    std::vector<int64_t> arg;   // reduce axes | permutation | shrink begins | cat axis | iota axis
    double cval = 0.0;          // constant value
    int device_id = 0;
    std::shared_ptr<Buffer> buffer;  // set once the node is materialised (row-major contiguous)
    // Host-resident bytes of a CPU tensor (device_id == kCpuDevice): the data of a tensor created
    // from a slice, or the destination of a device -> CPU copy.  host_from is the device whose
    // stream must be synchronized before the bytes of such a copy are read (kCpuDevice: none).
    std::shared_ptr<std::vector<uint8_t>> host;
    int host_from = kCpuDevice;
    // fused-kernel hint: the node is the root of a composed graph a hand-written kernel covers
    HintKind hint = HintKind::None;
    std::vector<TensorRef> hint_inputs;
    double hint_scale = 0.0;
    bool hint_causal = false;
    double hint_softcap = 0.0;  // Sdpa: 0 = none; hint_inputs[3] is the attn_mask when there is one

    int64_t numel() const {
        int64_t n = 1;
        for (int64_t d : shape) n *= d;
        return n;
    }
};

// What the last realize() on this thread did (Tensor::kernels(), tensor/src/lib.rs:213).
struct RealizeStats {
    std::vector<std::string> kernel_names;
    std::vector<std::string> kernel_sources;  // rendered HIP C; empty for hand-written kernels
    size_t cached_kernels = 0;
    size_t buffers_reused = 0;  // memory planner (tensor/src/memory_planner.rs:84-96)
    size_t memory_saved = 0;
    size_t intermediate_bytes = 0;  // device bytes the plan's intermediates occupy
    size_t beam_candidates = 0;  // generated-kernel candidates compiled and timed (MOROK_BEAM)
    size_t beam_cache_hits = 0;  // generated kernels whose choices came from the on-disk cache
    double elapsed_ms = 0.0;
};

class Tensor {
  public:
    Tensor() = default;
    explicit Tensor(TensorRef n) : n_(std::move(n)) {}
    bool valid() const { return n_ != nullptr; }
    const TensorRef& node() const { return n_; }
    const std::vector<int64_t>& shape() const { return n_->shape; }
    Scalar dtype() const { return n_->dtype; }
    int64_t ndim() const { return static_cast<int64_t>(n_->shape.size()); }

    // ---- creation (tensor/src/data.rs:23-96)
    static Tensor from_raw_bytes(int device_id, const void* data, size_t nbytes, const std::vector<int64_t>& shape,
                                 Scalar dtype);
    static Tensor from_buffer(std::shared_ptr<Buffer> buf, const std::vector<int64_t>& shape, Scalar dtype);
    // Tensor::from_slice / from_raw_bytes without a device (data.rs:27-36,81-96): the bytes stay in
    // host memory; nothing touches a GPU until the tensor is moved with to() and realized.
    static Tensor from_host_bytes(const void* data, size_t nbytes, const std::vector<int64_t>& shape, Scalar dtype);
    // Tensor::to (lib.rs:479-486): same device -> the same tensor; otherwise a lazy COPY node, which
    // realization turns into a copy item of the execution plan (realize.rs:1002-1011).
    Tensor to(int device_id) const;
    int device() const { return n_ ? n_->device_id : 0; }  // lib.rs:464-466; kCpuDevice for host data
    static Tensor const_(double value, Scalar dtype, int device_id = 0);                           // lib.rs:432
    static Tensor full(const std::vector<int64_t>& shape, double value, Scalar dtype, int device_id = 0);  // lib.rs:251

    // ---- movement
    Tensor try_reshape(const std::vector<int64_t>& shape) const;  // one -1 allowed
    Tensor try_permute(const std::vector<int64_t>& perm) const;
    Tensor try_transpose(int64_t a, int64_t b) const;
    Tensor try_expand(const std::vector<int64_t>& shape) const;   // -1 keeps a dim
    Tensor try_shrink(const std::vector<int64_t>& begin, const std::vector<int64_t>& end) const;
    Tensor try_unsqueeze(int64_t axis) const;
    Tensor try_squeeze(int64_t axis) const;
    Tensor contiguous() const;  // lib.rs:548
    static Tensor cat(const std::vector<Tensor>& parts, int64_t axis);

    // ---- elementwise
    Tensor cast(Scalar dtype) const;  // lib.rs:495
    Tensor unary(UnaryOp op) const;
    Tensor binary(BinaryOp op, const Tensor& other) const;  // broadcasting + dtype promotion
    Tensor where_(const Tensor& cond, const Tensor& other) const;  // cond ? self : other
    Tensor try_add(const Tensor& o) const { return binary(BinaryOp::Add, o); }
    Tensor try_sub(const Tensor& o) const { return binary(BinaryOp::Sub, o); }
    Tensor try_mul(const Tensor& o) const { return binary(BinaryOp::Mul, o); }
    Tensor try_div(const Tensor& o) const { return binary(BinaryOp::Fdiv, o); }
    Tensor maximum(const Tensor& o) const { return binary(BinaryOp::Max, o); }
    Tensor try_exp() const { return unary(UnaryOp::Exp); }
    Tensor try_exp2() const { return unary(UnaryOp::Exp2); }
    Tensor try_rsqrt() const { return unary(UnaryOp::Rsqrt); }
    Tensor square() const { return unary(UnaryOp::Square); }
    Tensor sigmoid() const;  // activation.rs:42-52
    Tensor swish() const;    // activation.rs:309-313
    Tensor tanh() const;     // activation.rs:64-74
    Tensor silu() const { return swish(); }

    // ---- reductions (reduce.rs:620-692)
    Tensor reduce(ReduceOp op, std::vector<int64_t> axes, bool keepdim, bool promote) const;
    Tensor sum(int64_t axis, bool keepdim = false) const { return reduce(ReduceOp::Add, {axis}, keepdim, true); }
    Tensor max(int64_t axis, bool keepdim = false) const { return reduce(ReduceOp::Max, {axis}, keepdim, false); }
    Tensor mean(std::vector<int64_t> axes, bool keepdim) const;

    // ---- composite ops on the hot path
    // matmul.rs:82-110: 1-D x 1-D (scalar), 1-D x 2-D, 2-D x 1-D, 2-D x 2-D, batched with broadcast
    // batch axes.  `acc` other than Void: accumulate in and return that dtype (matmul_with().dtype()).
    Tensor matmul(const Tensor& other, Scalar acc = Scalar::Void) const;
    Tensor dot(const Tensor& other) const { return matmul(other); }              // matmul.rs:40-42
    // alpha * op(A) @ op(B) + beta * C  (matmul.rs:112-135); c may be null
    Tensor gemm(const Tensor& b, float alpha, float beta, bool trans_a, bool trans_b, const Tensor* c) const;
    // self @ weight^T + bias, weight [out, in] (a 1-D weight multiplies elementwise); matmul.rs:160-190
    Tensor linear(const Tensor& weight, const Tensor* bias, Scalar acc = Scalar::Void) const;
    Tensor softmax(int64_t axis) const;                                     // activation.rs:90-101
    Tensor log_softmax(int64_t axis) const;  // activation.rs:117-128
    Tensor logsumexp(int64_t axis) const;    // activation.rs:143-157
    Tensor rms_norm(int64_t axis, double eps) const;                        // nn/norm.rs:92-111
    Tensor embedding(const Tensor& indices) const;                          // transformer.rs:12-25
    Tensor apply_rotary_emb(const Tensor& cos, const Tensor& sin, bool interleaved) const;  // transformer.rs:32-69
    // transformer.rs:78-137.  scale <= 0: 1/sqrt(head_dim); attn_mask (optional): Bool (true =
    // attend) or additive, broadcastable to [.., Sq, Sk]; softcap > 0: cap * tanh(scores / cap).
    Tensor scaled_dot_product_attention(const Tensor& key, const Tensor& value, double scale, bool is_causal,
                                        const Tensor* attn_mask = nullptr, double softcap = 0.0) const;

    // ---- realization (realize.rs:83-127) and extraction (data.rs:211-236)
    int realize() const;
    // Schedules and compiles without executing (Tensor::prepare, realize.rs:299-357): the
    // returned plan can be executed any number of times; the tensor's buffer holds valid data
    // once the plan has run.
    int prepare(std::unique_ptr<class ExecutionPlan>* out) const;
    int to_bytes(void* dst, size_t nbytes) const;  // realize if needed, then copy out
    std::shared_ptr<Buffer> buffer() const;

  private:
    TensorRef n_;
};

// Per-thread switch: hand-written fused kernels on (default) or off (every op goes through
// generated kernels) - the counterpart of choosing a backend through PrepareConfig
// (tensor/src/config.rs:17-89).
void set_fusion_enabled(bool on);
bool fusion_enabled();
const RealizeStats& last_realize_stats();

size_t scalar_size(Scalar s);
// dtype/src/cast.rs:88
Scalar least_upper_dtype(Scalar a, Scalar b);

}  // namespace mrk
