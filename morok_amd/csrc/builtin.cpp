// Hand-written gfx950 kernels wrapped as Programs so that execution plans can hold them
// beside generated kernels (device/src/device.rs:34-60).  Buffer order follows the
// reference's PARAM numbering: outputs first, then inputs.
#include <cstring>

#include "builtin.h"
#include "error.h"
#include "kernels/kernels.h"

namespace mrk {

namespace {

class BuiltinProgram final : public Program {
  public:
    using Fn = std::function<int(ffi::Stream, void* const*, const std::vector<int64_t>&)>;
    BuiltinProgram(int device_id, ffi::Stream stream, std::string name, size_t nbufs, std::vector<int64_t> params, Fn fn)
        : device_id_(device_id),
          stream_(stream),
          name_(std::move(name)),
          nbufs_(nbufs),
          params_(std::move(params)),
          fn_(std::move(fn)) {}
    int execute(void* const* buffers, size_t nbufs, const int64_t* vals, size_t nvals, const size_t* global,
                const size_t* local) override {
        return execute_on(stream_, buffers, nbufs, vals, nvals, global, local);
    }
    int execute_on(ffi::Stream stream, void* const* buffers, size_t nbufs, const int64_t*, size_t nvals, const size_t*,
                   const size_t*) override {
        if (nbufs != nbufs_)
            return failf(kInvalidArgument, "kernel '%s' expects %zu buffers, got %zu", name_.c_str(), nbufs_, nbufs);
        if (nvals != 0)
            return failf(kInvalidArgument, "kernel '%s' takes no variable values, got %zu", name_.c_str(), nvals);
        for (size_t i = 0; i < nbufs; i++)
            if (!buffers[i]) return failf(kInvalidArgument, "kernel '%s': buffer %zu is null", name_.c_str(), i);
        MRK_HIP(ffi::set_device(device_id_), "hipSetDevice");
        int rc = fn_(stream, buffers, params_);
        if (rc != 0) return fail_hip(rc, name_.c_str());
        return kOk;
    }
    const char* name() const override { return name_.c_str(); }

  private:
    int device_id_;
    ffi::Stream stream_;
    std::string name_;
    size_t nbufs_;
    std::vector<int64_t> params_;
    Fn fn_;
};

class CopyProgram final : public Program {
  public:
    CopyProgram(int device_id, ffi::Stream stream, bool to_device, std::shared_ptr<std::vector<uint8_t>> host)
        : device_id_(device_id), stream_(stream), to_device_(to_device), host_(std::move(host)) {
        name_ = std::string(to_device ? "copy_h2d_" : "copy_d2h_") + std::to_string(host_->size());
    }
    int execute(void* const* buffers, size_t nbufs, const int64_t* vals, size_t nvals, const size_t* global,
                const size_t* local) override {
        return execute_on(stream_, buffers, nbufs, vals, nvals, global, local);
    }
    int execute_on(ffi::Stream stream, void* const* buffers, size_t nbufs, const int64_t*, size_t nvals, const size_t*,
                   const size_t*) override {
        if (nbufs != 1 || nvals != 0 || !buffers[0])
            return failf(kInvalidArgument, "copy item '%s' takes exactly one device buffer", name_.c_str());
        if (host_->empty()) return kOk;
        MRK_HIP(ffi::set_device(device_id_), "hipSetDevice");
        if (to_device_) MRK_HIP(ffi::memcpy_htod_async(buffers[0], host_->data(), host_->size(), stream), "hipMemcpyAsync(HtoD)");
        else MRK_HIP(ffi::memcpy_dtoh_async(host_->data(), buffers[0], host_->size(), stream), "hipMemcpyAsync(DtoH)");
        return kOk;
    }
    const char* name() const override { return name_.c_str(); }
    bool capturable() const override { return false; }

  private:
    int device_id_;
    ffi::Stream stream_;
    bool to_device_;
    std::shared_ptr<std::vector<uint8_t>> host_;
    std::string name_;
};

}  // namespace

int create_copy_program(int device_id, ffi::Stream stream, bool to_device, std::shared_ptr<std::vector<uint8_t>> host,
                        std::unique_ptr<Program>* out) {
    if (!host) return fail(kInvalidArgument, "copy item: no host memory");
    out->reset(new CopyProgram(device_id, stream, to_device, std::move(host)));
    return kOk;
}

int create_builtin_program(int device_id, ffi::Stream stream, const char* kind, const int64_t* params, size_t nparams,
                           std::unique_ptr<Program>* out) {
    std::vector<int64_t> p(params, params + nparams);
    std::string k(kind ? kind : "");
    auto need = [&](size_t n) -> int {
        if (nparams != n)
            return failf(kInvalidArgument, "builtin '%s' takes %zu parameters, got %zu", k.c_str(), n, nparams);
        return kOk;
    };
    if (k == "softmax_f32") {
        MRK_TRY(need(2));
        if (p[0] < 0 || p[1] < 0) return fail(kInvalidArgument, "softmax_f32: negative shape");
        std::string name = "softmax_f32_" + std::to_string(p[0]) + "_" + std::to_string(p[1]);
        out->reset(new BuiltinProgram(device_id, stream, name, 2, p,
                                      [](ffi::Stream s, void* const* b, const std::vector<int64_t>& q) {
                                          return launch_softmax_f32(s, b[1], b[0], q[0], q[1], 0);
                                      }));
        return kOk;
    }
    // "gemm_f16" / "gemm_f16_nt": the same kernels on IEEE half precision operands and result
    if (k == "gemm_bf16" || k == "gemm_f16") {  // {M, N, K}, {M, N, K, batch} or {M, N, K, batch, workspace bytes}
        const bool f16 = k == "gemm_f16";
        if (nparams < 3 || nparams > 5)
            return failf(kInvalidArgument, "builtin '%s' takes 3 to 5 parameters, got %zu", k.c_str(), nparams);
        while (p.size() < 4) p.push_back(1);
        if (p.size() < 5) p.push_back(0);
        if (p[0] < 0 || p[1] < 0 || p[2] < 0 || p[3] < 1 || p[3] > 65535 || p[4] < 0)
            return fail(kInvalidArgument, k + ": bad shape (M, N, K >= 0, 1 <= batch <= 65535, workspace >= 0)");
        std::string name = k + "_" + std::to_string(p[0]) + "_" + std::to_string(p[1]) + "_" + std::to_string(p[2]);
        if (p[3] > 1) name += "_x" + std::to_string(p[3]);
        if (p[4] > 0) {  // a fourth buffer of p[4] bytes: scratch for the split-K partial results
            out->reset(new BuiltinProgram(device_id, stream, name + "_splitk", 4, p,
                                          [f16](ffi::Stream s, void* const* b, const std::vector<int64_t>& q) {
                                              return launch_gemm_bf16(s, b[1], b[2], b[0], q[0], q[1], q[2], 0, q[3], b[3],
                                                                      static_cast<size_t>(q[4]), false, f16);
                                          }));
            return kOk;
        }
        out->reset(new BuiltinProgram(device_id, stream, name, 3, p,
                                      [f16](ffi::Stream s, void* const* b, const std::vector<int64_t>& q) {
                                          return launch_gemm_bf16(s, b[1], b[2], b[0], q[0], q[1], q[2], 0, q[3], nullptr, 0, false, f16);
                                      }));
        return kOk;
    }
    // the "_nt" kinds take the second operand as B^T [N, K] (a Linear layer's weight as it is stored)
    if (k == "gemm_bf16_nt" || k == "gemm_f16_nt") {  // {M, N, K}, {M, N, K, batch} or {M, N, K, batch, workspace bytes}; buffers {c, a, bt[, scratch]}
        const bool f16 = k == "gemm_f16_nt";
        if (nparams < 3 || nparams > 5)
            return failf(kInvalidArgument, "builtin '%s' takes 3 to 5 parameters, got %zu", k.c_str(), nparams);
        while (p.size() < 4) p.push_back(1);
        if (p.size() < 5) p.push_back(0);
        if (p[4] < 0) return fail(kInvalidArgument, k + ": negative workspace size");
        if (!gemm_bf16_nt_supported(p[0], p[1], p[2], p[3]))
            return fail(kInvalidArgument, k + ": shape not covered (K a multiple of 8; at most 64 rows, or N a multiple of 8)");
        std::string name = k + "_" + std::to_string(p[0]) + "_" + std::to_string(p[1]) + "_" + std::to_string(p[2]);
        if (p[3] > 1) name += "_x" + std::to_string(p[3]);
        if (p[4] > 0) {  // a fourth buffer of p[4] bytes: scratch for the split-K partial results
            out->reset(new BuiltinProgram(device_id, stream, name + "_splitk", 4, p,
                                          [f16](ffi::Stream s, void* const* b, const std::vector<int64_t>& q) {
                                              return launch_gemm_bf16(s, b[1], b[2], b[0], q[0], q[1], q[2], 0, q[3], b[3],
                                                                      static_cast<size_t>(q[4]), true, f16);
                                          }));
            return kOk;
        }
        out->reset(new BuiltinProgram(device_id, stream, name, 3, p,
                                      [f16](ffi::Stream s, void* const* b, const std::vector<int64_t>& q) {
                                          return launch_gemm_bf16(s, b[1], b[2], b[0], q[0], q[1], q[2], 0, q[3], nullptr, 0, true, f16);
                                      }));
        return kOk;
    }
    // c = a b + r in the product's own kernels: r a matrix of c's shape ("_residual") or one row [N] ("_bias");
    // {M, N, K}, {M, N, K, batch} or {M, N, K, batch, workspace bytes}; buffers {c, a, b, r[, scratch]}
    if (k == "gemm_bf16_bias" || k == "gemm_bf16_nt_bias" || k == "gemm_bf16_residual" || k == "gemm_bf16_nt_residual") {
        const bool nt = k.find("_nt_") != std::string::npos, row = k.find("_bias") != std::string::npos;
        if (nparams < 3 || nparams > 5)
            return failf(kInvalidArgument, "builtin '%s' takes 3 to 5 parameters, got %zu", k.c_str(), nparams);
        while (p.size() < 4) p.push_back(1);
        if (p.size() < 5) p.push_back(0);
        if (p[4] < 0) return fail(kInvalidArgument, k + ": negative workspace size");
        if (!gemm_bf16_bias_launchable(p[0], p[1], p[2], p[3], nt))
            return failf(kInvalidArgument, "%s: shape not covered (N and K multiples of 8%s)", k.c_str(),
                         nt ? "; or up to 64 rows with K a multiple of 8" : "");
        std::string name = k + "_" + std::to_string(p[0]) + "_" + std::to_string(p[1]) + "_" + std::to_string(p[2]);
        if (p[3] > 1) name += "_x" + std::to_string(p[3]);
        if (p[4] > 0) {  // a fifth buffer of p[4] bytes: scratch for the partial results of a product spread along K
            out->reset(new BuiltinProgram(device_id, stream, name + "_splitk", 5, p,
                                          [nt, row](ffi::Stream s, void* const* b, const std::vector<int64_t>& q) {
                                              return launch_gemm_bf16_residual(s, b[1], b[2], b[3], b[0], q[0], q[1], q[2], q[3], nt, row, b[4],
                                                                               static_cast<size_t>(q[4]));
                                          }));
            return kOk;
        }
        out->reset(new BuiltinProgram(device_id, stream, name, 4, p,
                                      [nt, row](ffi::Stream s, void* const* b, const std::vector<int64_t>& q) {
                                          return launch_gemm_bf16_residual(s, b[1], b[2], b[3], b[0], q[0], q[1], q[2], q[3], nt, row);
                                      }));
        return kOk;
    }
    if (k == "gemm_bf16_swiglu" || k == "gemm_bf16_nt_swiglu") {  // {M, F, K}; buffers {c [M, F], a [M, K], w [K, 2F] = gate | up ([2F, K]: _nt)}
        const bool nt = k == "gemm_bf16_nt_swiglu";
        MRK_TRY(need(3));
        if (!gemm_bf16_swiglu_supported(p[0], p[1], p[2], nt))
            return failf(kInvalidArgument, "%s: shape not covered (M, F, K > 0; F and K multiples of 8)", k.c_str());
        std::string name = k + "_" + std::to_string(p[0]) + "_" + std::to_string(p[1]) + "_" + std::to_string(p[2]);
        out->reset(new BuiltinProgram(device_id, stream, name, 3, p,
                                      [nt](ffi::Stream s, void* const* b, const std::vector<int64_t>& q) {
                                          return launch_gemm_bf16_swiglu(s, b[1], b[2], b[0], q[0], q[1], q[2], nt);
                                      }));
        return kOk;
    }
    if (k == "gemm_bf16_rope" || k == "gemm_bf16_nt_rope") {
        const bool nt = k == "gemm_bf16_nt_rope";  // (b stored [N, K])
        // {M, N, K, split, seq}; buffers {c_rot [M, split], a [M, K], b [K, N], c_rest [M, N - split], cos [seq, 64] f32, sin}:
        // the product with the rotary embedding of its first `split` columns (heads of 128) in the epilogue
        MRK_TRY(need(5));
        if (!gemm_bf16_rope_supported(p[0], p[1], p[2], p[3], p[4]))
            return fail(kInvalidArgument, k + ": shape not covered (K a multiple of 64, N of 8, split a multiple of 256 within N, seq > 0)");
        std::string name = k + "_" + std::to_string(p[0]) + "_" + std::to_string(p[1]) + "_" + std::to_string(p[2]) + "_s" + std::to_string(p[3]);
        out->reset(new BuiltinProgram(device_id, stream, name, 6, p,
                                      [nt](ffi::Stream s, void* const* b, const std::vector<int64_t>& q) {
                                          return launch_gemm_bf16_rope(s, b[1], b[2], b[0], b[3], q[0], q[1], q[2], q[3], b[4], b[5], q[4], nt);
                                      }));
        return kOk;
    }
    if (k == "flash_fwd_bf16") {  // {BH, Sq, Sk, D, causal, scale bits[, workspace bytes]}; buffers {o, q, k, v[, scratch]}
        if (nparams != 6 && nparams != 7)
            return failf(kInvalidArgument, "builtin '%s' takes 6 or 7 parameters, got %zu", k.c_str(), nparams);
        if (p.size() < 7) p.push_back(0);
        if (p[6] < 0) return fail(kInvalidArgument, "flash_fwd_bf16: negative workspace size");
        if (p[0] < 0 || p[1] < 0 || p[2] <= 0 || (p[3] != 256 && p[3] != 128 && p[3] != 64))
            return fail(kInvalidArgument, "flash_fwd_bf16: bad shape (params BH, Sq, Sk, D = 256, 128 or 64, causal, scale bits)");
        std::string name = "flash_fwd_bf16_" + std::to_string(p[0]) + "_" + std::to_string(p[1]) + "_" + std::to_string(p[2]) + (p[3] != 128 ? "_d" + std::to_string(p[3]) : "");
        // a fifth buffer of p[6] bytes: scratch for the partial results of a key sequence split over workgroups
        const bool ws = p[6] > 0;
        out->reset(new BuiltinProgram(device_id, stream, name + (ws ? "_splitkv" : ""), ws ? 5 : 4, p,
                                      [ws](ffi::Stream s, void* const* b, const std::vector<int64_t>& q) {
                                          uint32_t bits = static_cast<uint32_t>(q[5]);
                                          float scale;
                                          std::memcpy(&scale, &bits, 4);
                                          return launch_flash_fwd_bf16(s, b[1], b[2], b[3], b[0], q[0], q[1], q[2], q[3],
                                                                       scale, q[4] != 0, ws ? b[4] : nullptr, ws ? static_cast<size_t>(q[6]) : 0);
                                      }));
        return kOk;
    }
    if (k == "flash_fwd_bf16_strided") {
        // params: B, H, Sq, Sk, D, causal, scale bits, element offsets of q k v o into their
        // buffers (4), then (batch, head, row) element strides of q k v o (12)
        // optionally a 24th: workspace bytes, with a fifth buffer of that size (scratch for a split key sequence)
        if (nparams != 23 && nparams != 24)
            return failf(kInvalidArgument, "builtin '%s' takes 23 or 24 parameters, got %zu", k.c_str(), nparams);
        if (p.size() < 24) p.push_back(0);
        if (p[23] < 0) return fail(kInvalidArgument, "flash_fwd_bf16_strided: negative workspace size");
        if (p[0] < 0 || p[1] < 0 || p[2] < 0 || p[3] <= 0 || (p[4] != 256 && p[4] != 128 && p[4] != 64))
            return fail(kInvalidArgument, "flash_fwd_bf16_strided: bad shape (params B, H, Sq, Sk, D = 256, 128 or 64, causal, scale bits, 4 offsets, 12 strides)");
        for (int i = 7; i < 23; i++)
            if (p[i] < 0 || p[i] % 8) return fail(kInvalidArgument, "flash_fwd_bf16_strided: offsets and strides must be non-negative multiples of 8 elements");
        std::string name = "flash_fwd_bf16_strided_" + std::to_string(p[0] * p[1]) + "_" + std::to_string(p[2]) + "_" + std::to_string(p[3]) + (p[4] != 128 ? "_d" + std::to_string(p[4]) : "");
        const bool ws = p[23] > 0;
        out->reset(new BuiltinProgram(device_id, stream, name + (ws ? "_splitkv" : ""), ws ? 5 : 4, p,
                                      [ws](ffi::Stream s, void* const* b, const std::vector<int64_t>& q) {
                                          uint32_t bits = static_cast<uint32_t>(q[6]);
                                          float scale;
                                          std::memcpy(&scale, &bits, 4);
                                          long strides[12];
                                          for (int i = 0; i < 12; i++) strides[i] = static_cast<long>(q[11 + i]);
                                          auto at = [&](int buf, int which) {
                                              return static_cast<char*>(b[buf]) + q[7 + which] * 2;
                                          };
                                          return launch_flash_fwd_bf16_strided(s, at(1, 0), at(2, 1), at(3, 2), at(0, 3), q[0], q[1],
                                                                               q[2], q[3], q[4], scale, q[5] != 0, strides, ws ? b[4] : nullptr,
                                                                               ws ? static_cast<size_t>(q[23]) : 0);
                                      }));
        return kOk;
    }
    if (k == "flash_fwd_bf16_ext") {
        // attn_mask / softcap (tensor/src/transformer.rs:112-132).  params: B, H, Sq, Sk, D, causal, scale bits,
        // softcap bits (0 = none), mask kind (0 none, 1 Bool bytes, 2 additive bf16), element offsets of
        // q k v o mask into their buffers (5), (batch, head, row) element strides of q k v o (12) and of
        // the mask (3).  buffers {o, q, k, v, mask}; without a mask the fifth buffer is not read.
        // optionally a 30th: workspace bytes, with a sixth buffer of that size (scratch for a split key sequence)
        if (nparams != 29 && nparams != 30)
            return failf(kInvalidArgument, "builtin '%s' takes 29 or 30 parameters, got %zu", k.c_str(), nparams);
        if (p.size() < 30) p.push_back(0);
        if (p[29] < 0) return fail(kInvalidArgument, "flash_fwd_bf16_ext: negative workspace size");
        if (p[0] < 0 || p[1] < 0 || p[2] < 0 || p[3] <= 0 || (p[4] != 256 && p[4] != 128 && p[4] != 64) || p[8] < 0 || p[8] > 2)
            return fail(kInvalidArgument, "flash_fwd_bf16_ext: bad shape (params B, H, Sq, Sk, D = 256, 128 or 64, causal, scale bits, "
                                          "softcap bits, mask kind 0..2, 5 offsets, 12 strides, 3 mask strides)");
        for (int i = 9; i < 26; i++)
            if (p[i] < 0 || (i != 13 && p[i] % 8)) return fail(kInvalidArgument, "flash_fwd_bf16_ext: offsets and strides must be non-negative multiples of 8 elements");
        for (int i = 26; i < 29; i++)
            if (p[i] < 0 || p[i] % 4) return fail(kInvalidArgument, "flash_fwd_bf16_ext: mask strides must be non-negative multiples of 4 elements");
        if (p[8] != 0 && (p[3] % 4 || p[13] % 4)) return fail(kInvalidArgument, "flash_fwd_bf16_ext: with a mask, Sk and the mask offset must be multiples of 4");
        std::string name = std::string("flash_fwd_bf16_ext") + (p[8] == 1 ? "_bool" : p[8] == 2 ? "_add" : "") + (p[7] ? "_cap" : "") + "_" +
                           std::to_string(p[0] * p[1]) + "_" + std::to_string(p[2]) + "_" + std::to_string(p[3]) + (p[4] != 128 ? "_d" + std::to_string(p[4]) : "");
        const bool ws = p[29] > 0;
        out->reset(new BuiltinProgram(device_id, stream, name + (ws ? "_splitkv" : ""), ws ? 6 : 5, p,
                                      [ws](ffi::Stream s, void* const* b, const std::vector<int64_t>& q) {
                                          uint32_t bits = static_cast<uint32_t>(q[6]), cbits = static_cast<uint32_t>(q[7]);
                                          float scale, cap;
                                          std::memcpy(&scale, &bits, 4);
                                          std::memcpy(&cap, &cbits, 4);
                                          long strides[12], mstrides[3];
                                          for (int i = 0; i < 12; i++) strides[i] = static_cast<long>(q[14 + i]);
                                          for (int i = 0; i < 3; i++) mstrides[i] = static_cast<long>(q[26 + i]);
                                          auto at = [&](int buf, int which) { return static_cast<char*>(b[buf]) + q[9 + which] * 2; };
                                          const int kind = static_cast<int>(q[8]);
                                          const void* mask = kind ? static_cast<char*>(b[4]) + q[13] * (kind == 2 ? 2 : 1) : nullptr;
                                          return launch_flash_fwd_bf16_ext(s, at(1, 0), at(2, 1), at(3, 2), at(0, 3), q[0], q[1], q[2], q[3], q[4],
                                                                           scale, q[5] != 0, strides, mask, kind, mstrides, cap, ws ? b[5] : nullptr,
                                                                           ws ? static_cast<size_t>(q[29]) : 0);
                                      }));
        return kOk;
    }
    return fail(kInvalidArgument, "unknown builtin kernel kind: " + k);
}

}  // namespace mrk
