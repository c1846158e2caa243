// Program backed by a loaded code object: hipModuleLoadData + hipModuleGetFunction at
// creation, hipModuleLaunchKernel per execute.  Replaces the ELF loader + libffi call of
// the CPU backend (runtime/src/jit_loader.rs:171-323, runtime/src/dispatch.rs:45-80) behind
// the same `Program::execute(buffers, vals, global, local)` signature
// (device/src/device.rs:50-56).  Argument order: buffer pointers, then scalar variables in
// var_names order, each narrowed to its rendered C type (cf. codegen/src/c/mod.rs:154-160).
#include <cstring>

#include "device.h"
#include "error.h"

namespace mrk {

namespace {

class ModuleProgram final : public Program {
  public:
    ModuleProgram(int device_id, ffi::Stream stream, ffi::Module m, ffi::Function f, const CompiledSpec& spec)
        : device_id_(device_id),
          stream_(stream),
          module_(m),
          function_(f),
          name_(spec.name),
          buf_count_(spec.buf_count),
          var_is_i64_(spec.var_is_i64),
          nvars_(spec.var_names.size()),
          has_sizes_(spec.has_sizes),
          global_(spec.global_size),
          local_(spec.local_size) {}
    ~ModuleProgram() override {
        ffi::set_device(device_id_);
        ffi::stream_synchronize(stream_);
        ffi::module_unload(module_);
    }

    int execute(void* const* buffers, size_t nbufs, const int64_t* vals, size_t nvals, const size_t* global,
                const size_t* local) override {
        return execute_on(stream_, buffers, nbufs, vals, nvals, global, local);
    }
    int execute_on(ffi::Stream stream, void* const* buffers, size_t nbufs, const int64_t* vals, size_t nvals,
                   const size_t* global, const size_t* local) override {
        if (nbufs != buf_count_)
            return failf(kInvalidArgument, "kernel '%s' expects %zu buffers, got %zu", name_.c_str(), buf_count_, nbufs);
        if (nvals != nvars_)
            return failf(kInvalidArgument, "kernel '%s' expects %zu variable values, got %zu", name_.c_str(), nvars_,
                         nvals);
        const size_t* g = global ? global : (has_sizes_ ? global_.data() : nullptr);
        const size_t* l = local ? local : (has_sizes_ ? local_.data() : nullptr);
        if (!g || !l) return failf(kInvalidArgument, "kernel '%s' launched without global/local sizes", name_.c_str());
        unsigned grid[3], block[3];
        size_t threads = 1;
        for (int i = 0; i < 3; i++) {
            if (g[i] == 0 || l[i] == 0) return kOk;  // empty launch: nothing to do
            if (g[i] > 0x7fffffffull || l[i] > 1024)
                return failf(kInvalidArgument, "kernel '%s': launch dims out of range", name_.c_str());
            grid[i] = static_cast<unsigned>(g[i]);
            block[i] = static_cast<unsigned>(l[i]);
            threads *= l[i];
        }
        if (threads > 1024)
            return failf(kInvalidArgument, "kernel '%s': workgroup of %zu work-items exceeds 1024", name_.c_str(),
                         threads);
        if (grid[1] > 65535 || grid[2] > 65535)
            return failf(kInvalidArgument, "kernel '%s': grid y/z exceeds 65535", name_.c_str());
        // Local copies so that concurrent executes from several threads never share storage.
        std::vector<void*> ptr_store(buffers, buffers + nbufs);
        std::vector<int64_t> v64(nvals);
        std::vector<int32_t> v32(nvals);
        std::vector<void*> params(nbufs + nvals);
        for (size_t i = 0; i < nbufs; i++) params[i] = &ptr_store[i];
        for (size_t i = 0; i < nvals; i++) {
            if (i < var_is_i64_.size() && var_is_i64_[i]) {
                v64[i] = vals[i];
                params[nbufs + i] = &v64[i];
            } else {
                v32[i] = static_cast<int32_t>(vals[i]);
                params[nbufs + i] = &v32[i];
            }
        }
        MRK_HIP(ffi::set_device(device_id_), "hipSetDevice");
        MRK_HIP(ffi::module_launch(function_, grid, block, 0, stream, params.data()), "hipModuleLaunchKernel");
        return kOk;
    }
    const char* name() const override { return name_.c_str(); }

  private:
    int device_id_;
    ffi::Stream stream_;
    ffi::Module module_;
    ffi::Function function_;
    std::string name_;
    size_t buf_count_;
    std::vector<uint8_t> var_is_i64_;
    size_t nvars_;
    bool has_sizes_;
    std::array<size_t, 3> global_, local_;
};

}  // namespace

int create_module_program(int device_id, ffi::Stream stream, const CompiledSpec& spec, std::unique_ptr<Program>* out) {
    if (spec.bytes.empty())
        return failf(kRuntime, "runtime error: compiled spec for '%s' carries no code object bytes", spec.name.c_str());
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    ffi::Module m = nullptr;
    MRK_HIP(ffi::module_load_data(&m, spec.bytes.data()), "hipModuleLoadData");
    ffi::Function f = nullptr;
    int rc = ffi::module_get_function(&f, m, spec.name.c_str());
    if (rc != 0) {
        ffi::module_unload(m);
        ffi::clear_last_error();
        return failf(kHipError, "HIP error: hipModuleGetFunction failed for entry point '%s': %s (%d)", spec.name.c_str(),
                     ffi::error_name(rc), rc);
    }
    out->reset(new ModuleProgram(device_id, stream, m, f, spec));
    return kOk;
}

}  // namespace mrk
