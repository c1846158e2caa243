// In-process HIP-C -> gfx950 code object compiler.  Stands where the reference's CPU
// backend runs a clang subprocess (runtime/src/jit_loader.rs:131-164) behind the
// pass-through `Compiler` of runtime/src/devices/cpu.rs:178-195; being an AOT backend it
// fills CompiledSpec.bytes and leaves src empty (device/src/device.rs:118-120,153-169).
#include <hip/hiprtc.h>

#include <string>
#include <vector>

#include "device.h"
#include "error.h"

namespace mrk {

namespace {

class HiprtcCompiler final : public Compiler {
  public:
    int compile(const ProgramSpec& spec, CompiledSpec* out) override {
        hiprtcProgram prog = nullptr;
        hiprtcResult r = hiprtcCreateProgram(&prog, spec.src.c_str(), (spec.name + ".hip").c_str(), 0, nullptr, nullptr);
        if (r != HIPRTC_SUCCESS)
            return failf(kCompileError, "hiprtcCreateProgram failed: %s", hiprtcGetErrorString(r));
        // No fast-math: generated kernels must keep IEEE semantics for parity with the CPU
        // backend.  Packed-FP32 instruction selection is disabled for every kernel of this
        // runtime, generated or hand-written.
        const char* opts[] = {"--offload-arch=gfx950", "-O3",         "-std=c++17",       "-Xclang",
                              "-target-feature",       "-Xclang",     "-packed-fp32-ops", "-ffp-contract=off"};
        r = hiprtcCompileProgram(prog, sizeof(opts) / sizeof(opts[0]), opts);
        size_t log_size = 0;
        hiprtcGetProgramLogSize(prog, &log_size);
        std::string log(log_size, '\0');
        if (log_size) hiprtcGetProgramLog(prog, &log[0]);
        if (r != HIPRTC_SUCCESS) {
            hiprtcDestroyProgram(&prog);
            return failf(kCompileError, "hiprtc compile of kernel '%s' failed: %s\n%s", spec.name.c_str(),
                         hiprtcGetErrorString(r), log.c_str());
        }
        size_t code_size = 0;
        hiprtcGetCodeSize(prog, &code_size);
        out->bytes.resize(code_size);
        hiprtcGetCode(prog, reinterpret_cast<char*>(out->bytes.data()));
        hiprtcDestroyProgram(&prog);
        out->name = spec.name;
        out->has_src = false;
        out->src.clear();
        out->ast_hash = spec.ast_hash;
        out->var_names = spec.var_names;
        out->var_is_i64 = spec.var_is_i64;
        out->has_sizes = spec.has_sizes;
        out->global_size = spec.global_size;
        out->local_size = spec.local_size;
        out->buf_count = spec.buf_count;
        return kOk;
    }
    const char* cache_key() const override { return "hip-gfx950"; }
};

}  // namespace

std::shared_ptr<Compiler> make_hiprtc_compiler() { return std::make_shared<HiprtcCompiler>(); }

}  // namespace mrk
