// The device boundary: ProgramSpec / CompiledSpec / Program / Compiler / Renderer /
// RuntimeFactory / Device and the two registries, mirroring
// device/src/device.rs:34-60,72-133,142-177,186-222,234,255-313,327-410,
// device/src/registry.rs:26-141 and runtime/src/device_registry.rs:27-127.
#pragma once
#include <array>
#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "allocator.h"

namespace mrk {

struct LinearKernel;  // renderer input: the linearized UOp stream (see uop.h)

// device/src/device.rs:420-436
struct Variable {
    std::string name;
    int64_t min = 0;
    int64_t max = 0;
};

// device/src/device.rs:327-367.  Launch-dimension convention of this backend:
// global_size = grid extent in workgroups, local_size = workgroup extent in work-items
// (the `gidx`/`lidx` extents produced by schedule/src/gpudims.rs:153-156).
struct ProgramSpec {
    std::string name;
    std::string src;
    int device_id = 0;
    uint64_t ast_hash = 0;
    bool has_sizes = false;
    std::array<size_t, 3> global_size{1, 1, 1};
    std::array<size_t, 3> local_size{1, 1, 1};
    std::vector<Variable> vars;
    std::vector<std::string> var_names;
    std::vector<uint8_t> var_is_i64;  // rendered C type of each scalar argument
    std::vector<size_t> globals, outs, ins;
    size_t buf_count = 0;
};

// device/src/device.rs:72-133.  This is an AOT backend: `bytes` holds the gfx950 code
// object and `has_src` is false after compile().
struct CompiledSpec {
    std::string name;
    bool has_src = false;
    std::string src;
    std::vector<uint8_t> bytes;
    uint64_t ast_hash = 0;
    std::vector<std::string> var_names;
    std::vector<uint8_t> var_is_i64;
    bool has_sizes = false;
    std::array<size_t, 3> global_size{1, 1, 1};
    std::array<size_t, 3> local_size{1, 1, 1};
    size_t buf_count = 0;
};

// device/src/device.rs:34-60.  Implementations are thread-safe: kernels are shared
// across threads by the kernel cache (runtime/src/kernel_cache.rs:46-50).
class Program {
  public:
    virtual ~Program() = default;
    // buffers then vals, positional; vals order = var_names.  global/local may be null:
    // then the sizes recorded at compile time are used.
    virtual int execute(void* const* buffers, size_t nbufs, const int64_t* vals, size_t nvals, const size_t* global,
                        const size_t* local) = 0;
    // The same launch on another stream of the same device (hardware queues own their streams).
    virtual int execute_on(ffi::Stream stream, void* const* buffers, size_t nbufs, const int64_t* vals, size_t nvals,
                           const size_t* global, const size_t* local) = 0;
    virtual const char* name() const = 0;
    // false for items that are not kernel launches (COPY items between host and device memory):
    // they are not recorded into HIP graphs.
    virtual bool capturable() const { return true; }
};

class Compiler {
  public:
    virtual ~Compiler() = default;
    virtual int compile(const ProgramSpec& spec, CompiledSpec* out) = 0;
    virtual const char* cache_key() const = 0;
};

class Renderer {
  public:
    virtual ~Renderer() = default;
    virtual int render(const LinearKernel& kernel, const char* name, ProgramSpec* out) = 0;
    virtual int device_id() const = 0;
};

using RuntimeFactory = std::function<int(const CompiledSpec&, std::unique_ptr<Program>*)>;

// device/src/device.rs:255-313
struct Device {
    int device_id = 0;
    std::shared_ptr<Allocator> allocator;
    std::shared_ptr<Renderer> renderer;
    std::shared_ptr<Compiler> compiler;
    RuntimeFactory runtime;
    static const char* base_device_key() { return "HIP"; }
};

// Parses "HIP", "hip:1", "AMD:0", "GPU" ... -> device id (device/src/registry.rs:26-81 with
// a HIP arm).  Other device strings -> kInvalidDevice.
int parse_device_spec(const char* spec, int* device_id);

// device/src/registry.rs:84-141: one cached LRU-wrapped allocator per device id.
class AllocatorRegistry {
  public:
    static AllocatorRegistry& global();
    int get(int device_id, std::shared_ptr<Allocator>* out);
    // Drops all cached allocators (tests only; outstanding buffers keep theirs alive).
    void reset();

  private:
    std::mutex mu_;
    std::unordered_map<int, std::shared_ptr<Allocator>> devices_;
};

// runtime/src/device_registry.rs:27-127: factories keyed by base device type; devices are
// created once per spec under a double-checked lock.
using DeviceFactory = std::function<int(int device_id, AllocatorRegistry&, std::shared_ptr<Device>*)>;
class DeviceFactoryRegistry {
  public:
    static DeviceFactoryRegistry& global();
    void register_factory(const std::string& device_type, DeviceFactory f);
    int device(const std::string& device_type, int device_id, std::shared_ptr<Device>* out);
    // lookup only: null when the device has not been created yet (creates and allocates nothing)
    std::shared_ptr<Device> find(const std::string& device_type, int device_id);
    void reset();

  private:
    DeviceFactoryRegistry();
    std::mutex mu_;
    std::unordered_map<std::string, DeviceFactory> factories_;
    std::unordered_map<std::string, std::shared_ptr<Device>> devices_;
};

// The HIP factory registered under "HIP" (the pattern of runtime/src/devices/cpu.rs:434-464).
int create_hip_device(int device_id, AllocatorRegistry& registry, std::shared_ptr<Device>* out);

// hiprtc in-process compiler (replaces the clang subprocess of runtime/src/jit_loader.rs:131-164).
std::shared_ptr<Compiler> make_hiprtc_compiler();
// HIP-C renderer for linearized UOp kernels (see renderer.cpp).
std::shared_ptr<Renderer> make_hip_renderer(int device_id);
// hipModuleLoadData + hipModuleGetFunction (replaces the ELF loader, jit_loader.rs:171-323).
int create_module_program(int device_id, ffi::Stream stream, const CompiledSpec& spec, std::unique_ptr<Program>* out);

}  // namespace mrk
