#include "device.h"
#include "kernels/kernels.h"

#include <algorithm>
#include <cctype>
#include <cstdlib>

#include "error.h"

namespace mrk {

int parse_device_spec(const char* spec, int* device_id) {
    if (!spec) return fail(kInvalidDevice, "invalid device: (null)");
    std::string s(spec);
    std::transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return std::toupper(c); });
    std::string base = s, idx;
    size_t colon = s.find(':');
    if (colon != std::string::npos) {
        base = s.substr(0, colon);
        idx = s.substr(colon + 1);
    }
    if (base != "HIP" && base != "AMD" && base != "GPU") return fail(kInvalidDevice, "invalid device: " + s);
    int id = 0;
    if (colon != std::string::npos) {
        if (idx.empty() || !std::all_of(idx.begin(), idx.end(), [](unsigned char c) { return std::isdigit(c); }))
            return fail(kInvalidDevice, "invalid device: " + s);
        id = std::atoi(idx.c_str());
    }
    *device_id = id;
    return kOk;
}

AllocatorRegistry& AllocatorRegistry::global() {
    static AllocatorRegistry* r = new AllocatorRegistry();  // never destroyed: outlives static dtors
    return *r;
}

int AllocatorRegistry::get(int device_id, std::shared_ptr<Allocator>* out) {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = devices_.find(device_id);
    if (it != devices_.end()) {
        *out = it->second;
        return kOk;
    }
    std::unique_ptr<HipAllocator> base;
    MRK_TRY(HipAllocator::create(device_id, &base));
    std::shared_ptr<Allocator> lru = std::make_shared<LruAllocator>(std::move(base));
    devices_[device_id] = lru;
    *out = lru;
    return kOk;
}

void AllocatorRegistry::reset() {
    std::lock_guard<std::mutex> lock(mu_);
    devices_.clear();
}

DeviceFactoryRegistry::DeviceFactoryRegistry() { factories_["HIP"] = create_hip_device; }

DeviceFactoryRegistry& DeviceFactoryRegistry::global() {
    static DeviceFactoryRegistry* r = new DeviceFactoryRegistry();
    return *r;
}

void DeviceFactoryRegistry::register_factory(const std::string& device_type, DeviceFactory f) {
    std::lock_guard<std::mutex> lock(mu_);
    factories_[device_type] = std::move(f);
}

int DeviceFactoryRegistry::device(const std::string& device_type, int device_id, std::shared_ptr<Device>* out) {
    std::string key = device_type + ":" + std::to_string(device_id);
    std::lock_guard<std::mutex> lock(mu_);
    auto it = devices_.find(key);
    if (it != devices_.end()) {
        *out = it->second;
        return kOk;
    }
    auto f = factories_.find(device_type);
    if (f == factories_.end())
        return fail(kUnsupportedDevice, "unsupported device: no factory registered for " + device_type);
    std::shared_ptr<Device> dev;
    MRK_TRY(f->second(device_id, AllocatorRegistry::global(), &dev));
    devices_[key] = dev;
    *out = dev;
    return kOk;
}

std::shared_ptr<Device> DeviceFactoryRegistry::find(const std::string& device_type, int device_id) {
    std::string key = device_type + ":" + std::to_string(device_id);
    std::lock_guard<std::mutex> lock(mu_);
    auto it = devices_.find(key);
    return it == devices_.end() ? nullptr : it->second;
}

void DeviceFactoryRegistry::reset() {
    std::lock_guard<std::mutex> lock(mu_);
    devices_.clear();
}

int create_hip_device(int device_id, AllocatorRegistry& registry, std::shared_ptr<Device>* out) {
    auto dev = std::make_shared<Device>();
    dev->device_id = device_id;
    MRK_TRY(registry.get(device_id, &dev->allocator));
    // set-up work that must not happen later, inside entry points that promise not to allocate:
    // the per-device address of the split-K scratch array (this device is current here)
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    MRK_HIP(gemm_bf16_static_workspace_init(device_id), "hipGetSymbolAddress(split-K scratch)");
    dev->renderer = make_hip_renderer(device_id);
    dev->compiler = make_hiprtc_compiler();
    ffi::Stream stream = dev->allocator->stream();
    dev->runtime = [device_id, stream](const CompiledSpec& spec, std::unique_ptr<Program>* p) {
        return create_module_program(device_id, stream, spec, p);
    };
    *out = dev;
    return kOk;
}

}  // namespace mrk
