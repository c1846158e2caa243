// Allocators for the HIP device: the counterpart of morok's `Allocator` trait and
// `LruAllocator` (device/src/allocator.rs:180-190,330-442), with `HipAllocator` taking
// the place `CudaAllocator` holds in the reference (allocator.rs:258-309).
#pragma once
#include <cstddef>
#include <cstdint>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "hip_ffi.h"

namespace mrk {

// device/src/allocator.rs:161-178.  Note the reference default is cpu_accessible = true;
// device buffers of this backend are created with cpu_accessible = false.
struct BufferOptions {
    bool zero_init = false;
    bool cpu_accessible = false;
};

// One raw allocation (device/src/allocator.rs:87-107).  `ptr` is a device virtual
// address; for cpu_accessible allocations it is managed memory valid on host too.
struct RawBuffer {
    void* ptr = nullptr;
    size_t size = 0;
    bool cpu_accessible = false;
};

class Allocator {
  public:
    virtual ~Allocator() = default;
    virtual int alloc(size_t size, const BufferOptions& options, RawBuffer* out) = 0;
    virtual void free(const RawBuffer& buffer, const BufferOptions& options) = 0;
    virtual int synchronize() = 0;
    virtual const char* name() const = 0;
    virtual int device_id() const = 0;
    virtual ffi::Stream stream() const = 0;
};

// hipMalloc / hipMallocManaged on one device, one in-order stream for all work on it.
class HipAllocator final : public Allocator {
  public:
    static int create(int device_id, std::unique_ptr<HipAllocator>* out);
    ~HipAllocator() override;
    int alloc(size_t size, const BufferOptions& options, RawBuffer* out) override;
    void free(const RawBuffer& buffer, const BufferOptions& options) override;
    int synchronize() override;
    const char* name() const override { return "HIP"; }
    int device_id() const override { return device_id_; }
    ffi::Stream stream() const override { return stream_; }

  private:
    HipAllocator(int device_id, ffi::Stream s) : device_id_(device_id), stream_(s) {}
    int device_id_;
    ffi::Stream stream_;
};

// Caches freed buffers keyed by (size, cpu_accessible), at most `max_per_key` per key,
// zeroes a reused buffer when zero_init is requested, and on an inner allocation failure
// clears the cache and retries once (device/src/allocator.rs:366-429).
class LruAllocator final : public Allocator {
  public:
    explicit LruAllocator(std::unique_ptr<Allocator> inner, size_t max_per_key = 32);
    ~LruAllocator() override;
    int alloc(size_t size, const BufferOptions& options, RawBuffer* out) override;
    void free(const RawBuffer& buffer, const BufferOptions& options) override;
    int synchronize() override { return inner_->synchronize(); }
    const char* name() const override { return inner_->name(); }
    int device_id() const override { return inner_->device_id(); }
    ffi::Stream stream() const override { return inner_->stream(); }

    size_t cache_count(size_t size, bool cpu_accessible);
    size_t total_cached();
    void clear();

  private:
    struct Key {
        size_t size;
        bool cpu_accessible;
        bool operator==(const Key& o) const { return size == o.size && cpu_accessible == o.cpu_accessible; }
    };
    struct KeyHash {
        size_t operator()(const Key& k) const { return std::hash<size_t>()(k.size * 2 + (k.cpu_accessible ? 1 : 0)); }
    };
    std::unique_ptr<Allocator> inner_;
    std::mutex mu_;
    std::unordered_map<Key, std::vector<RawBuffer>, KeyHash> cache_;
    size_t max_per_key_;
};

}  // namespace mrk
