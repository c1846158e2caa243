#include "allocator.h"

#include "error.h"

namespace mrk {

int HipAllocator::create(int device_id, std::unique_ptr<HipAllocator>* out) {
    int count = 0;
    MRK_HIP(ffi::device_count(&count), "hipGetDeviceCount");
    if (device_id < 0 || device_id >= count)
        return failf(kInvalidDevice, "invalid device: HIP:%d (device count %d)", device_id, count);
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    ffi::Stream s = nullptr;
    MRK_HIP(ffi::stream_create(&s), "hipStreamCreateWithFlags");
    out->reset(new HipAllocator(device_id, s));
    return kOk;
}

HipAllocator::~HipAllocator() {
    if (stream_) {
        ffi::set_device(device_id_);
        ffi::stream_synchronize(stream_);
        ffi::stream_destroy(stream_);
    }
}

int HipAllocator::alloc(size_t size, const BufferOptions& options, RawBuffer* out) {
    MRK_HIP(ffi::set_device(device_id_), "hipSetDevice");
    void* p = nullptr;
    // A zero-byte request still yields a distinct, valid allocation.
    size_t bytes = size == 0 ? 1 : size;
    int rc = options.cpu_accessible ? ffi::malloc_managed(&p, bytes) : ffi::malloc_device(&p, bytes);
    if (rc != 0) {
        ffi::clear_last_error();
        return fail_hip(rc, options.cpu_accessible ? "hipMallocManaged" : "hipMalloc");
    }
    if (options.zero_init) {
        rc = ffi::memset_async(p, 0, bytes, stream_);
        if (rc != 0) {
            ffi::free_device(p);
            return fail_hip(rc, "hipMemsetAsync");
        }
    }
    out->ptr = p;
    out->size = size;
    out->cpu_accessible = options.cpu_accessible;
    return kOk;
}

void HipAllocator::free(const RawBuffer& buffer, const BufferOptions&) {
    if (!buffer.ptr) return;
    ffi::set_device(device_id_);
    // hipFree waits for outstanding work that may still read the allocation.
    ffi::free_device(buffer.ptr);
}

int HipAllocator::synchronize() {
    MRK_HIP(ffi::set_device(device_id_), "hipSetDevice");
    MRK_HIP(ffi::stream_synchronize(stream_), "hipStreamSynchronize");
    return kOk;
}

LruAllocator::LruAllocator(std::unique_ptr<Allocator> inner, size_t max_per_key)
    : inner_(std::move(inner)), max_per_key_(max_per_key) {}

LruAllocator::~LruAllocator() { clear(); }

int LruAllocator::alloc(size_t size, const BufferOptions& options, RawBuffer* out) {
    Key key{size, options.cpu_accessible};
    bool hit = false;
    RawBuffer cached;
    {
        std::lock_guard<std::mutex> lock(mu_);
        auto it = cache_.find(key);
        if (it != cache_.end() && !it->second.empty()) {
            cached = it->second.back();
            it->second.pop_back();
            if (it->second.empty()) cache_.erase(it);
            hit = true;
        }
    }  // lock dropped before any device work
    if (hit) {
        if (options.zero_init) {
            MRK_HIP(ffi::set_device(inner_->device_id()), "hipSetDevice");
            MRK_HIP(ffi::memset_async(cached.ptr, 0, size == 0 ? 1 : size, inner_->stream()), "hipMemsetAsync");
        }
        *out = cached;
        return kOk;
    }
    int rc = inner_->alloc(size, options, out);
    if (rc == kOk) return rc;
    // Allocation failed: drop every cached buffer and retry once, reporting the
    // first error if the retry fails too.
    std::string first_error = last_error();
    clear();
    int rc2 = inner_->alloc(size, options, out);
    if (rc2 != kOk) return fail(static_cast<Status>(rc), first_error);
    clear_error();
    return kOk;
}

void LruAllocator::free(const RawBuffer& buffer, const BufferOptions& options) {
    Key key{buffer.size, options.cpu_accessible};
    {
        std::lock_guard<std::mutex> lock(mu_);
        auto& v = cache_[key];
        if (v.size() < max_per_key_) {
            v.push_back(buffer);
            return;
        }
    }
    inner_->free(buffer, options);
}

size_t LruAllocator::cache_count(size_t size, bool cpu_accessible) {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = cache_.find(Key{size, cpu_accessible});
    return it == cache_.end() ? 0 : it->second.size();
}

size_t LruAllocator::total_cached() {
    std::lock_guard<std::mutex> lock(mu_);
    size_t n = 0;
    for (auto& kv : cache_) n += kv.second.size();
    return n;
}

void LruAllocator::clear() {
    std::unordered_map<Key, std::vector<RawBuffer>, KeyHash> drained;
    {
        std::lock_guard<std::mutex> lock(mu_);
        drained.swap(cache_);
    }
    for (auto& kv : drained) {
        BufferOptions o;
        o.cpu_accessible = kv.first.cpu_accessible;
        for (auto& b : kv.second) inner_->free(b, o);
    }
}

}  // namespace mrk
