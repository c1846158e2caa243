#include "buffer.h"

#include "error.h"

namespace mrk {

static std::atomic<uint64_t> g_next_buffer_id{1};

BufferData::BufferData(std::shared_ptr<Allocator> allocator, size_t size, BufferOptions options)
    : id_(g_next_buffer_id.fetch_add(1)), allocator_(std::move(allocator)), total_size_(size), options_(options) {}

BufferData::~BufferData() {
    if (allocated_.load()) allocator_->free(raw_, options_);
}

int BufferData::ensure_allocated() {
    if (allocated_.load(std::memory_order_acquire)) return kOk;
    std::lock_guard<std::mutex> lock(mu_);
    if (allocated_.load(std::memory_order_relaxed)) return kOk;
    MRK_TRY(allocator_->alloc(total_size_, options_, &raw_));
    allocated_.store(true, std::memory_order_release);
    return kOk;
}

Buffer::Buffer(std::shared_ptr<Allocator> allocator, size_t size, BufferOptions options)
    : data_(std::make_shared<BufferData>(std::move(allocator), size, options)), offset_(0), size_(size) {}

int Buffer::view(size_t offset, size_t size, std::unique_ptr<Buffer>* out) const {
    if (offset + size > size_ || offset + size < offset)
        return failf(kInvalidView, "invalid view: offset %zu + size %zu exceeds buffer size %zu", offset, size, size_);
    out->reset(new Buffer(data_, offset_ + offset, size));
    return kOk;
}

int Buffer::copyin(const void* src, size_t n) {
    MRK_TRY(ensure_allocated());
    if (n != size_) return failf(kSizeMismatch, "size mismatch: expected %zu, got %zu", size_, n);
    if (n == 0) return kOk;
    Allocator* a = data_->allocator();
    MRK_HIP(ffi::set_device(a->device_id()), "hipSetDevice");
    char* dst = static_cast<char*>(data_->raw().ptr) + offset_;
    MRK_HIP(ffi::memcpy_htod_async(dst, src, n, a->stream()), "hipMemcpyAsync(HtoD)");
    // The host slice is only borrowed for the duration of the call.
    MRK_HIP(ffi::stream_synchronize(a->stream()), "hipStreamSynchronize");
    return kOk;
}

int Buffer::copyout(void* dst, size_t n) const {
    MRK_TRY(ensure_allocated());
    if (n != size_) return failf(kSizeMismatch, "size mismatch: expected %zu, got %zu", size_, n);
    if (n == 0) return kOk;
    Allocator* a = data_->allocator();
    MRK_HIP(ffi::set_device(a->device_id()), "hipSetDevice");
    const char* src = static_cast<const char*>(data_->raw().ptr) + offset_;
    // In-order stream: the copy is queued behind every kernel launched so far, and the
    // synchronize makes the bytes visible before returning (cf. buffer.rs:391-397).
    MRK_HIP(ffi::memcpy_dtoh_async(dst, src, n, a->stream()), "hipMemcpyAsync(DtoH)");
    MRK_HIP(ffi::stream_synchronize(a->stream()), "hipStreamSynchronize");
    return kOk;
}

int Buffer::copy_from(const Buffer& src) {
    MRK_TRY(ensure_allocated());
    MRK_TRY(src.ensure_allocated());
    if (src.size_ != size_) return failf(kSizeMismatch, "size mismatch: expected %zu, got %zu", size_, src.size_);
    if (size_ == 0) return kOk;
    Allocator* a = data_->allocator();
    if (src.device_id() != a->device_id())
        return failf(kCopyFailed, "copy operation failed: cross-device copy HIP:%d -> HIP:%d is not supported",
                     src.device_id(), a->device_id());
    MRK_HIP(ffi::set_device(a->device_id()), "hipSetDevice");
    char* d = static_cast<char*>(data_->raw().ptr) + offset_;
    const char* s = static_cast<const char*>(src.data_->raw().ptr) + src.offset_;
    MRK_HIP(ffi::memcpy_dtod_async(d, s, size_, a->stream()), "hipMemcpyAsync(DtoD)");
    return kOk;
}

int Buffer::as_raw_ptr(void** out) const {
    if (!is_allocated()) return fail(kNotAllocated, "buffer not allocated");
    *out = static_cast<char*>(data_->raw().ptr) + offset_;
    return kOk;
}

}  // namespace mrk
