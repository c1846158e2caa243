// Device buffer with lazy allocation and byte-offset views: the counterpart of
// `Buffer`/`BufferData` (device/src/buffer.rs:40-155,327-574).
#pragma once
#include <atomic>
#include <memory>
#include <mutex>

#include "allocator.h"

namespace mrk {

// Shared state of one base allocation (buffer.rs:40-93): allocated on first use, returned
// to the allocator when the last view is released.
class BufferData {
  public:
    BufferData(std::shared_ptr<Allocator> allocator, size_t size, BufferOptions options);
    ~BufferData();
    int ensure_allocated();
    bool is_allocated() const { return allocated_.load(std::memory_order_acquire); }
    const RawBuffer& raw() const { return raw_; }
    uint64_t id() const { return id_; }
    size_t total_size() const { return total_size_; }
    Allocator* allocator() const { return allocator_.get(); }
    const BufferOptions& options() const { return options_; }

  private:
    uint64_t id_;
    std::shared_ptr<Allocator> allocator_;
    size_t total_size_;
    BufferOptions options_;
    std::mutex mu_;
    std::atomic<bool> allocated_{false};
    RawBuffer raw_;
};

class Buffer {
  public:
    // buffer.rs:112-121: lazy - nothing is allocated until first use.
    Buffer(std::shared_ptr<Allocator> allocator, size_t size, BufferOptions options);
    // buffer.rs:136-150: InvalidView if offset + size exceeds this view.
    int view(size_t offset, size_t size, std::unique_ptr<Buffer>* out) const;
    int ensure_allocated() const { return data_->ensure_allocated(); }
    bool is_allocated() const { return data_->is_allocated(); }
    uint64_t id() const { return data_->id(); }  // views share the id (buffer.rs:327-329)
    size_t size() const { return size_; }
    size_t offset() const { return offset_; }
    int device_id() const { return data_->allocator()->device_id(); }
    // buffer.rs:332-368 / 371-408 / 411-534: sizes must match exactly.
    int copyin(const void* src, size_t n);
    int copyout(void* dst, size_t n) const;
    int copy_from(const Buffer& src);
    // buffer.rs:554-574: pointer handed to kernels; for this backend the device VA + offset.
    int as_raw_ptr(void** out) const;
    int synchronize() const { return data_->allocator()->synchronize(); }
    // true when this handle covers its whole base allocation (not a sub-range view)
    bool is_whole() const { return offset_ == 0 && size_ == data_->total_size(); }
    const BufferOptions& options() const { return data_->options(); }

  private:
    Buffer(std::shared_ptr<BufferData> data, size_t offset, size_t size)
        : data_(std::move(data)), offset_(offset), size_(size) {}
    std::shared_ptr<BufferData> data_;
    size_t offset_;
    size_t size_;
};

}  // namespace mrk
