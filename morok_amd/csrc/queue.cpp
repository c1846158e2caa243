#include "queue.h"

#include <chrono>
#include <thread>

#include "device.h"
#include "error.h"

namespace mrk {

HardwareQueue::HardwareQueue(int device_id, bool copy_queue) : device_id_(device_id), copy_queue_(copy_queue) {}

HardwareQueue::~HardwareQueue() {
    if (stream_) {
        ffi::set_device(device_id_);
        ffi::stream_synchronize(stream_);
        retire(true, /*after_synchronize=*/true);
        ffi::stream_destroy(stream_);
    }
}

void HardwareQueue::retire(bool all, bool after_synchronize) {
    while (!in_flight_.empty()) {
        InFlight& f = in_flight_.front();
        if (!all && f.done && ffi::event_query(f.done) != 0) {  // batches complete in order
            ffi::clear_last_error();  // "not ready" is an answer, not a failure
            break;
        }
        // the blocks may return to the allocator's cache now: device-stream work queued from
        // here on starts after this batch (a no-op when the event has already fired)
        // (nothing to order after a full synchronize of the queue's stream: every batch has finished)
        if (f.done && device_stream_ && !after_synchronize) ffi::stream_wait_event(device_stream_, f.done);
        f.batch.clear();
        if (f.done) ffi::event_destroy(f.done);
        if (f.ready) ffi::event_destroy(f.ready);
        in_flight_.pop_front();
    }
}

int HardwareQueue::init() {
    MRK_HIP(ffi::set_device(device_id_), "hipSetDevice");
    MRK_HIP(ffi::stream_create(&stream_), "hipStreamCreate");
    std::shared_ptr<Device> dev;
    MRK_TRY(DeviceFactoryRegistry::global().device("HIP", device_id_, &dev));
    device_allocator_ = dev->allocator;  // keeps the stream below alive for as long as this queue exists
    device_stream_ = device_allocator_->stream();
    return kOk;
}

void HardwareQueue::wait(std::shared_ptr<TimelineSignal> signal, uint64_t value) {
    Command c;
    c.kind = Kind::Wait;
    c.signal = std::move(signal);
    c.value = value;
    cmds_.push_back(std::move(c));
}

void HardwareQueue::signal(std::shared_ptr<TimelineSignal> signal, uint64_t value) {
    Command c;
    c.kind = Kind::Signal;
    c.signal = std::move(signal);
    c.value = value;
    cmds_.push_back(std::move(c));
}

void HardwareQueue::exec(std::shared_ptr<CachedKernel> kernel, std::vector<std::shared_ptr<Buffer>> buffers,
                         std::vector<int64_t> vals, const size_t* global, const size_t* local) {
    Command c;
    c.kind = Kind::Exec;
    c.kernel = std::move(kernel);
    c.buffers = std::move(buffers);
    c.vals = std::move(vals);
    if (global && local) {
        c.has_sizes = true;
        for (int i = 0; i < 3; i++) {
            c.global[i] = global[i];
            c.local[i] = local[i];
        }
    }
    cmds_.push_back(std::move(c));
}

void HardwareQueue::copy(std::shared_ptr<Buffer> dst, std::shared_ptr<Buffer> src) {
    Command c;
    c.kind = Kind::Copy;
    c.buffers = {std::move(dst), std::move(src)};
    cmds_.push_back(std::move(c));
}

int HardwareQueue::submit(uint64_t wait_timeout_ms) {
    if (!stream_) return fail(kRuntime, "runtime error: queue used before init()");
    MRK_HIP(ffi::set_device(device_id_), "hipSetDevice");
    retire(false);
    // the batch leaves the queue whatever happens: a failed submit is not replayed
    in_flight_.emplace_back();
    std::vector<Command>& batch = in_flight_.back().batch;
    batch.swap(cmds_);
    int rc = issue(batch, wait_timeout_ms);
    // whatever part of the batch reached the stream is tracked until it has run
    ffi::Event done = nullptr;
    if (ffi::event_create(&done) == 0 && ffi::event_record(done, stream_) == 0) {
        in_flight_.back().done = done;
    } else {
        if (done) ffi::event_destroy(done);
        ffi::stream_synchronize(stream_);
        retire(true);
    }
    return rc;
}

int HardwareQueue::issue(std::vector<Command>& batch, uint64_t wait_timeout_ms) {
    // Allocate first (a lazy or zero_init buffer queues its allocation-time fill on the device
    // stream), then make this queue's stream wait for the device stream once per batch.
    bool touches_memory = false;
    for (Command& c : batch) {
        if (c.kind == Kind::Copy && c.buffers[0]->size() != c.buffers[1]->size())
            return failf(kSizeMismatch, "size mismatch: expected %zu, got %zu", c.buffers[0]->size(), c.buffers[1]->size());
        if (c.kind == Kind::Exec || c.kind == Kind::Copy) {
            touches_memory = true;
            for (auto& b : c.buffers) MRK_TRY(b->ensure_allocated());
        }
    }
    if (touches_memory && device_stream_) {
        ffi::Event& ready = in_flight_.back().ready;  // destroyed when the batch retires
        MRK_HIP(ffi::event_create(&ready), "hipEventCreate");
        MRK_HIP(ffi::event_record(ready, device_stream_), "hipEventRecord");
        MRK_HIP(ffi::stream_wait_event(stream_, ready), "hipStreamWaitEvent");
    }
    for (Command& c : batch) {
        switch (c.kind) {
            case Kind::Wait: {
                const auto deadline = std::chrono::steady_clock::now() + std::chrono::milliseconds(wait_timeout_ms);
                for (;;) {
                    bool pending = false;
                    MRK_TRY(c.signal->stream_wait(c.value, stream_, &pending));
                    if (!pending) break;
                    if (std::chrono::steady_clock::now() >= deadline)
                        return failf(kTimeout, "runtime error: queue wait on value %llu that nobody signalled within %llu ms",
                                     (unsigned long long)c.value, (unsigned long long)wait_timeout_ms);
                    std::this_thread::sleep_for(std::chrono::microseconds(50));
                }
                break;
            }
            case Kind::Signal: MRK_TRY(c.signal->set_on(c.value, stream_)); break;
            case Kind::Exec: {
                std::vector<void*> ptrs(c.buffers.size());
                for (size_t i = 0; i < c.buffers.size(); i++) MRK_TRY(c.buffers[i]->as_raw_ptr(&ptrs[i]));
                const size_t* g = c.has_sizes ? c.global : (c.kernel->has_sizes ? c.kernel->global_size.data() : nullptr);
                const size_t* l = c.has_sizes ? c.local : (c.kernel->has_sizes ? c.kernel->local_size.data() : nullptr);
                MRK_TRY(c.kernel->program->execute_on(stream_, ptrs.data(), ptrs.size(), c.vals.data(), c.vals.size(), g, l));
                break;
            }
            case Kind::Copy: {
                Buffer& dst = *c.buffers[0];
                const Buffer& src = *c.buffers[1];
                void *d = nullptr, *s = nullptr;
                MRK_TRY(dst.as_raw_ptr(&d));
                MRK_TRY(src.as_raw_ptr(&s));
                MRK_HIP(ffi::memcpy_dtod_async(d, s, dst.size(), stream_), "hipMemcpyAsync");
                break;
            }
        }
    }
    return kOk;
}

int HardwareQueue::synchronize() {
    if (!stream_) return kOk;
    MRK_HIP(ffi::set_device(device_id_), "hipSetDevice");
    MRK_HIP(ffi::stream_synchronize(stream_), "hipStreamSynchronize");
    retire(true);
    return kOk;
}

}  // namespace mrk
