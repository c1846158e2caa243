// Hardware command queues over HIP streams: device/src/queue.rs:76-161.  A queue batches
// wait / signal / exec / copy commands and hands them to its own stream on submit();
// ordering between queues is expressed with timeline signals
// (device/src/sync.rs:44-71), which become hipStreamWaitEvent dependencies on the GPU, so
// a copy queue and a compute queue overlap exactly where no signal orders them.
//
// Ordering against the device's own stream (allocations, zero-fills, uploads, Tensor::realize):
// a batch starts only after everything queued on the device stream at submit() time has
// finished (one event per submit), so a zero_init fill or an upload lands before the batch's
// kernels touch the buffer.  Lifetime: the buffers and kernels of a batch stay referenced by
// the queue until the batch has completed on the GPU, so a caller may release them right after
// submit(); when they are finally dropped the device stream is made to wait for that batch
// first, so that a block going back to the allocator's cache is not handed to device-stream
// work that would overtake the batch.  The reverse direction is the caller's: device-stream
// work (copyout included) that must see a batch's results needs queue.synchronize() or a
// signal wait first.
#pragma once
#include <deque>
#include <memory>
#include <vector>

#include "buffer.h"
#include "runtime.h"

namespace mrk {

class HardwareQueue {
  public:
    // copy_queue only names the queue's role (both kinds are HIP streams of default priority).
    HardwareQueue(int device_id, bool copy_queue);
    ~HardwareQueue();
    HardwareQueue(const HardwareQueue&) = delete;
    HardwareQueue& operator=(const HardwareQueue&) = delete;
    int init();

    // queue.rs:93-99: commands after this one start only when `signal` has reached `value`
    void wait(std::shared_ptr<TimelineSignal> signal, uint64_t value);
    // queue.rs:101-105: `signal` takes `value` when every earlier command has finished
    void signal(std::shared_ptr<TimelineSignal> signal, uint64_t value);
    // queue.rs:107-121
    void exec(std::shared_ptr<CachedKernel> kernel, std::vector<std::shared_ptr<Buffer>> buffers, std::vector<int64_t> vals,
              const size_t* global, const size_t* local);
    // queue.rs:123-128: sizes must match (Buffer::copy_from, device/src/buffer.rs:411-534)
    void copy(std::shared_ptr<Buffer> dst, std::shared_ptr<Buffer> src);
    // queue.rs:130-134: a stream executes in order and each command sees the memory effects
    // of the previous one, so this records nothing
    void memory_barrier() {}
    // queue.rs:136-141: hands the batch to the stream; does not wait for completion.  A wait
    // on a value nobody has signalled yet is retried for wait_timeout_ms, then kTimeout.
    int submit(uint64_t wait_timeout_ms = 10000);
    int synchronize();
    size_t pending_commands() const { return cmds_.size(); }
    size_t batches_in_flight() const { return in_flight_.size(); }
    bool is_copy_queue() const { return copy_queue_; }
    ffi::Stream stream() const { return stream_; }

  private:
    enum class Kind { Wait, Signal, Exec, Copy };
    struct Command {
        Kind kind;
        std::shared_ptr<TimelineSignal> signal;
        uint64_t value = 0;
        std::shared_ptr<CachedKernel> kernel;
        std::vector<std::shared_ptr<Buffer>> buffers;
        std::vector<int64_t> vals;
        bool has_sizes = false;
        size_t global[3] = {1, 1, 1}, local[3] = {1, 1, 1};
    };
    struct InFlight {
        ffi::Event done = nullptr;   // recorded on the queue's stream behind the batch
        ffi::Event ready = nullptr;  // recorded on the device stream in front of the batch
        std::vector<Command> batch;
    };
    // drops the batches whose completion event has fired (all of them when `all`, after the
    // caller has synchronized the stream)
    void retire(bool all, bool after_synchronize = false);
    int issue(std::vector<Command>& batch, uint64_t wait_timeout_ms);
    int device_id_;
    bool copy_queue_;
    ffi::Stream stream_ = nullptr;
    std::shared_ptr<Allocator> device_allocator_;  // owner of device_stream_
    ffi::Stream device_stream_ = nullptr;  // the allocator's stream of this device
    std::vector<Command> cmds_;
    std::deque<InFlight> in_flight_;
};

}  // namespace mrk
