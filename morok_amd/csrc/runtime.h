// Kernel cache and execution plan: the counterparts of runtime/src/kernel_cache.rs:27-158
// and runtime/src/execution_plan.rs:50-250,391-411.
#pragma once
#include <array>
#include <chrono>
#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "buffer.h"
#include "device.h"

namespace mrk {

// runtime/src/kernel_cache.rs:27-44
struct CachedKernel {
    std::unique_ptr<Program> program;
    std::string device;  // "HIP:0"
    std::string code;    // rendered source (empty for hand-written kernels)
    std::string entry_point;
    std::vector<std::string> var_names;
    bool has_sizes = false;
    std::array<size_t, 3> global_size{1, 1, 1};
    std::array<size_t, 3> local_size{1, 1, 1};
};

// Global dedup cache keyed by (AST content hash, device string)
// (kernel_cache.rs:52-56,87-118).  Two threads racing on one key may both compile; the
// first insert wins and both receive the winner.
class KernelCache {
  public:
    static KernelCache& global();
    using CompileFn = std::function<int(std::shared_ptr<CachedKernel>*)>;
    int get_or_compile(uint64_t ast_hash, const std::string& device, const CompileFn& compile_fn,
                       std::shared_ptr<CachedKernel>* out, bool* was_cached = nullptr);
    // the cached kernel, if there is one (no compile)
    bool lookup(uint64_t ast_hash, const std::string& device, std::shared_ptr<CachedKernel>* out);
    size_t size();
    void clear_all();  // kernel_cache.rs:124-130

  private:
    std::mutex mu_;
    std::unordered_map<std::string, std::shared_ptr<CachedKernel>> map_;
};

// Render -> compile -> load through the three hooks of a Device, memoised in the cache:
// what prepare_execution_plan does per kernel (tensor/src/realize.rs:1052-1070).
int get_or_compile_linear_kernel(const Device& dev, const LinearKernel& k, const char* name,
                                 std::shared_ptr<CachedKernel>* out, bool* was_cached = nullptr);
// The cache lookup alone: true and the kernel when this device already holds it.
bool lookup_linear_kernel(const Device& dev, const LinearKernel& k, std::shared_ptr<CachedKernel>* out);

// execution_plan.rs:50-82
struct PreparedKernel {
    uint64_t id = 0;
    std::shared_ptr<CachedKernel> kernel;
    std::vector<size_t> buffer_indices;
    std::vector<int64_t> vals;
    std::vector<void*> buffer_ptrs;  // precomputed with Buffer::as_raw_ptr (execution_plan.rs:391-397)
    std::vector<uint64_t> buffer_ids;
};

// runtime/src/profiler.rs:30-39; elapsed is measured with HIP events on the device stream
// (the reference uses Instant around a blocking CPU call).
struct KernelProfile {
    std::string entry_point;
    size_t num_buffers = 0;
    double elapsed_ms = 0.0;
};

// tensor/src/memory_planner.rs:84-96
struct MemoryPlanStats {
    size_t planned = 0;         // intermediates that took part
    size_t buffers_reused = 0;  // of those, how many were given an already used block
    size_t memory_saved = 0;    // bytes not allocated thanks to reuse
    size_t memory_planned = 0;  // bytes the intermediates occupy (after reuse when the planner ran; one block each otherwise)
};

class ExecutionPlan {
  public:
    explicit ExecutionPlan(int device_id) : device_id_(device_id) {}
    ~ExecutionPlan();
    ExecutionPlan(const ExecutionPlan&) = delete;
    ExecutionPlan& operator=(const ExecutionPlan&) = delete;
    // Builder (execution_plan.rs:330-411): the plan owns clones of all buffers, which keeps
    // the precomputed pointers valid.
    size_t add_buffer(std::shared_ptr<Buffer> b);
    int add_kernel(std::shared_ptr<CachedKernel> kernel, const std::vector<size_t>& buffer_indices,
                   const std::vector<int64_t>& vals);
    void set_outputs(const std::vector<size_t>& idx) { outputs_ = idx; }
    // Liveness-based reuse of intermediate buffers (tensor/src/memory_planner.rs:1-45): at
    // build(), every buffer that is not yet allocated, not an output and not a view is given
    // a block from a pool keyed by its size rounded up to 4 KiB; a block returns to the pool
    // after the last kernel that touches its buffer.  Kernels run in order on one stream,
    // so a block may be rewritten as soon as the kernel after its last reader is queued.
    void enable_memory_planner() { plan_memory_ = true; }
    const MemoryPlanStats& memory_plan() const { return mem_stats_; }
    int build();  // ensure_allocated on every buffer, compute raw pointers

    // execution_plan.rs:168-181: tight loop, no allocation, no per-launch sync.
    int execute();
    // The same launches replayed as one HIP graph: the first call records execute() on the
    // device's stream (kernel launches only) and instantiates the graph, later calls are a
    // single hipGraphLaunch.  For launch-bound plans (many short kernels); no counterpart in
    // the reference, whose CPU kernels are plain function calls.  Rebinding variables or
    // adding kernels drops the recorded graph.
    int execute_graph();
    bool has_graph() const { return graph_exec_ != nullptr; }
    // execution_plan.rs:200-221
    int execute_profiled(std::vector<KernelProfile>* out);
    // execution_plan.rs:239-250: rebinding by name, kernels are not recompiled.
    int execute_with_vars(const std::vector<std::pair<std::string, int64_t>>& var_vals);

    size_t kernel_count() const { return kernels_.size(); }
    const PreparedKernel& kernel(size_t i) const { return kernels_[i]; }
    size_t buffer_count() const { return buffers_.size(); }
    std::shared_ptr<Buffer> buffer(size_t i) const { return buffers_[i]; }
    const std::vector<size_t>& outputs() const { return outputs_; }
    int device_id() const { return device_id_; }

  private:
    int plan_memory();
    int launch_all(ffi::Stream on);  // nullptr: every program's own stream
    void drop_graph();
    ffi::GraphExec graph_exec_ = nullptr;
    int device_id_;
    bool built_ = false;
    bool plan_memory_ = false, memory_planned_ = false, census_done_ = false;
    MemoryPlanStats mem_stats_;
    std::vector<PreparedKernel> kernels_;
    std::vector<std::shared_ptr<Buffer>> buffers_;
    std::vector<size_t> outputs_;
};

// runtime/src/benchmark.rs:23-27,64-91: warm-up runs, timed runs, minimum; timed with HIP
// events instead of a wall clock so that the asynchronous launch is measured correctly.
struct BenchmarkResult {
    double min_ms = 0, mean_ms = 0, max_ms = 0;
    int runs = 0;
};
int benchmark_kernel(int device_id, ffi::Stream stream, Program* program, void* const* buffers, size_t nbufs,
                     const int64_t* vals, size_t nvals, const size_t* global, const size_t* local, int warmup,
                     int runs, BenchmarkResult* out);
// runtime/src/benchmark.rs:100-137: the same, but a candidate whose first timed run takes more than
// three times `cutoff_ms` is given up at once (*skipped = true, nothing else is filled in): a
// beam search spends no further launches on it.  cutoff_ms <= 0 disables the check.
int benchmark_kernel_with_cutoff(int device_id, ffi::Stream stream, Program* program, void* const* buffers, size_t nbufs,
                                 const int64_t* vals, size_t nvals, const size_t* global, const size_t* local, int warmup,
                                 int runs, double cutoff_ms, BenchmarkResult* out, bool* skipped);

// Beam-search timing hook (tensor/src/realize.rs:1190-1242): render and compile `k` (not timed),
// load it, then time only the execution with HIP events.  Candidates are timed one at a time
// (a process-wide lock): concurrent timing on one GPU would measure the contention, not the
// kernel.  A candidate that fails to render, compile or launch yields a status, never an
// abort (the reference wraps this in catch_unwind).
int compile_and_time(const Device& dev, const LinearKernel& k, const char* name, void* const* buffers, size_t nbufs,
                     const int64_t* vals, size_t nvals, int warmup, int runs, BenchmarkResult* out, double cutoff_ms = 0.0,
                     bool* skipped = nullptr);

// On-disk cache of search results keyed (ast_hash, beam_width, device), the role sled plays in
// schedule/src/optimizer/beam.rs:390-440: one small file per key under
// $MOROK_CACHE_DIR, else $XDG_CACHE_HOME/morok, else $HOME/.cache/morok, in beam_cache_hip/.
// IGNORE_BEAM_CACHE=1 turns lookups off (beam.rs:16-19).
class BeamCache {
  public:
    static std::string directory();
    static bool get(uint64_t ast_hash, int width, const std::string& device, std::vector<uint8_t>* value);
    static int put(uint64_t ast_hash, int width, const std::string& device, const void* value, size_t len);
};

// Beam search over the f32 matmul action space (beam.rs:1-20): stage by stage (LOCAL, UPCAST,
// UNROLL) every valid action is applied to the `width` best candidates so far, each result is
// compiled and timed, and the `width` fastest survive.  Scratch operands are allocated on the
// device for the timing runs.  *from_cache tells whether the answer came from the disk cache.
struct MatmulF32Opts;
int beam_search_matmul_f32(const Device& dev, int64_t M, int64_t N, int64_t K, int width, MatmulF32Opts* best,
                           double* best_ms, bool* from_cache, int* candidates_timed);
// The same search over the LDS-staged tensor-core matmul (bf16 in and out): LOCAL = the grid of
// waves in a workgroup, UPCAST = tensor-core tiles per wave, UNROLL = tensor-core K steps per
// barrier pair (schedule/src/optimizer/beam.rs:36-120 with the TC action applied first,
// tc.rs:358-674).
struct WmmaLdsOpts;
struct TensorCore;
int beam_search_wmma_matmul(const Device& dev, const TensorCore& tc, int tc_index, int64_t M, int64_t N, int64_t K, int width,
                            WmmaLdsOpts* best, double* best_ms, bool* from_cache, int* candidates_timed);

// device/src/sync.rs:44-71,192-310: monotonically increasing timeline value backed by one
// HIP event per recorded value (the last 16 are kept).
class TimelineSignal {
  public:
    TimelineSignal(int device_id, ffi::Stream stream) : device_id_(device_id), stream_(stream) {}
    ~TimelineSignal();
    uint64_t value();                       // highest value whose event has completed
    int set(uint64_t value);                // record an event for `value` on the stream
    int set_on(uint64_t value, ffi::Stream stream);  // the same on another stream (hardware queues)
    // Makes later work on `stream` wait on the GPU until the signal reaches `value`.  *pending
    // = true when no event for such a value has been recorded yet (the producer has not
    // submitted): the caller decides whether to retry.
    int stream_wait(uint64_t value, ffi::Stream stream, bool* pending);
    int wait(uint64_t value, uint64_t timeout_ms);  // kTimeout if not reached in time
    bool is_reached(uint64_t value) { return this->value() >= value; }

  private:
    int device_id_;
    ffi::Stream stream_;
    std::mutex mu_;
    uint64_t completed_ = 0;
    std::vector<std::pair<uint64_t, ffi::Event>> pending_;
};

}  // namespace mrk
