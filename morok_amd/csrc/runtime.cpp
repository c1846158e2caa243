#include "runtime.h"

#include <cstring>
#include <functional>
#include <thread>

#include "error.h"
#include "uop.h"

namespace mrk {

KernelCache& KernelCache::global() {
    static KernelCache* c = new KernelCache();
    return *c;
}

int KernelCache::get_or_compile(uint64_t ast_hash, const std::string& device, const CompileFn& compile_fn,
                                std::shared_ptr<CachedKernel>* out, bool* was_cached) {
    const std::string key = std::to_string(ast_hash) + "@" + device;
    {
        std::lock_guard<std::mutex> lock(mu_);
        auto it = map_.find(key);
        if (it != map_.end()) {
            *out = it->second;
            if (was_cached) *was_cached = true;
            return kOk;
        }
    }
    // compile outside the lock (expensive); a racing thread may compile the same kernel
    std::shared_ptr<CachedKernel> fresh;
    MRK_TRY(compile_fn(&fresh));
    std::lock_guard<std::mutex> lock(mu_);
    auto ins = map_.emplace(key, fresh);
    *out = ins.first->second;  // first insert wins
    if (was_cached) *was_cached = false;
    return kOk;
}

size_t KernelCache::size() {
    std::lock_guard<std::mutex> lock(mu_);
    return map_.size();
}

void KernelCache::clear_all() {
    std::unordered_map<std::string, std::shared_ptr<CachedKernel>> drained;
    {
        std::lock_guard<std::mutex> lock(mu_);
        drained.swap(map_);
    }
}

int get_or_compile_linear_kernel(const Device& dev, const LinearKernel& k, const char* name,
                                 std::shared_ptr<CachedKernel>* out, bool* was_cached) {
    const std::string device = std::string(Device::base_device_key()) + ":" + std::to_string(dev.device_id);
    // the cache key also covers the compiler backend (tensor/src/realize.rs:1052-1054)
    const uint64_t key = k.content_hash ^ fnv1a64(reinterpret_cast<const uint8_t*>(dev.compiler->cache_key()),
                                                  std::strlen(dev.compiler->cache_key()));
    return KernelCache::global().get_or_compile(
        key, device,
        [&](std::shared_ptr<CachedKernel>* fresh) -> int {
            ProgramSpec spec;
            MRK_TRY(dev.renderer->render(k, name, &spec));
            CompiledSpec compiled;
            MRK_TRY(dev.compiler->compile(spec, &compiled));
            std::unique_ptr<Program> prog;
            MRK_TRY(dev.runtime(compiled, &prog));
            auto ck = std::make_shared<CachedKernel>();
            ck->program = std::move(prog);
            ck->device = device;
            ck->code = spec.src;
            ck->entry_point = spec.name;
            ck->var_names = spec.var_names;
            ck->has_sizes = spec.has_sizes;
            ck->global_size = spec.global_size;
            ck->local_size = spec.local_size;
            *fresh = std::move(ck);
            return kOk;
        },
        out, was_cached);
}

size_t ExecutionPlan::add_buffer(std::shared_ptr<Buffer> b) {
    for (size_t i = 0; i < buffers_.size(); i++)
        if (buffers_[i].get() == b.get()) return i;
    buffers_.push_back(std::move(b));
    return buffers_.size() - 1;
}

int ExecutionPlan::add_kernel(std::shared_ptr<CachedKernel> kernel, const std::vector<size_t>& buffer_indices,
                              const std::vector<int64_t>& vals) {
    for (size_t i : buffer_indices)
        if (i >= buffers_.size()) return fail(kInvalidArgument, "execution plan: buffer index out of range");
    if (vals.size() != kernel->var_names.size())
        return failf(kInvalidArgument, "execution plan: kernel '%s' has %zu variables, %zu values given",
                     kernel->entry_point.c_str(), kernel->var_names.size(), vals.size());
    PreparedKernel pk;
    pk.id = kernels_.size();
    pk.kernel = std::move(kernel);
    pk.buffer_indices = buffer_indices;
    pk.vals = vals;
    kernels_.push_back(std::move(pk));
    built_ = false;
    return kOk;
}

int ExecutionPlan::build() {
    for (auto& b : buffers_) MRK_TRY(b->ensure_allocated());  // tensor/src/realize.rs:974-981
    for (auto& pk : kernels_) {
        pk.buffer_ptrs.clear();
        pk.buffer_ids.clear();
        for (size_t i : pk.buffer_indices) {
            void* p = nullptr;
            MRK_TRY(buffers_[i]->as_raw_ptr(&p));
            pk.buffer_ptrs.push_back(p);
            pk.buffer_ids.push_back(buffers_[i]->id());
        }
    }
    built_ = true;
    return kOk;
}

int ExecutionPlan::execute() {
    if (!built_) MRK_TRY(build());
    for (auto& pk : kernels_) {
        const CachedKernel& ck = *pk.kernel;
        int rc = ck.program->execute(pk.buffer_ptrs.data(), pk.buffer_ptrs.size(), pk.vals.data(), pk.vals.size(),
                                     ck.has_sizes ? ck.global_size.data() : nullptr,
                                     ck.has_sizes ? ck.local_size.data() : nullptr);
        if (rc != kOk) {
            std::string inner = last_error();
            return failf(static_cast<Status>(rc), "Kernel %llu failed: %s", (unsigned long long)pk.id, inner.c_str());
        }
    }
    return kOk;
}

int ExecutionPlan::execute_profiled(std::vector<KernelProfile>* out) {
    if (!built_) MRK_TRY(build());
    out->clear();
    if (kernels_.empty()) return kOk;
    ffi::Stream stream = buffers_.empty() ? nullptr : nullptr;
    std::shared_ptr<Allocator> alloc;
    MRK_TRY(AllocatorRegistry::global().get(device_id_, &alloc));
    stream = alloc->stream();
    MRK_HIP(ffi::set_device(device_id_), "hipSetDevice");
    std::vector<ffi::Event> ev(kernels_.size() + 1, nullptr);
    for (auto& e : ev) MRK_HIP(ffi::event_create(&e), "hipEventCreate");
    int rc = kOk;
    MRK_HIP(ffi::event_record(ev[0], stream), "hipEventRecord");
    for (size_t i = 0; i < kernels_.size() && rc == kOk; i++) {
        auto& pk = kernels_[i];
        const CachedKernel& ck = *pk.kernel;
        rc = ck.program->execute(pk.buffer_ptrs.data(), pk.buffer_ptrs.size(), pk.vals.data(), pk.vals.size(),
                                 ck.has_sizes ? ck.global_size.data() : nullptr,
                                 ck.has_sizes ? ck.local_size.data() : nullptr);
        if (rc == kOk && ffi::event_record(ev[i + 1], stream) != 0) rc = fail(kHipError, "hipEventRecord failed");
    }
    if (rc == kOk) {
        if (ffi::event_synchronize(ev.back()) != 0) rc = fail(kHipError, "hipEventSynchronize failed");
        for (size_t i = 0; i < kernels_.size() && rc == kOk; i++) {
            float ms = 0;
            ffi::event_elapsed_ms(&ms, ev[i], ev[i + 1]);
            KernelProfile p;
            p.entry_point = kernels_[i].kernel->entry_point;
            p.num_buffers = kernels_[i].buffer_ptrs.size();
            p.elapsed_ms = ms;
            out->push_back(p);
        }
    }
    for (auto& e : ev) ffi::event_destroy(e);
    return rc;
}

int ExecutionPlan::execute_with_vars(const std::vector<std::pair<std::string, int64_t>>& var_vals) {
    for (auto& pk : kernels_) {
        const auto& names = pk.kernel->var_names;
        for (size_t i = 0; i < names.size(); i++)
            for (const auto& kv : var_vals)
                if (kv.first == names[i]) pk.vals[i] = kv.second;
    }
    return execute();
}

int benchmark_kernel(int device_id, ffi::Stream stream, Program* program, void* const* buffers, size_t nbufs,
                     const int64_t* vals, size_t nvals, const size_t* global, const size_t* local, int warmup,
                     int runs, BenchmarkResult* out) {
    if (runs <= 0) return fail(kInvalidArgument, "benchmark: runs must be positive");
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    for (int i = 0; i < warmup; i++) MRK_TRY(program->execute(buffers, nbufs, vals, nvals, global, local));
    ffi::Event e0 = nullptr, e1 = nullptr;
    MRK_HIP(ffi::event_create(&e0), "hipEventCreate");
    MRK_HIP(ffi::event_create(&e1), "hipEventCreate");
    double mn = 1e300, mx = 0, sum = 0;
    int rc = kOk;
    for (int i = 0; i < runs && rc == kOk; i++) {
        ffi::event_record(e0, stream);
        rc = program->execute(buffers, nbufs, vals, nvals, global, local);
        ffi::event_record(e1, stream);
        if (rc != kOk) break;
        if (ffi::event_synchronize(e1) != 0) {
            rc = fail(kHipError, "hipEventSynchronize failed");
            break;
        }
        float ms = 0;
        ffi::event_elapsed_ms(&ms, e0, e1);
        mn = ms < mn ? ms : mn;
        mx = ms > mx ? ms : mx;
        sum += ms;
    }
    ffi::event_destroy(e0);
    ffi::event_destroy(e1);
    if (rc != kOk) return rc;
    out->min_ms = mn;
    out->max_ms = mx;
    out->mean_ms = sum / runs;
    out->runs = runs;
    return kOk;
}

TimelineSignal::~TimelineSignal() {
    for (auto& p : pending_) ffi::event_destroy(p.second);
}

uint64_t TimelineSignal::value() {
    std::lock_guard<std::mutex> lock(mu_);
    // events complete in stream order: retire from the front
    while (!pending_.empty() && ffi::event_query(pending_.front().second) == 0) {
        completed_ = pending_.front().first > completed_ ? pending_.front().first : completed_;
        ffi::event_destroy(pending_.front().second);
        pending_.erase(pending_.begin());
    }
    return completed_;
}

int TimelineSignal::set(uint64_t value) {
    MRK_HIP(ffi::set_device(device_id_), "hipSetDevice");
    ffi::Event e = nullptr;
    MRK_HIP(ffi::event_create(&e), "hipEventCreate");
    int rc = ffi::event_record(e, stream_);
    if (rc != 0) {
        ffi::event_destroy(e);
        return fail_hip(rc, "hipEventRecord");
    }
    std::lock_guard<std::mutex> lock(mu_);
    pending_.emplace_back(value, e);
    // keep the last 16 events; older ones are waited for and folded into the completed value
    while (pending_.size() > 16) {
        ffi::event_synchronize(pending_.front().second);
        completed_ = pending_.front().first > completed_ ? pending_.front().first : completed_;
        ffi::event_destroy(pending_.front().second);
        pending_.erase(pending_.begin());
    }
    return kOk;
}

int TimelineSignal::wait(uint64_t target, uint64_t timeout_ms) {
    auto deadline = std::chrono::steady_clock::now() + std::chrono::milliseconds(timeout_ms);
    for (;;) {
        uint64_t v = value();
        if (v >= target) return kOk;
        if (std::chrono::steady_clock::now() >= deadline)
            return failf(kTimeout, "runtime error: timeline signal wait timed out after %llu ms (value %llu, waiting for %llu)",
                         (unsigned long long)timeout_ms, (unsigned long long)v, (unsigned long long)target);
        std::this_thread::sleep_for(std::chrono::microseconds(50));
    }
}

}  // namespace mrk
