// extern "C" surface of libmorok_hip.so (declared in include/morok_hip.h).
#include <cstdlib>
#include <cctype>
#include <cstring>

#include "../../include/morok_hip.h"
#include "buffer.h"
#include "builtin.h"
#include "device.h"
#include "error.h"
#include "kernels/kernels.h"
#include "queue.h"
#include "runtime.h"
#include "schedule.h"
#include "tensor.h"
#include "uop.h"

using namespace mrk;

struct mrk_buffer {
    std::unique_ptr<Buffer> b;
};
struct mrk_program_spec {
    ProgramSpec s;
};
struct mrk_compiled_spec {
    CompiledSpec c;
};
struct mrk_program {
    std::unique_ptr<Program> p;
};
struct mrk_kernel {
    std::shared_ptr<CachedKernel> k;
};
struct mrk_plan {
    std::unique_ptr<ExecutionPlan> p;
};
struct mrk_signal {
    std::shared_ptr<TimelineSignal> s;
};
struct mrk_queue {
    std::unique_ptr<HardwareQueue> q;
};
struct mrk_tensor {
    Tensor t;
};
struct mrk_event {
    int device_id;
    ffi::Event e;
    ffi::Stream stream;
};

namespace {

int get_device(int device_id, std::shared_ptr<Device>* out) {
    return DeviceFactoryRegistry::global().device("HIP", device_id, out);
}
int get_lru(int device_id, LruAllocator** out) {
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    *out = static_cast<LruAllocator*>(d->allocator.get());
    return kOk;
}
#define MRK_NONNULL(p)                                                                     \
    do {                                                                                   \
        if (!(p)) return fail(kInvalidArgument, "null argument: " #p);                     \
    } while (0)

}  // namespace

extern "C" {

const char* mrk_hip_last_error(void) { return last_error(); }

int mrk_hip_device_parse(const char* spec, int* device_id) {
    MRK_NONNULL(device_id);
    return parse_device_spec(spec, device_id);
}
int mrk_hip_device_count(int* count) {
    MRK_NONNULL(count);
    MRK_HIP(ffi::device_count(count), "hipGetDeviceCount");
    return kOk;
}
int mrk_hip_device_create(int device_id) {
    std::shared_ptr<Device> d;
    return get_device(device_id, &d);
}
int mrk_hip_device_create_by_type(const char* device_type, int device_id) {
    MRK_NONNULL(device_type);
    std::shared_ptr<Device> d;
    return DeviceFactoryRegistry::global().device(device_type, device_id, &d);
}
const char* mrk_hip_name(void) { return Device::base_device_key(); }
int mrk_hip_device_stream(int device_id, void** stream) {
    MRK_NONNULL(stream);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    *stream = d->allocator->stream();
    return kOk;
}

int mrk_hip_alloc(int device_id, size_t size, int zero_init, int cpu_accessible, void** out) {
    MRK_NONNULL(out);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    BufferOptions o;
    o.zero_init = zero_init != 0;
    o.cpu_accessible = cpu_accessible != 0;
    RawBuffer rb;
    MRK_TRY(d->allocator->alloc(size, o, &rb));
    *out = rb.ptr;
    return kOk;
}
int mrk_hip_free(int device_id, void* ptr, size_t size, int cpu_accessible) {
    if (!ptr) return kOk;
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    BufferOptions o;
    o.cpu_accessible = cpu_accessible != 0;
    RawBuffer rb;
    rb.ptr = ptr;
    rb.size = size;
    rb.cpu_accessible = o.cpu_accessible;
    d->allocator->free(rb, o);
    return kOk;
}
int mrk_hip_sync(int device_id) {
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    return d->allocator->synchronize();
}
int mrk_hip_lru_cache_count(int device_id, size_t size, int cpu_accessible, size_t* count) {
    MRK_NONNULL(count);
    LruAllocator* lru;
    MRK_TRY(get_lru(device_id, &lru));
    *count = lru->cache_count(size, cpu_accessible != 0);
    return kOk;
}
int mrk_hip_lru_total_cached(int device_id, size_t* count) {
    MRK_NONNULL(count);
    LruAllocator* lru;
    MRK_TRY(get_lru(device_id, &lru));
    *count = lru->total_cached();
    return kOk;
}
int mrk_hip_lru_clear(int device_id) {
    LruAllocator* lru;
    MRK_TRY(get_lru(device_id, &lru));
    lru->clear();
    return kOk;
}
int mrk_hip_copyin(int device_id, void* dst, size_t dst_offset, const void* src_host, size_t size) {
    if (size == 0) return kOk;
    MRK_NONNULL(dst);
    MRK_NONNULL(src_host);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    MRK_HIP(ffi::memcpy_htod_async(static_cast<char*>(dst) + dst_offset, src_host, size, d->allocator->stream()),
            "hipMemcpyAsync(HtoD)");
    MRK_HIP(ffi::stream_synchronize(d->allocator->stream()), "hipStreamSynchronize");
    return kOk;
}
int mrk_hip_copyout(int device_id, void* dst_host, const void* src, size_t src_offset, size_t size) {
    if (size == 0) return kOk;
    MRK_NONNULL(dst_host);
    MRK_NONNULL(src);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    MRK_HIP(ffi::memcpy_dtoh_async(dst_host, static_cast<const char*>(src) + src_offset, size, d->allocator->stream()),
            "hipMemcpyAsync(DtoH)");
    MRK_HIP(ffi::stream_synchronize(d->allocator->stream()), "hipStreamSynchronize");
    return kOk;
}
int mrk_hip_copy_dd(int device_id, void* dst, size_t dst_offset, const void* src, size_t src_offset, size_t size) {
    if (size == 0) return kOk;
    MRK_NONNULL(dst);
    MRK_NONNULL(src);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    MRK_HIP(ffi::memcpy_dtod_async(static_cast<char*>(dst) + dst_offset, static_cast<const char*>(src) + src_offset,
                                   size, d->allocator->stream()),
            "hipMemcpyAsync(DtoD)");
    return kOk;
}

int mrk_hip_buffer_new(int device_id, size_t size, int zero_init, int cpu_accessible, mrk_buffer** out) {
    MRK_NONNULL(out);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    BufferOptions o;
    o.zero_init = zero_init != 0;
    o.cpu_accessible = cpu_accessible != 0;
    auto* h = new mrk_buffer();
    h->b.reset(new Buffer(d->allocator, size, o));
    *out = h;
    return kOk;
}
int mrk_hip_buffer_ensure_allocated(mrk_buffer* b) {
    MRK_NONNULL(b);
    return b->b->ensure_allocated();
}
int mrk_hip_buffer_is_allocated(const mrk_buffer* b) { return b && b->b->is_allocated() ? 1 : 0; }
int mrk_hip_buffer_view(const mrk_buffer* b, size_t offset, size_t size, mrk_buffer** out) {
    MRK_NONNULL(b);
    MRK_NONNULL(out);
    std::unique_ptr<Buffer> v;
    MRK_TRY(b->b->view(offset, size, &v));
    auto* h = new mrk_buffer();
    h->b = std::move(v);
    *out = h;
    return kOk;
}
int mrk_hip_buffer_copyin(mrk_buffer* b, const void* src, size_t size) {
    MRK_NONNULL(b);
    if (size) MRK_NONNULL(src);
    return b->b->copyin(src, size);
}
int mrk_hip_buffer_copyout(const mrk_buffer* b, void* dst, size_t size) {
    MRK_NONNULL(b);
    if (size) MRK_NONNULL(dst);
    return b->b->copyout(dst, size);
}
int mrk_hip_buffer_copy_from(mrk_buffer* dst, const mrk_buffer* src) {
    MRK_NONNULL(dst);
    MRK_NONNULL(src);
    return dst->b->copy_from(*src->b);
}
int mrk_hip_buffer_raw_ptr(const mrk_buffer* b, void** out) {
    MRK_NONNULL(b);
    MRK_NONNULL(out);
    return b->b->as_raw_ptr(out);
}
uint64_t mrk_hip_buffer_id(const mrk_buffer* b) { return b ? b->b->id() : 0; }
size_t mrk_hip_buffer_size(const mrk_buffer* b) { return b ? b->b->size() : 0; }
int mrk_hip_buffer_synchronize(const mrk_buffer* b) {
    MRK_NONNULL(b);
    return b->b->synchronize();
}
void mrk_hip_buffer_release(mrk_buffer* b) { delete b; }

int mrk_hip_render(int device_id, const uint8_t* kernel, size_t len, const char* name, mrk_program_spec** out) {
    MRK_NONNULL(kernel);
    MRK_NONNULL(out);
    LinearKernel k;
    MRK_TRY(parse_linear_kernel(kernel, len, &k));
    // The renderer needs no device: rendering works on a host without a GPU.
    auto renderer = make_hip_renderer(device_id);
    auto* h = new mrk_program_spec();
    int rc = renderer->render(k, name, &h->s);
    if (rc != kOk) {
        delete h;
        return rc;
    }
    *out = h;
    return kOk;
}

int mrk_hip_program_spec_from_source(const char* name, const char* src, size_t buf_count, const char* const* var_names,
                                     const uint8_t* var_is_i64, size_t nvars, const size_t global_size[3],
                                     const size_t local_size[3], mrk_program_spec** out) {
    MRK_NONNULL(name);
    MRK_NONNULL(src);
    MRK_NONNULL(out);
    if (nvars) MRK_NONNULL(var_names);
    for (size_t i = 0; i < nvars; i++) MRK_NONNULL(var_names[i]);
    auto* h = new mrk_program_spec();
    h->s.name = name;
    h->s.src = src;
    h->s.buf_count = buf_count;
    for (size_t i = 0; i < nvars; i++) {
        h->s.var_names.push_back(var_names[i]);
        h->s.var_is_i64.push_back(var_is_i64 ? var_is_i64[i] : 0);
        h->s.vars.push_back(Variable{var_names[i], 0, 0});
    }
    if (global_size && local_size) {
        h->s.has_sizes = true;
        for (int i = 0; i < 3; i++) {
            h->s.global_size[i] = global_size[i];
            h->s.local_size[i] = local_size[i];
        }
    }
    for (size_t i = 0; i < buf_count; i++) h->s.globals.push_back(i);
    *out = h;
    return kOk;
}
const char* mrk_hip_program_spec_name(const mrk_program_spec* s) { return s ? s->s.name.c_str() : ""; }
const char* mrk_hip_program_spec_src(const mrk_program_spec* s) { return s ? s->s.src.c_str() : ""; }
size_t mrk_hip_program_spec_buf_count(const mrk_program_spec* s) { return s ? s->s.buf_count : 0; }
size_t mrk_hip_program_spec_var_count(const mrk_program_spec* s) { return s ? s->s.var_names.size() : 0; }
const char* mrk_hip_program_spec_var_name(const mrk_program_spec* s, size_t i) {
    return (s && i < s->s.var_names.size()) ? s->s.var_names[i].c_str() : "";
}
int mrk_hip_program_spec_sizes(const mrk_program_spec* s, size_t global_size[3], size_t local_size[3]) {
    if (!s || !s->s.has_sizes) return 0;
    for (int i = 0; i < 3; i++) {
        if (global_size) global_size[i] = s->s.global_size[i];
        if (local_size) local_size[i] = s->s.local_size[i];
    }
    return 1;
}
size_t mrk_hip_program_spec_slots(const mrk_program_spec* s, int which, size_t* out, size_t cap) {
    if (!s) return 0;
    const std::vector<size_t>& v = which == 0 ? s->s.globals : which == 1 ? s->s.outs : s->s.ins;
    for (size_t i = 0; i < v.size() && i < cap; i++) out[i] = v[i];
    return v.size();
}
void mrk_hip_program_spec_release(mrk_program_spec* s) { delete s; }

int mrk_hip_compile(const mrk_program_spec* spec, mrk_compiled_spec** out) {
    MRK_NONNULL(spec);
    MRK_NONNULL(out);
    auto compiler = make_hiprtc_compiler();
    auto* h = new mrk_compiled_spec();
    int rc = compiler->compile(spec->s, &h->c);
    if (rc != kOk) {
        delete h;
        return rc;
    }
    *out = h;
    return kOk;
}
const char* mrk_hip_cache_key(void) {
    static std::shared_ptr<Compiler> c = make_hiprtc_compiler();
    return c->cache_key();
}
const char* mrk_hip_compiled_spec_name(const mrk_compiled_spec* c) { return c ? c->c.name.c_str() : ""; }
size_t mrk_hip_compiled_spec_bytes(const mrk_compiled_spec* c, const uint8_t** bytes) {
    if (!c) return 0;
    if (bytes) *bytes = c->c.bytes.data();
    return c->c.bytes.size();
}
int mrk_hip_compiled_spec_has_src(const mrk_compiled_spec* c) { return c && c->c.has_src ? 1 : 0; }
void mrk_hip_compiled_spec_release(mrk_compiled_spec* c) { delete c; }

int mrk_hip_program_create(int device_id, const mrk_compiled_spec* spec, mrk_program** out) {
    MRK_NONNULL(spec);
    MRK_NONNULL(out);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    std::unique_ptr<Program> p;
    MRK_TRY(d->runtime(spec->c, &p));
    auto* h = new mrk_program();
    h->p = std::move(p);
    *out = h;
    return kOk;
}
int mrk_hip_program_execute(mrk_program* p, void* const* buffers, size_t nbufs, const int64_t* vals, size_t nvals,
                            const size_t global_size[3], const size_t local_size[3]) {
    MRK_NONNULL(p);
    if (nbufs) MRK_NONNULL(buffers);
    if (nvals) MRK_NONNULL(vals);
    return p->p->execute(buffers, nbufs, vals, nvals, global_size, local_size);
}
const char* mrk_hip_program_name(const mrk_program* p) { return p ? p->p->name() : ""; }
void mrk_hip_program_destroy(mrk_program* p) { delete p; }

int mrk_hip_program_builtin(int device_id, const char* kind, const int64_t* params, size_t nparams, mrk_program** out) {
    MRK_NONNULL(kind);
    MRK_NONNULL(out);
    if (nparams) MRK_NONNULL(params);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    std::unique_ptr<Program> p;
    MRK_TRY(create_builtin_program(device_id, d->allocator->stream(), kind, params, nparams, &p));
    auto* h = new mrk_program();
    h->p = std::move(p);
    *out = h;
    return kOk;
}

int mrk_hip_kernel_get_or_compile(int device_id, const uint8_t* kernel, size_t len, const char* name, mrk_kernel** out,
                                  int* was_cached) {
    MRK_NONNULL(kernel);
    MRK_NONNULL(out);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    LinearKernel k;
    MRK_TRY(parse_linear_kernel(kernel, len, &k));
    std::shared_ptr<CachedKernel> ck;
    bool cached = false;
    MRK_TRY(get_or_compile_linear_kernel(*d, k, name, &ck, &cached));
    if (was_cached) *was_cached = cached ? 1 : 0;
    *out = new mrk_kernel{ck};
    return kOk;
}
int mrk_hip_kernel_builtin(int device_id, const char* kind, const int64_t* params, size_t nparams, mrk_kernel** out) {
    MRK_NONNULL(kind);
    MRK_NONNULL(out);
    if (nparams) MRK_NONNULL(params);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    std::string key = std::string("builtin:") + kind;
    for (size_t i = 0; i < nparams; i++) key += ":" + std::to_string(params[i]);
    const std::string device = std::string("HIP:") + std::to_string(device_id);
    std::shared_ptr<CachedKernel> ck;
    MRK_TRY(KernelCache::global().get_or_compile(
        fnv1a64(reinterpret_cast<const uint8_t*>(key.data()), key.size()), device,
        [&](std::shared_ptr<CachedKernel>* fresh) -> int {
            std::unique_ptr<Program> p;
            MRK_TRY(create_builtin_program(device_id, d->allocator->stream(), kind, params, nparams, &p));
            auto k = std::make_shared<CachedKernel>();
            k->entry_point = p->name();
            k->program = std::move(p);
            k->device = device;
            *fresh = std::move(k);
            return kOk;
        },
        &ck));
    *out = new mrk_kernel{ck};
    return kOk;
}
const char* mrk_hip_kernel_entry_point(const mrk_kernel* k) { return k ? k->k->entry_point.c_str() : ""; }
const char* mrk_hip_kernel_code(const mrk_kernel* k) { return k ? k->k->code.c_str() : ""; }
size_t mrk_hip_kernel_var_count(const mrk_kernel* k) { return k ? k->k->var_names.size() : 0; }
const char* mrk_hip_kernel_var_name(const mrk_kernel* k, size_t i) {
    return (k && i < k->k->var_names.size()) ? k->k->var_names[i].c_str() : "";
}
int mrk_hip_kernel_same(const mrk_kernel* a, const mrk_kernel* b) { return a && b && a->k.get() == b->k.get(); }
void mrk_hip_kernel_release(mrk_kernel* k) { delete k; }
size_t mrk_hip_kernel_cache_size(void) { return KernelCache::global().size(); }
void mrk_hip_kernel_cache_clear(void) { KernelCache::global().clear_all(); }

int mrk_hip_plan_create(int device_id, mrk_plan** out) {
    MRK_NONNULL(out);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    auto* h = new mrk_plan();
    h->p.reset(new ExecutionPlan(device_id));
    *out = h;
    return kOk;
}
int mrk_hip_plan_add_buffer(mrk_plan* plan, const mrk_buffer* b, size_t* index) {
    MRK_NONNULL(plan);
    MRK_NONNULL(b);
    MRK_NONNULL(index);
    *index = plan->p->add_buffer(std::make_shared<Buffer>(*b->b));
    return kOk;
}
int mrk_hip_plan_add_kernel(mrk_plan* plan, const mrk_kernel* k, const size_t* buffer_indices, size_t nbufs,
                            const int64_t* vals, size_t nvals) {
    MRK_NONNULL(plan);
    MRK_NONNULL(k);
    if (nbufs) MRK_NONNULL(buffer_indices);
    if (nvals) MRK_NONNULL(vals);
    return plan->p->add_kernel(k->k, std::vector<size_t>(buffer_indices, buffer_indices + nbufs),
                               std::vector<int64_t>(vals, vals + nvals));
}
int mrk_hip_plan_build(mrk_plan* plan) {
    MRK_NONNULL(plan);
    return plan->p->build();
}
int mrk_hip_plan_execute(mrk_plan* plan) {
    MRK_NONNULL(plan);
    return plan->p->execute();
}
int mrk_hip_plan_execute_graph(mrk_plan* plan) {
    MRK_NONNULL(plan);
    return plan->p->execute_graph();
}
int mrk_hip_plan_execute_profiled(mrk_plan* plan, double* elapsed_ms, size_t cap, size_t* count) {
    MRK_NONNULL(plan);
    std::vector<KernelProfile> prof;
    MRK_TRY(plan->p->execute_profiled(&prof));
    if (count) *count = prof.size();
    for (size_t i = 0; i < prof.size() && i < cap && elapsed_ms; i++) elapsed_ms[i] = prof[i].elapsed_ms;
    return kOk;
}
int mrk_hip_plan_execute_with_vars(mrk_plan* plan, const char* const* names, const int64_t* vals, size_t n) {
    MRK_NONNULL(plan);
    if (n) {
        MRK_NONNULL(names);
        MRK_NONNULL(vals);
    }
    std::vector<std::pair<std::string, int64_t>> kv;
    for (size_t i = 0; i < n; i++) {
        MRK_NONNULL(names[i]);
        kv.emplace_back(names[i], vals[i]);
    }
    return plan->p->execute_with_vars(kv);
}
size_t mrk_hip_plan_kernel_count(const mrk_plan* plan) { return plan ? plan->p->kernel_count() : 0; }
const char* mrk_hip_plan_kernel_name(const mrk_plan* plan, size_t i) {
    return (plan && i < plan->p->kernel_count()) ? plan->p->kernel(i).kernel->entry_point.c_str() : "";
}
void mrk_hip_plan_release(mrk_plan* plan) { delete plan; }

int mrk_hip_benchmark_kernel(int device_id, mrk_program* p, void* const* buffers, size_t nbufs, const int64_t* vals,
                             size_t nvals, const size_t global_size[3], const size_t local_size[3], int warmup, int runs,
                             double* min_ms, double* mean_ms) {
    MRK_NONNULL(p);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    BenchmarkResult r;
    MRK_TRY(benchmark_kernel(device_id, d->allocator->stream(), p->p.get(), buffers, nbufs, vals, nvals, global_size,
                             local_size, warmup, runs, &r));
    if (min_ms) *min_ms = r.min_ms;
    if (mean_ms) *mean_ms = r.mean_ms;
    return kOk;
}

int mrk_hip_benchmark_kernel_with_cutoff(int device_id, mrk_program* p, void* const* buffers, size_t nbufs, const int64_t* vals,
                                         size_t nvals, const size_t global_size[3], const size_t local_size[3], int warmup,
                                         int runs, double cutoff_ms, double* min_ms, double* mean_ms, int* skipped) {
    MRK_NONNULL(p);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    BenchmarkResult r;
    bool sk = false;
    MRK_TRY(benchmark_kernel_with_cutoff(device_id, d->allocator->stream(), p->p.get(), buffers, nbufs, vals, nvals, global_size,
                                         local_size, warmup, runs, cutoff_ms, &r, &sk));
    if (min_ms) *min_ms = r.min_ms;
    if (mean_ms) *mean_ms = r.mean_ms;
    if (skipped) *skipped = sk ? 1 : 0;
    return kOk;
}

int mrk_hip_signal_create(int device_id, mrk_signal** out) {
    MRK_NONNULL(out);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    auto* h = new mrk_signal();
    h->s.reset(new TimelineSignal(device_id, d->allocator->stream()));
    *out = h;
    return kOk;
}
int mrk_hip_signal_set(mrk_signal* s, uint64_t value) {
    MRK_NONNULL(s);
    return s->s->set(value);
}
uint64_t mrk_hip_signal_value(mrk_signal* s) { return s ? s->s->value() : 0; }
int mrk_hip_signal_wait(mrk_signal* s, uint64_t value, uint64_t timeout_ms) {
    MRK_NONNULL(s);
    return s->s->wait(value, timeout_ms);
}
void mrk_hip_signal_destroy(mrk_signal* s) { delete s; }

// ---- hardware queues
int mrk_hip_queue_create(int device_id, int copy_queue, mrk_queue** out) {
    MRK_NONNULL(out);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    std::unique_ptr<HardwareQueue> q(new HardwareQueue(device_id, copy_queue != 0));
    MRK_TRY(q->init());
    *out = new mrk_queue{std::move(q)};
    return kOk;
}
int mrk_hip_queue_wait(mrk_queue* q, mrk_signal* s, uint64_t value) {
    MRK_NONNULL(q);
    MRK_NONNULL(s);
    q->q->wait(s->s, value);
    return kOk;
}
int mrk_hip_queue_signal(mrk_queue* q, mrk_signal* s, uint64_t value) {
    MRK_NONNULL(q);
    MRK_NONNULL(s);
    q->q->signal(s->s, value);
    return kOk;
}
int mrk_hip_queue_exec(mrk_queue* q, const mrk_kernel* k, mrk_buffer* const* buffers, size_t nbufs, const int64_t* vals,
                       size_t nvals, const size_t* global, const size_t* local) {
    MRK_NONNULL(q);
    MRK_NONNULL(k);
    if (nbufs) MRK_NONNULL(buffers);
    if (nvals) MRK_NONNULL(vals);
    std::vector<std::shared_ptr<Buffer>> bufs;
    for (size_t i = 0; i < nbufs; i++) {
        MRK_NONNULL(buffers[i]);
        bufs.push_back(std::make_shared<Buffer>(*buffers[i]->b));
    }
    q->q->exec(k->k, std::move(bufs), std::vector<int64_t>(vals, vals + nvals), global, local);
    return kOk;
}
int mrk_hip_queue_copy(mrk_queue* q, mrk_buffer* dst, const mrk_buffer* src) {
    MRK_NONNULL(q);
    MRK_NONNULL(dst);
    MRK_NONNULL(src);
    q->q->copy(std::make_shared<Buffer>(*dst->b), std::make_shared<Buffer>(*src->b));
    return kOk;
}
int mrk_hip_queue_memory_barrier(mrk_queue* q) {
    MRK_NONNULL(q);
    q->q->memory_barrier();
    return kOk;
}
int mrk_hip_queue_submit(mrk_queue* q, uint64_t wait_timeout_ms) {
    MRK_NONNULL(q);
    return q->q->submit(wait_timeout_ms);
}
int mrk_hip_queue_synchronize(mrk_queue* q) {
    MRK_NONNULL(q);
    return q->q->synchronize();
}
size_t mrk_hip_queue_pending(const mrk_queue* q) { return q ? q->q->pending_commands() : 0; }
void mrk_hip_queue_destroy(mrk_queue* q) { delete q; }

// ---- scheduling helpers
size_t mrk_hip_sched_find_smallest_divisor(size_t n) { return find_smallest_divisor(n); }
static int put_dims(const std::vector<size_t>& v, size_t* out, size_t cap, size_t* n) {
    if (n) *n = v.size();
    for (size_t i = 0; i < v.size() && i < cap && out; i++) out[i] = v[i];
    return kOk;
}
int mrk_hip_sched_group_dims(const size_t* dims, size_t n, const size_t* max_sizes, size_t nmax, size_t* out, size_t cap,
                             size_t* nout) {
    std::vector<size_t> r;
    if (!group_dims(std::vector<size_t>(dims, dims + n), std::vector<size_t>(max_sizes, max_sizes + nmax), &r)) return 0;
    put_dims(r, out, cap, nout);
    return 1;
}
int mrk_hip_sched_split_dims(const size_t* dims, size_t n, const size_t* max_sizes, size_t nmax, size_t* out, size_t cap,
                             size_t* nout) {
    return put_dims(split_dims(std::vector<size_t>(dims, dims + n), std::vector<size_t>(max_sizes, max_sizes + nmax)), out,
                    cap, nout);
}
int mrk_hip_sched_limit_dims(const size_t* dims, size_t n, const size_t* max_sizes, size_t nmax, size_t* out, size_t cap,
                             size_t* nout) {
    return put_dims(limit_dims(std::vector<size_t>(dims, dims + n), std::vector<size_t>(max_sizes, max_sizes + nmax)), out,
                    cap, nout);
}
int mrk_hip_sched_get_contraction(const size_t* original, size_t n, const size_t* limited, size_t nl, size_t* group_of_dim) {
    std::vector<std::vector<size_t>> c;
    if (!get_contraction(std::vector<size_t>(original, original + n), std::vector<size_t>(limited, limited + nl), &c)) return 0;
    for (size_t g = 0; g < c.size(); g++)
        for (size_t d : c[g])
            if (group_of_dim) group_of_dim[d] = g;
    return 1;
}
int mrk_hip_sched_grouped_dims(const size_t* dims, size_t n, const size_t* max_sizes, size_t nmax, int reverse,
                               size_t* launch, size_t cap, size_t* nlaunch, const size_t* raw, size_t* index_per_dim) {
    std::vector<size_t> mx(max_sizes, max_sizes + nmax);
    if (reverse < 0 || reverse > 2) return fail(kInvalidArgument, "grouped_dims: reverse must be 0, 1 or 2");
    GroupedDims g = get_grouped_dims(std::vector<size_t>(dims, dims + n), max_sizes ? &mx : nullptr, static_cast<DimOrder>(reverse));
    put_dims(g.launch, launch, cap, nlaunch);
    if (raw && index_per_dim) {
        std::vector<size_t> r(raw, raw + g.launch.size());
        for (size_t i = 0; i < r.size(); i++)
            if (r[i] >= g.launch[i]) return fail(kInvalidArgument, "grouped_dims: raw index out of range");
        std::vector<size_t> m = g.map(r);
        for (size_t i = 0; i < m.size(); i++) index_per_dim[i] = m[i];
    }
    return kOk;
}
const char* mrk_hip_sched_caps(void) {
    static std::string desc = [] {
        RendererCaps c = amd_cdna4_caps();
        std::string s = "device=" + c.device + ";has_local=" + std::to_string(c.has_local) +
                        ";has_shared=" + std::to_string(c.has_shared) + ";has_threads=" + std::to_string(c.has_threads) +
                        ";shared_max=" + std::to_string(c.shared_max) + ";global_max=";
        for (size_t i = 0; i < c.global_max.size(); i++) s += (i ? "," : "") + std::to_string(c.global_max[i]);
        s += ";local_max=" + std::to_string(c.local_max) + ";upcast_max=" + std::to_string(c.upcast_max) + ";tensor_cores=";
        for (size_t i = 0; i < c.tensor_cores.size(); i++) s += (i ? "," : "") + wmma_name(c.tensor_cores[i]);
        return s;
    }();
    return desc.c_str();
}
int mrk_hip_sched_tc_select(int in0_scalar, int in1_scalar, int acc_scalar) {
    return select_tensor_core(cdna4_tensor_cores(), static_cast<Scalar>(in0_scalar), static_cast<Scalar>(in1_scalar),
                              static_cast<Scalar>(acc_scalar));
}
int mrk_hip_sched_tc_info(int tc_index, int dims[3], int* threads, int elements_per_thread[3]) {
    auto tcs = cdna4_tensor_cores();
    if (tc_index < 0 || tc_index >= (int)tcs.size()) return fail(kInvalidArgument, "tc index out of range");
    for (int i = 0; i < 3; i++) {
        if (dims) dims[i] = tcs[tc_index].dims[i];
        if (elements_per_thread) elements_per_thread[i] = tcs[tc_index].elements_per_thread[i];
    }
    if (threads) *threads = tcs[tc_index].threads;
    return kOk;
}
int mrk_hip_sched_tc_operand_element(int tc_index, int operand, int lane, int elem, int* mn, int* k) {
    auto tcs = cdna4_tensor_cores();
    if (tc_index < 0 || tc_index >= (int)tcs.size() || operand < 0 || operand > 2)
        return fail(kInvalidArgument, "tc index or operand out of range");
    if (operand == 2) tc_acc_element(tcs[tc_index], lane, elem, mn, k);
    else tc_operand_element(tcs[tc_index], operand, lane, elem, mn, k);
    return kOk;
}
static int export_kernel(const LinearKernel& k, KernelBuilder* /*unused*/, const std::vector<uint8_t>& bytes, uint8_t** out,
                         size_t* len) {
    (void)k;
    uint8_t* p = static_cast<uint8_t*>(std::malloc(bytes.size() ? bytes.size() : 1));
    if (!p) return fail(kRuntime, "out of host memory");
    std::memcpy(p, bytes.data(), bytes.size());
    *out = p;
    *len = bytes.size();
    return kOk;
}
static std::vector<uint8_t> reserialize(const LinearKernel& k) {
    KernelBuilder b;
    for (const UOp& u : k.nodes) b.add(u.op, u.dtype, u.src, u.arg_i, u.arg_f, u.sub, u.str, u.extra);
    return b.serialize();
}
int mrk_hip_sched_build_matmul_f32(int64_t m, int64_t n, int64_t k, uint8_t** kernel, size_t* len) {
    MRK_NONNULL(kernel);
    MRK_NONNULL(len);
    if (m <= 0 || n <= 0 || k < 0 || m % 64 || n % 64)
        return fail(kInvalidArgument, "matmul_f32 kernel: M and N must be positive multiples of 64");
    LinearKernel lk = build_matmul_f32_kernel(m, n, k);
    return export_kernel(lk, nullptr, reserialize(lk), kernel, len);
}
int mrk_hip_sched_build_wmma_matmul(int tc_index, int64_t m, int64_t n, int64_t k, int out_scalar, uint8_t** kernel,
                                    size_t* len) {
    MRK_NONNULL(kernel);
    MRK_NONNULL(len);
    auto tcs = cdna4_tensor_cores();
    if (tc_index < 0 || tc_index >= (int)tcs.size()) return fail(kInvalidArgument, "tc index out of range");
    LinearKernel lk;
    MRK_TRY(build_wmma_matmul_kernel(tcs[tc_index], m, n, k, static_cast<Scalar>(out_scalar), &lk));
    return export_kernel(lk, nullptr, reserialize(lk), kernel, len);
}
int mrk_hip_sched_build_wmma_matmul_lds(int tc_index, int64_t m, int64_t n, int64_t k, int out_scalar, uint8_t** kernel,
                                        size_t* len) {
    MRK_NONNULL(kernel);
    MRK_NONNULL(len);
    auto tcs = cdna4_tensor_cores();
    if (tc_index < 0 || tc_index >= (int)tcs.size()) return fail(kInvalidArgument, "tc index out of range");
    LinearKernel lk;
    MRK_TRY(build_wmma_matmul_lds_kernel(tcs[tc_index], m, n, k, static_cast<Scalar>(out_scalar), WmmaLdsOpts(), &lk));
    return export_kernel(lk, nullptr, reserialize(lk), kernel, len);
}
int mrk_hip_sched_build_wmma_matmul_lds_opts(int tc_index, int64_t m, int64_t n, int64_t k, int out_scalar, const int opts[6],
                                             uint8_t** kernel, size_t* len) {
    MRK_NONNULL(opts);
    MRK_NONNULL(kernel);
    MRK_NONNULL(len);
    auto tcs = cdna4_tensor_cores();
    if (tc_index < 0 || tc_index >= (int)tcs.size()) return fail(kInvalidArgument, "tc index out of range");
    WmmaLdsOpts o{opts[0], opts[1], opts[2], opts[3], opts[4], opts[5]};
    LinearKernel lk;
    MRK_TRY(build_wmma_matmul_lds_kernel(tcs[tc_index], m, n, k, static_cast<Scalar>(out_scalar), o, &lk));
    return export_kernel(lk, nullptr, reserialize(lk), kernel, len);
}
void mrk_hip_sched_free(void* p) { std::free(p); }
int mrk_hip_sched_build_matmul_f32_opts(int64_t m, int64_t n, int64_t k, const int opts[6], uint8_t** kernel, size_t* len) {
    MRK_NONNULL(opts);
    MRK_NONNULL(kernel);
    MRK_NONNULL(len);
    MatmulF32Opts o{opts[0], opts[1], opts[2], opts[3], opts[4], opts[5]};
    if (!matmul_f32_opts_valid(o, m, n, k))
        return fail(kInvalidArgument, "matmul f32: LOCAL/UPCAST/UNROLL/GROUP choices do not fit the shape");
    LinearKernel lk = build_matmul_f32_kernel(m, n, k, o);
    return export_kernel(lk, nullptr, reserialize(lk), kernel, len);
}

int mrk_hip_compile_and_time(int device_id, const void* kernel, size_t len, const char* name, mrk_buffer* const* buffers,
                             size_t nbufs, const int64_t* vals, size_t nvals, int warmup, int runs, double* min_ms) {
    MRK_NONNULL(kernel);
    MRK_NONNULL(min_ms);
    if (nbufs) MRK_NONNULL(buffers);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    LinearKernel k;
    MRK_TRY(parse_linear_kernel(static_cast<const uint8_t*>(kernel), len, &k));
    std::vector<void*> ptrs(nbufs);
    for (size_t i = 0; i < nbufs; i++) {
        MRK_NONNULL(buffers[i]);
        MRK_TRY(buffers[i]->b->ensure_allocated());
        MRK_TRY(buffers[i]->b->as_raw_ptr(&ptrs[i]));
    }
    BenchmarkResult r;
    MRK_TRY(compile_and_time(*d, k, name, ptrs.data(), nbufs, vals, nvals, warmup, runs, &r));
    *min_ms = r.min_ms;
    return kOk;
}
int mrk_hip_beam_cache_get(uint64_t ast_hash, int width, const char* device, void* value, size_t capacity, size_t* len) {
    MRK_NONNULL(device);
    MRK_NONNULL(len);
    std::vector<uint8_t> v;
    *len = 0;
    if (!BeamCache::get(ast_hash, width, device, &v)) return kOk;
    if (v.size() > capacity) return fail(kInvalidArgument, "beam cache: value larger than the buffer");
    if (!v.empty()) {
        MRK_NONNULL(value);
        std::memcpy(value, v.data(), v.size());
    }
    *len = v.size();
    return kOk;
}
int mrk_hip_beam_cache_put(uint64_t ast_hash, int width, const char* device, const void* value, size_t len) {
    MRK_NONNULL(device);
    if (len) MRK_NONNULL(value);
    return BeamCache::put(ast_hash, width, device, value, len);
}
int mrk_hip_beam_search_matmul_f32(int device_id, int64_t m, int64_t n, int64_t k, int width, int opts[6],
                                   double* best_ms, int* from_cache, int* timed) {
    MRK_NONNULL(opts);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    MatmulF32Opts o;
    bool cached = false;
    int n_timed = 0;
    double ms = 0;
    MRK_TRY(beam_search_matmul_f32(*d, m, n, k, width, &o, &ms, &cached, &n_timed));
    opts[0] = o.local_x;
    opts[1] = o.local_y;
    opts[2] = o.up_n;
    opts[3] = o.up_m;
    opts[4] = o.unroll_k;
    opts[5] = o.lds_k;
    if (best_ms) *best_ms = ms;
    if (from_cache) *from_cache = cached ? 1 : 0;
    if (timed) *timed = n_timed;
    return kOk;
}

int mrk_hip_beam_search_wmma_matmul(int device_id, int tc_index, int64_t m, int64_t n, int64_t k, int width, int opts[6],
                                    double* best_ms, int* from_cache, int* timed) {
    MRK_NONNULL(opts);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    auto tcs = cdna4_tensor_cores();
    if (tc_index < 0 || tc_index >= (int)tcs.size()) return fail(kInvalidArgument, "tc index out of range");
    WmmaLdsOpts o;
    bool cached = false;
    int n_timed = 0;
    double ms = 0;
    MRK_TRY(beam_search_wmma_matmul(*d, tcs[tc_index], tc_index, m, n, k, width, &o, &ms, &cached, &n_timed));
    opts[0] = o.waves_m;
    opts[1] = o.waves_n;
    opts[2] = o.up_m;
    opts[3] = o.up_n;
    opts[4] = o.unroll_k;
    opts[5] = o.stages;
    if (best_ms) *best_ms = ms;
    if (from_cache) *from_cache = cached ? 1 : 0;
    if (timed) *timed = n_timed;
    return kOk;
}

int mrk_hip_softmax_f32_variant(int device_id, const void* x, void* y, int64_t rows, int64_t cols, int variant) {
    if (rows < 0 || cols < 0) return fail(kInvalidArgument, "softmax_f32: negative shape");
    if (rows == 0 || cols == 0) return kOk;
    MRK_NONNULL(x);
    MRK_NONNULL(y);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    MRK_HIP(launch_softmax_f32(d->allocator->stream(), x, y, rows, cols, variant), "softmax_f32 launch");
    return kOk;
}
int mrk_hip_softmax_f32(int device_id, const void* x, void* y, int64_t rows, int64_t cols) {
    return mrk_hip_softmax_f32_variant(device_id, x, y, rows, cols, 0);
}

static int gemm_16bit(int device_id, const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k, int variant, bool f16) {
    if (m < 0 || n < 0 || k < 0) return fail(kInvalidArgument, f16 ? "gemm_f16: negative shape" : "gemm_bf16: negative shape");
    if (m == 0 || n == 0) return kOk;
    MRK_NONNULL(c);
    if (k > 0) {
        MRK_NONNULL(a);
        MRK_NONNULL(b);
    }
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    // Few output tiles against a long K: scratch for split-K partials comes from the device's
    // allocator (kept in its LRU cache between calls) and goes back right after the launch; the
    // next user of the block queues behind this product on the same in-order stream.
    const size_t ws = variant == 0 ? gemm_bf16_workspace_bytes(m, n, k, 1) : 0;
    RawBuffer scratch;
    BufferOptions so;
    if (ws) MRK_TRY(d->allocator->alloc(ws, so, &scratch));
    int rc = launch_gemm_bf16(d->allocator->stream(), a, b, c, m, n, k, variant, 1, ws ? scratch.ptr : nullptr, ws, false, f16);
    if (ws) d->allocator->free(scratch, so);
    MRK_HIP(rc, f16 ? "gemm_f16 launch" : "gemm_bf16 launch");
    return kOk;
}
int mrk_hip_gemm_bf16_variant(int device_id, const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k,
                               int variant) {
    return gemm_16bit(device_id, a, b, c, m, n, k, variant, false);
}
int mrk_hip_gemm_f16(int device_id, const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k) {
    return gemm_16bit(device_id, a, b, c, m, n, k, 0, true);
}
size_t mrk_hip_gemm_bf16_workspace_bytes(int64_t m, int64_t n, int64_t k, int64_t batch) {
    return gemm_bf16_workspace_bytes(m, n, k, batch);
}
int mrk_hip_gemm_bf16(int device_id, const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k) {
    return mrk_hip_gemm_bf16_variant(device_id, a, b, c, m, n, k, 0);
}

static int gemm_16bit_nt(int device_id, const void* a, const void* bt, void* c, int64_t m, int64_t n, int64_t k, bool f16);
int mrk_hip_gemm_bf16_nt(int device_id, const void* a, const void* bt, void* c, int64_t m, int64_t n, int64_t k) {
    return gemm_16bit_nt(device_id, a, bt, c, m, n, k, false);
}
int mrk_hip_gemm_f16_nt(int device_id, const void* a, const void* bt, void* c, int64_t m, int64_t n, int64_t k) {
    return gemm_16bit_nt(device_id, a, bt, c, m, n, k, true);
}
static int gemm_16bit_nt(int device_id, const void* a, const void* bt, void* c, int64_t m, int64_t n, int64_t k, bool f16) {
    if (m < 0 || n < 0 || k < 0) return fail(kInvalidArgument, "gemm_bf16_nt: negative shape");
    if (m == 0 || n == 0) return kOk;
    MRK_NONNULL(a);
    MRK_NONNULL(bt);
    MRK_NONNULL(c);
    if (!gemm_bf16_nt_supported(m, n, k, 1))
        return fail(kInvalidArgument, "gemm_bf16_nt: shape not covered for a second operand stored [N, K] (K a multiple of 8, K > 0; "
                                      "at most 64 rows, or N a multiple of 8); transpose it and run mrk_hip_gemm_bf16");
    std::shared_ptr<Device> dv;
    MRK_TRY(get_device(device_id, &dv));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    // few output tiles against a long K, more than 64 rows: scratch for split-K partials, as for the [K, N] form
    const size_t ws = gemm_bf16_nt_workspace_bytes(m, n, k, 1);
    RawBuffer scratch;
    BufferOptions so;
    if (ws) MRK_TRY(dv->allocator->alloc(ws, so, &scratch));
    int rc = launch_gemm_bf16(dv->allocator->stream(), a, bt, c, m, n, k, 0, 1, ws ? scratch.ptr : nullptr, ws, true, f16);
    if (ws) dv->allocator->free(scratch, so);
    MRK_HIP(rc, "gemm_bf16_nt launch");
    return kOk;
}

int mrk_hip_gemm_bf16_rope(int device_id, const void* a, const void* b, const void* cos, const void* sin, void* c_rot, void* c_rest,
                           int64_t m, int64_t n, int64_t k, int64_t split, int64_t seq) {
    if (m < 0 || n < 0 || k < 0) return fail(kInvalidArgument, "gemm_bf16_rope: negative shape");
    if (m == 0 || n == 0) return kOk;
    MRK_NONNULL(a);
    MRK_NONNULL(b);
    MRK_NONNULL(cos);
    MRK_NONNULL(sin);
    MRK_NONNULL(c_rot);
    if (!gemm_bf16_rope_supported(m, n, k, split, seq))
        return fail(kInvalidArgument, "gemm_bf16_rope: shape not covered by the rotary epilogue (K a multiple of 64, N of 8, split a multiple of "
                                      "256 within N, seq > 0); run mrk_hip_gemm_bf16 and rotate separately");
    if (split < n) MRK_NONNULL(c_rest);
    std::shared_ptr<Device> dv;
    MRK_TRY(get_device(device_id, &dv));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    MRK_HIP(launch_gemm_bf16_rope(dv->allocator->stream(), a, b, c_rot, c_rest, m, n, k, split, cos, sin, seq), "gemm_bf16_rope launch");
    return kOk;
}

int mrk_hip_gemm_bf16_swiglu(int device_id, const void* a, const void* w, void* c, int64_t m, int64_t f, int64_t k) {
    if (m < 0 || f < 0 || k < 0) return fail(kInvalidArgument, "gemm_bf16_swiglu: negative shape");
    if (m == 0 || f == 0) return kOk;
    MRK_NONNULL(a);
    MRK_NONNULL(w);
    MRK_NONNULL(c);
    if (!gemm_bf16_swiglu_supported(m, f, k))
        return fail(kInvalidArgument, "gemm_bf16_swiglu: shape not covered by the gated epilogue (F and K multiples of 8, K > 0); run "
                                      "mrk_hip_gemm_bf16 on the [K, 2F] matrix and apply the gate separately");
    std::shared_ptr<Device> dv;
    MRK_TRY(get_device(device_id, &dv));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    MRK_HIP(launch_gemm_bf16_swiglu(dv->allocator->stream(), a, w, c, m, f, k), "gemm_bf16_swiglu launch");
    return kOk;
}
size_t mrk_hip_gemm_bf16_noalloc_capacity(void) { return gemm_bf16_static_workspace_capacity(); }
int mrk_hip_gemm_bf16_noalloc(int device_id, const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k) {
    if (m < 0 || n < 0 || k < 0) return fail(kInvalidArgument, "gemm_bf16_noalloc: negative shape");
    if (m == 0 || n == 0) return kOk;
    MRK_NONNULL(c);
    if (k > 0) {
        MRK_NONNULL(a);
        MRK_NONNULL(b);
    }
    // lookup only: creating a device allocates (streams, the allocator), which this call must not
    std::shared_ptr<Device> d = DeviceFactoryRegistry::global().find("HIP", device_id);
    if (!d)
        return failf(kInvalidArgument, "gemm_bf16_noalloc: device HIP:%d has not been created; call mrk_hip_device_create "
                                       "during set-up (this entry point allocates nothing, device creation does)", device_id);
    const size_t need = gemm_bf16_workspace_bytes(m, n, k, 1);
    if (need > gemm_bf16_static_workspace_capacity())
        return failf(kInvalidArgument, "gemm_bf16_noalloc: %lldx%lldx%lld needs %zu bytes of split-K scratch, the built-in "
                                       "scratch holds %zu; use mrk_hip_gemm_bf16", (long long)m, (long long)n, (long long)k,
                     need, gemm_bf16_static_workspace_capacity());
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    MRK_HIP(launch_gemm_bf16_static_ws(d->allocator->stream(), device_id, a, b, c, m, n, k), "gemm_bf16_noalloc launch");
    return kOk;
}

int mrk_hip_gemm_bf16_residual(int device_id, const void* a, const void* b, const void* r, void* c, int64_t m, int64_t n, int64_t k) {
    if (m < 0 || n < 0 || k < 0) return fail(kInvalidArgument, "gemm_bf16_residual: negative shape");
    if (m == 0 || n == 0) return kOk;
    MRK_NONNULL(a);
    MRK_NONNULL(b);
    MRK_NONNULL(r);
    MRK_NONNULL(c);
    if (!gemm_bf16_residual_supported(m, n, k, 1))
        return fail(kInvalidArgument, "gemm_bf16_residual: shape not covered by the fused epilogue (N and K multiples of 8, K > 0); "
                                      "run mrk_hip_gemm_bf16 and add separately");
    std::shared_ptr<Device> dv;
    MRK_TRY(get_device(device_id, &dv));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    // few output tiles against a long K: scratch for the partial results, as for the plain product
    const size_t ws = gemm_bf16_workspace_bytes(m, n, k, 1);
    RawBuffer scratch;
    BufferOptions so;
    if (ws) MRK_TRY(dv->allocator->alloc(ws, so, &scratch));
    int rc = launch_gemm_bf16_residual(dv->allocator->stream(), a, b, r, c, m, n, k, 1, false, false, ws ? scratch.ptr : nullptr, ws);
    if (ws) dv->allocator->free(scratch, so);
    MRK_HIP(rc, "gemm_bf16_residual launch");
    return kOk;
}

int mrk_hip_linear_bf16(int device_id, const void* x, const void* w, const void* bias, void* y, int64_t m, int64_t n, int64_t k) {
    if (!bias) return mrk_hip_gemm_bf16_nt(device_id, x, w, y, m, n, k);
    if (m < 0 || n < 0 || k < 0) return fail(kInvalidArgument, "linear_bf16: negative shape");
    if (m == 0 || n == 0) return kOk;
    MRK_NONNULL(x);
    MRK_NONNULL(w);
    MRK_NONNULL(y);
    if (!gemm_bf16_nt_supported(m, n, k, 1))
        return fail(kInvalidArgument, "linear_bf16: shape not covered (in_features a multiple of 8 and > 0; at most 64 rows, or "
                                      "out_features a multiple of 8)");
    std::shared_ptr<Device> dv;
    MRK_TRY(get_device(device_id, &dv));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    const size_t ws = gemm_bf16_nt_workspace_bytes(m, n, k, 1);
    RawBuffer scratch;
    BufferOptions so;
    if (ws) MRK_TRY(dv->allocator->alloc(ws, so, &scratch));
    int rc = launch_gemm_bf16_bias(dv->allocator->stream(), x, w, bias, y, m, n, k, 1, true, ws ? scratch.ptr : nullptr, ws);
    if (ws) dv->allocator->free(scratch, so);
    MRK_HIP(rc, "linear_bf16 launch");
    return kOk;
}

int mrk_hip_flash_attn_fwd_bf16(int device_id, const void* q, const void* k, const void* v, void* o, int64_t batch,
                                int64_t heads, int64_t sq, int64_t sk, int64_t d, float scale, int causal) {
    if (batch < 0 || heads < 0 || sq < 0 || sk < 0) return fail(kInvalidArgument, "flash_attn_fwd: negative shape");
    if (batch == 0 || heads == 0 || sq == 0) return kOk;
    if (d != 256 && d != 128 && d != 64) return failf(kInvalidArgument, "flash_attn_fwd: head_dim %lld is not supported (256, 128 and 64 only)", (long long)d);
    if (sk == 0) return fail(kInvalidArgument, "flash_attn_fwd: empty key sequence (softmax over no keys is undefined)");
    if (!(scale > 0.0f)) return fail(kInvalidArgument, "flash_attn_fwd: scale must be positive");
    if (!flash_fwd_rows_addressable(sq, d * 2, d) || !flash_fwd_rows_addressable(sk, d * 2, d))
        return failf(kInvalidArgument, "flash_attn_fwd: the rows of one (batch, head) must end below 4 GiB (row offsets are 32-bit): "
                                       "at head_dim %lld at most %lld rows", (long long)d, (long long)((0xffffffffLL - d * 2) / (d * 2) + 1));
    MRK_NONNULL(q);
    MRK_NONNULL(k);
    MRK_NONNULL(v);
    MRK_NONNULL(o);
    std::shared_ptr<Device> dv;
    MRK_TRY(get_device(device_id, &dv));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    // a handful of queries against many keys: the key sequence is split over workgroups, the ranges' partial
    // results go through scratch from the device's allocator (as for the products' split-K)
    const size_t ws = flash_fwd_workspace_bytes(batch * heads, sq, sk, d, causal ? 1 : 0);
    RawBuffer scratch;
    BufferOptions so;
    if (ws) MRK_TRY(dv->allocator->alloc(ws, so, &scratch));
    const int rc = launch_flash_fwd_bf16(dv->allocator->stream(), q, k, v, o, batch * heads, sq, sk, d, scale, causal ? 1 : 0,
                                         ws ? scratch.ptr : nullptr, ws);
    if (ws) dv->allocator->free(scratch, so);
    MRK_HIP(rc, "flash_attn_fwd launch");
    return kOk;
}
size_t mrk_hip_flash_attn_workspace_bytes(int64_t batch, int64_t heads, int64_t sq, int64_t sk, int64_t d, int causal) {
    if (batch <= 0 || heads <= 0) return 0;
    return flash_fwd_workspace_bytes(batch * heads, sq, sk, d, causal ? 1 : 0);
}

int mrk_hip_flash_attn_fwd_bf16_strided(int device_id, const void* q, const void* k, const void* v, void* o, int64_t batch,
                                        int64_t heads, int64_t sq, int64_t sk, int64_t d, float scale, int causal,
                                        const int64_t* strides) {
    if (batch < 0 || heads < 0 || sq < 0 || sk < 0) return fail(kInvalidArgument, "flash_attn_fwd_strided: negative shape");
    if (batch == 0 || heads == 0 || sq == 0) return kOk;
    if (d != 256 && d != 128 && d != 64) return failf(kInvalidArgument, "flash_attn_fwd_strided: head_dim %lld is not supported (256, 128 and 64 only)", (long long)d);
    if (sk == 0) return fail(kInvalidArgument, "flash_attn_fwd_strided: empty key sequence (softmax over no keys is undefined)");
    if (!(scale > 0.0f)) return fail(kInvalidArgument, "flash_attn_fwd_strided: scale must be positive");
    MRK_NONNULL(q);
    MRK_NONNULL(k);
    MRK_NONNULL(v);
    MRK_NONNULL(o);
    MRK_NONNULL(strides);
    long st[12];
    for (int i = 0; i < 12; i++) {
        if (strides[i] < 0 || strides[i] % 8)
            return failf(kInvalidArgument, "flash_attn_fwd_strided: stride %d (%lld) must be a non-negative multiple of 8 elements", i,
                         (long long)strides[i]);
        st[i] = static_cast<long>(strides[i]);
    }
    if (st[11] < d || (heads > 1 && st[10] == 0) || (batch > 1 && st[9] == 0))
        return fail(kInvalidArgument, "flash_attn_fwd_strided: output rows, heads and batches must not overlap");
    const int64_t row_counts[4] = {sq, sk, sk, sq};
    for (int t = 0; t < 4; t++)
        if (st[3 * t + 2] > (1L << 30) || !flash_fwd_rows_addressable(row_counts[t], st[3 * t + 2] * 2, d))
            return failf(kInvalidArgument, "flash_attn_fwd_strided: operand %d: the rows of one (batch, head) must end below 4 GiB "
                                           "(row offsets are 32-bit)", t);
    std::shared_ptr<Device> dv;
    MRK_TRY(get_device(device_id, &dv));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    const size_t ws = flash_fwd_workspace_bytes(batch * heads, sq, sk, d, causal ? 1 : 0);
    RawBuffer scratch;
    BufferOptions so;
    if (ws) MRK_TRY(dv->allocator->alloc(ws, so, &scratch));
    const int rc = launch_flash_fwd_bf16_strided(dv->allocator->stream(), q, k, v, o, batch, heads, sq, sk, d, scale, causal ? 1 : 0, st,
                                                 ws ? scratch.ptr : nullptr, ws);
    if (ws) dv->allocator->free(scratch, so);
    MRK_HIP(rc, "flash_attn_fwd_strided launch");
    return kOk;
}

int mrk_hip_flash_attn_fwd_bf16_ex(int device_id, const void* q, const void* k, const void* v, void* o, int64_t batch, int64_t heads,
                                   int64_t sq, int64_t sk, int64_t d, float scale, int causal, const int64_t* strides, const void* mask,
                                   int mask_kind, const int64_t* mask_strides, float softcap) {
    if (batch < 0 || heads < 0 || sq < 0 || sk < 0) return fail(kInvalidArgument, "flash_attn_fwd_ex: negative shape");
    if (mask_kind < 0 || mask_kind > 2) return fail(kInvalidArgument, "flash_attn_fwd_ex: mask_kind must be 0 (none), 1 (Bool bytes) or 2 (additive bf16)");
    if (!(softcap >= 0.0f)) return fail(kInvalidArgument, "flash_attn_fwd_ex: softcap must be 0 (none) or positive");
    if (batch == 0 || heads == 0 || sq == 0) return kOk;
    if (d != 256 && d != 128 && d != 64) return failf(kInvalidArgument, "flash_attn_fwd_ex: head_dim %lld is not supported (256, 128 and 64 only)", (long long)d);
    if (sk == 0) return fail(kInvalidArgument, "flash_attn_fwd_ex: empty key sequence (softmax over no keys is undefined)");
    if (!(scale > 0.0f)) return fail(kInvalidArgument, "flash_attn_fwd_ex: scale must be positive");
    MRK_NONNULL(q);
    MRK_NONNULL(k);
    MRK_NONNULL(v);
    MRK_NONNULL(o);
    long st[12];
    const int64_t row_counts[4] = {sq, sk, sk, sq};
    for (int t = 0; t < 4; t++) {  // no strides: dense [batch, heads, rows, d]
        st[3 * t] = strides ? strides[3 * t] : heads * row_counts[t] * d;
        st[3 * t + 1] = strides ? strides[3 * t + 1] : row_counts[t] * d;
        st[3 * t + 2] = strides ? strides[3 * t + 2] : d;
    }
    for (int i = 0; i < 12; i++)
        if (st[i] < 0 || st[i] % 8)
            return failf(kInvalidArgument, "flash_attn_fwd_ex: stride %d (%ld) must be a non-negative multiple of 8 elements", i, st[i]);
    if (st[11] < d || (heads > 1 && st[10] == 0) || (batch > 1 && st[9] == 0))
        return fail(kInvalidArgument, "flash_attn_fwd_ex: output rows, heads and batches must not overlap");
    for (int t = 0; t < 4; t++)
        if (st[3 * t + 2] > (1L << 30) || !flash_fwd_rows_addressable(row_counts[t], st[3 * t + 2] * 2, d))
            return failf(kInvalidArgument, "flash_attn_fwd_ex: operand %d: the rows of one (batch, head) must end below 4 GiB "
                                           "(row offsets are 32-bit)", t);
    long mst[3] = {0, 0, 0};
    if (mask_kind != 0) {
        MRK_NONNULL(mask);
        MRK_NONNULL(mask_strides);
        if (sk % 4) return failf(kInvalidArgument, "flash_attn_fwd_ex: with a mask the key count (%lld) must be a multiple of 4", (long long)sk);
        if (reinterpret_cast<uintptr_t>(mask) % (mask_kind == 2 ? 8 : 4)) return fail(kInvalidArgument, "flash_attn_fwd_ex: the mask must start on a multiple of 4 elements");
        for (int i = 0; i < 3; i++) {
            if (mask_strides[i] < 0 || mask_strides[i] % 4)
                return failf(kInvalidArgument, "flash_attn_fwd_ex: mask stride %d (%lld) must be a non-negative multiple of 4 elements", i, (long long)mask_strides[i]);
            mst[i] = static_cast<long>(mask_strides[i]);
        }
    }
    std::shared_ptr<Device> dv;
    MRK_TRY(get_device(device_id, &dv));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    // (a handful of queries without the causal rule take the kernel that splits the keys: scratch as in the plain call)
    const size_t ws = flash_fwd_workspace_bytes(batch * heads, sq, sk, d, causal ? 1 : 0);
    RawBuffer scratch;
    BufferOptions so;
    if (ws) MRK_TRY(dv->allocator->alloc(ws, so, &scratch));
    const int rc = launch_flash_fwd_bf16_ext(dv->allocator->stream(), q, k, v, o, batch, heads, sq, sk, d, scale, causal ? 1 : 0, st, mask, mask_kind, mst,
                                             softcap, ws ? scratch.ptr : nullptr, ws);
    if (ws) dv->allocator->free(scratch, so);
    MRK_HIP(rc, "flash_attn_fwd_ex launch");
    return kOk;
}

int mrk_hip_fill(int device_id, void* out, size_t n, int dtype, int mode, uint64_t seed, uint64_t tensor_id, float a,
                 float b) {
    if (n == 0) return kOk;
    MRK_NONNULL(out);
    if (dtype < 0 || dtype > 1 || mode < 0 || mode > 1) return fail(kInvalidArgument, "fill: bad dtype or mode");
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    MRK_HIP(launch_fill(d->allocator->stream(), out, n, dtype, mode, seed, tensor_id, a, b), "fill launch");
    return kOk;
}
int mrk_hip_fill_randint(int device_id, void* out, size_t n, uint64_t seed, uint64_t tensor_id, int high) {
    if (n == 0) return kOk;
    MRK_NONNULL(out);
    if (high <= 0) return fail(kInvalidArgument, "fill_randint: high must be positive");
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    MRK_HIP(launch_fill_randint(d->allocator->stream(), out, n, seed, tensor_id, high), "fill_randint launch");
    return kOk;
}

int mrk_hip_copy_kernel(int device_id, const void* src, void* dst, size_t bytes) {
    if (bytes == 0) return kOk;
    MRK_NONNULL(src);
    MRK_NONNULL(dst);
    if (bytes % 16 != 0) return fail(kInvalidArgument, "copy_kernel: size must be a multiple of 16 bytes");
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    MRK_HIP(launch_copy(d->allocator->stream(), src, dst, bytes), "copy_kernel launch");
    return kOk;
}

int mrk_hip_mfma_ceiling(int device_id, void* scratch, int64_t workgroups, int64_t k_steps, int random_operands) {
    MRK_NONNULL(scratch);
    if (workgroups <= 0 || k_steps <= 0) return fail(kInvalidArgument, "mfma_ceiling: workgroups and k_steps must be positive");
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    MRK_HIP(launch_mfma_ceiling(d->allocator->stream(), scratch, workgroups, k_steps, random_operands), "mfma_ceiling launch");
    return kOk;
}

int mrk_hip_event_create(int device_id, mrk_event** out) {
    MRK_NONNULL(out);
    std::shared_ptr<Device> d;
    MRK_TRY(get_device(device_id, &d));
    MRK_HIP(ffi::set_device(device_id), "hipSetDevice");
    ffi::Event e = nullptr;
    MRK_HIP(ffi::event_create(&e), "hipEventCreate");
    *out = new mrk_event{device_id, e, d->allocator->stream()};
    return kOk;
}
int mrk_hip_event_record(mrk_event* e) {
    MRK_NONNULL(e);
    MRK_HIP(ffi::set_device(e->device_id), "hipSetDevice");
    MRK_HIP(ffi::event_record(e->e, e->stream), "hipEventRecord");
    return kOk;
}
int mrk_hip_event_synchronize(mrk_event* e) {
    MRK_NONNULL(e);
    MRK_HIP(ffi::event_synchronize(e->e), "hipEventSynchronize");
    return kOk;
}
int mrk_hip_event_elapsed_ms(mrk_event* start, mrk_event* stop, float* ms) {
    MRK_NONNULL(start);
    MRK_NONNULL(stop);
    MRK_NONNULL(ms);
    MRK_HIP(ffi::event_elapsed_ms(ms, start->e, stop->e), "hipEventElapsedTime");
    return kOk;
}
void mrk_hip_event_destroy(mrk_event* e) {
    if (!e) return;
    ffi::event_destroy(e->e);
    delete e;
}

// ---- lazy tensors
namespace {
int wrap_tensor(Tensor t, mrk_tensor** out) {
    if (!t.valid()) return last_status() != kOk ? last_status() : fail(kInvalidArgument, "invalid tensor operand");
    *out = new mrk_tensor{std::move(t)};
    return kOk;
}
std::vector<int64_t> vec64(const int64_t* p, size_t n) { return p ? std::vector<int64_t>(p, p + n) : std::vector<int64_t>(); }
bool scalar_ok(int dtype) { return dtype >= 0 && dtype <= static_cast<int>(Scalar::Float64); }
}  // namespace
#define MRK_DTYPE(d)                                                             \
    do {                                                                         \
        if (!scalar_ok(d)) return fail(kInvalidArgument, "unknown dtype tag");   \
    } while (0)

int mrk_hip_tensor_from_bytes(int device_id, const void* data, size_t nbytes, const int64_t* shape, size_t ndim,
                              int dtype, mrk_tensor** out) {
    MRK_NONNULL(out);
    MRK_DTYPE(dtype);
    if (nbytes) MRK_NONNULL(data);
    clear_error();
    return wrap_tensor(Tensor::from_raw_bytes(device_id, data, nbytes, vec64(shape, ndim), static_cast<Scalar>(dtype)), out);
}
int mrk_hip_tensor_from_host_bytes(const void* data, size_t nbytes, const int64_t* shape, size_t ndim, int dtype, mrk_tensor** out) {
    MRK_NONNULL(out);
    MRK_DTYPE(dtype);
    if (nbytes) MRK_NONNULL(data);
    clear_error();
    return wrap_tensor(Tensor::from_host_bytes(data, nbytes, vec64(shape, ndim), static_cast<Scalar>(dtype)), out);
}
// "CPU" (any case) -> kCpuDevice, else the HIP spellings of parse_device_spec
static int parse_tensor_device(const char* spec, int* device_id) {
    std::string s(spec);
    for (char& c : s) c = static_cast<char>(std::toupper(static_cast<unsigned char>(c)));
    if (s == "CPU" || s == "CPU:0") {
        *device_id = kCpuDevice;
        return kOk;
    }
    return parse_device_spec(spec, device_id);
}
int mrk_hip_tensor_to(const mrk_tensor* t, const char* device, mrk_tensor** out) {
    MRK_NONNULL(t);
    MRK_NONNULL(device);
    MRK_NONNULL(out);
    clear_error();
    int id = 0;
    MRK_TRY(parse_tensor_device(device, &id));
    return wrap_tensor(t->t.to(id), out);
}
int mrk_hip_tensor_device(const mrk_tensor* t, char* out, size_t cap) {
    MRK_NONNULL(t);
    MRK_NONNULL(out);
    const int id = t->t.device();
    const std::string name = id == kCpuDevice ? std::string("CPU") : "HIP:" + std::to_string(id);
    if (cap < name.size() + 1) return fail(kInvalidArgument, "tensor_device: output too small");
    std::memcpy(out, name.c_str(), name.size() + 1);
    return kOk;
}
int mrk_hip_tensor_from_buffer(const mrk_buffer* b, const int64_t* shape, size_t ndim, int dtype, mrk_tensor** out) {
    MRK_NONNULL(b);
    MRK_NONNULL(out);
    MRK_DTYPE(dtype);
    clear_error();
    return wrap_tensor(Tensor::from_buffer(std::make_shared<Buffer>(*b->b), vec64(shape, ndim), static_cast<Scalar>(dtype)), out);
}
int mrk_hip_tensor_const(int device_id, double value, int dtype, mrk_tensor** out) {
    MRK_NONNULL(out);
    MRK_DTYPE(dtype);
    clear_error();
    return wrap_tensor(Tensor::const_(value, static_cast<Scalar>(dtype), device_id), out);
}
int mrk_hip_tensor_full(int device_id, const int64_t* shape, size_t ndim, double value, int dtype, mrk_tensor** out) {
    MRK_NONNULL(out);
    MRK_DTYPE(dtype);
    clear_error();
    return wrap_tensor(Tensor::full(vec64(shape, ndim), value, static_cast<Scalar>(dtype), device_id), out);
}
void mrk_hip_tensor_release(mrk_tensor* t) { delete t; }
size_t mrk_hip_tensor_ndim(const mrk_tensor* t) { return t ? static_cast<size_t>(t->t.ndim()) : 0; }
int mrk_hip_tensor_shape(const mrk_tensor* t, int64_t* shape_out, size_t capacity) {
    MRK_NONNULL(t);
    if (capacity < t->t.shape().size()) return fail(kInvalidArgument, "shape buffer too small");
    for (size_t i = 0; i < t->t.shape().size(); i++) shape_out[i] = t->t.shape()[i];
    return kOk;
}
int mrk_hip_tensor_dtype(const mrk_tensor* t) { return t ? static_cast<int>(t->t.dtype()) : -1; }

#define MRK_T1(t)       \
    MRK_NONNULL(t);     \
    MRK_NONNULL(out);   \
    clear_error()

int mrk_hip_tensor_reshape(const mrk_tensor* t, const int64_t* shape, size_t ndim, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.try_reshape(vec64(shape, ndim)), out);
}
int mrk_hip_tensor_permute(const mrk_tensor* t, const int64_t* perm, size_t ndim, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.try_permute(vec64(perm, ndim)), out);
}
int mrk_hip_tensor_transpose(const mrk_tensor* t, int64_t a, int64_t b, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.try_transpose(a, b), out);
}
int mrk_hip_tensor_expand(const mrk_tensor* t, const int64_t* shape, size_t ndim, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.try_expand(vec64(shape, ndim)), out);
}
int mrk_hip_tensor_shrink(const mrk_tensor* t, const int64_t* begin, const int64_t* end, size_t ndim, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.try_shrink(vec64(begin, ndim), vec64(end, ndim)), out);
}
int mrk_hip_tensor_contiguous(const mrk_tensor* t, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.contiguous(), out);
}
int mrk_hip_tensor_cat(const mrk_tensor* const* parts, size_t nparts, int64_t axis, mrk_tensor** out) {
    MRK_NONNULL(parts);
    MRK_NONNULL(out);
    clear_error();
    std::vector<Tensor> ts;
    for (size_t i = 0; i < nparts; i++) {
        MRK_NONNULL(parts[i]);
        ts.push_back(parts[i]->t);
    }
    return wrap_tensor(Tensor::cat(ts, axis), out);
}
int mrk_hip_tensor_cast(const mrk_tensor* t, int dtype, mrk_tensor** out) {
    MRK_T1(t);
    MRK_DTYPE(dtype);
    return wrap_tensor(t->t.cast(static_cast<Scalar>(dtype)), out);
}
int mrk_hip_tensor_unary(const mrk_tensor* t, int unary_op, mrk_tensor** out) {
    MRK_T1(t);
    if (unary_op < 0 || unary_op > static_cast<int>(UnaryOp::Not)) return fail(kInvalidArgument, "unknown unary op tag");
    return wrap_tensor(t->t.unary(static_cast<UnaryOp>(unary_op)), out);
}
int mrk_hip_tensor_binary(const mrk_tensor* a, int binary_op, const mrk_tensor* b, mrk_tensor** out) {
    MRK_T1(a);
    MRK_NONNULL(b);
    if (binary_op < 0 || binary_op > static_cast<int>(BinaryOp::Ne)) return fail(kInvalidArgument, "unknown binary op tag");
    return wrap_tensor(a->t.binary(static_cast<BinaryOp>(binary_op), b->t), out);
}
int mrk_hip_tensor_where(const mrk_tensor* cond, const mrk_tensor* a, const mrk_tensor* b, mrk_tensor** out) {
    MRK_T1(cond);
    MRK_NONNULL(a);
    MRK_NONNULL(b);
    return wrap_tensor(a->t.where_(cond->t, b->t), out);
}
int mrk_hip_tensor_sigmoid(const mrk_tensor* t, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.sigmoid(), out);
}
int mrk_hip_tensor_silu(const mrk_tensor* t, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.silu(), out);
}
int mrk_hip_tensor_reduce(const mrk_tensor* t, int reduce_op, const int64_t* axes, size_t naxes, int keepdim, int promote,
                          mrk_tensor** out) {
    MRK_T1(t);
    if (reduce_op < 0 || reduce_op > static_cast<int>(ReduceOp::Min)) return fail(kInvalidArgument, "unknown reduce op tag");
    return wrap_tensor(t->t.reduce(static_cast<ReduceOp>(reduce_op), vec64(axes, naxes), keepdim != 0, promote != 0), out);
}
int mrk_hip_tensor_mean(const mrk_tensor* t, const int64_t* axes, size_t naxes, int keepdim, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.mean(vec64(axes, naxes), keepdim != 0), out);
}
int mrk_hip_tensor_matmul(const mrk_tensor* a, const mrk_tensor* b, mrk_tensor** out) {
    MRK_T1(a);
    MRK_NONNULL(b);
    return wrap_tensor(a->t.matmul(b->t), out);
}
int mrk_hip_tensor_matmul_with(const mrk_tensor* a, const mrk_tensor* b, int acc_dtype, mrk_tensor** out) {
    MRK_T1(a);
    MRK_NONNULL(b);
    if (acc_dtype < -1 || acc_dtype >= static_cast<int>(Scalar::Void)) return fail(kInvalidArgument, "matmul_with: unknown dtype tag");
    return wrap_tensor(a->t.matmul(b->t, acc_dtype < 0 ? Scalar::Void : static_cast<Scalar>(acc_dtype)), out);
}
int mrk_hip_tensor_gemm(const mrk_tensor* a, const mrk_tensor* b, float alpha, float beta, int trans_a, int trans_b,
                        const mrk_tensor* c, mrk_tensor** out) {
    MRK_T1(a);
    MRK_NONNULL(b);
    return wrap_tensor(a->t.gemm(b->t, alpha, beta, trans_a != 0, trans_b != 0, c ? &c->t : nullptr), out);
}
int mrk_hip_tensor_linear(const mrk_tensor* x, const mrk_tensor* weight, const mrk_tensor* bias, int acc_dtype, mrk_tensor** out) {
    MRK_T1(x);
    MRK_NONNULL(weight);
    if (acc_dtype < -1 || acc_dtype >= static_cast<int>(Scalar::Void)) return fail(kInvalidArgument, "linear: unknown dtype tag");
    return wrap_tensor(x->t.linear(weight->t, bias ? &bias->t : nullptr, acc_dtype < 0 ? Scalar::Void : static_cast<Scalar>(acc_dtype)), out);
}
int mrk_hip_tensor_log_softmax(const mrk_tensor* t, int64_t axis, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.log_softmax(axis), out);
}
int mrk_hip_tensor_logsumexp(const mrk_tensor* t, int64_t axis, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.logsumexp(axis), out);
}
int mrk_hip_tensor_softmax(const mrk_tensor* t, int64_t axis, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.softmax(axis), out);
}
int mrk_hip_tensor_rms_norm(const mrk_tensor* t, int64_t axis, double eps, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.rms_norm(axis, eps), out);
}
int mrk_hip_tensor_embedding(const mrk_tensor* weight, const mrk_tensor* indices, mrk_tensor** out) {
    MRK_T1(weight);
    MRK_NONNULL(indices);
    return wrap_tensor(weight->t.embedding(indices->t), out);
}
int mrk_hip_tensor_rotary(const mrk_tensor* x, const mrk_tensor* cos, const mrk_tensor* sin, int interleaved,
                          mrk_tensor** out) {
    MRK_T1(x);
    MRK_NONNULL(cos);
    MRK_NONNULL(sin);
    return wrap_tensor(x->t.apply_rotary_emb(cos->t, sin->t, interleaved != 0), out);
}
int mrk_hip_tensor_sdpa(const mrk_tensor* q, const mrk_tensor* k, const mrk_tensor* v, double scale, int is_causal,
                        mrk_tensor** out) {
    MRK_T1(q);
    MRK_NONNULL(k);
    MRK_NONNULL(v);
    return wrap_tensor(q->t.scaled_dot_product_attention(k->t, v->t, scale, is_causal != 0), out);
}
int mrk_hip_tensor_sdpa_ex(const mrk_tensor* q, const mrk_tensor* k, const mrk_tensor* v, const mrk_tensor* attn_mask,
                           double scale, int is_causal, double softcap, mrk_tensor** out) {
    MRK_T1(q);
    MRK_NONNULL(k);
    MRK_NONNULL(v);
    return wrap_tensor(q->t.scaled_dot_product_attention(k->t, v->t, scale, is_causal != 0, attn_mask ? &attn_mask->t : nullptr, softcap),
                       out);
}
int mrk_hip_tensor_tanh(const mrk_tensor* t, mrk_tensor** out) {
    MRK_T1(t);
    return wrap_tensor(t->t.tanh(), out);
}
int mrk_hip_tensor_realize(const mrk_tensor* t) {
    MRK_NONNULL(t);
    return t->t.realize();
}
int mrk_hip_tensor_prepare(const mrk_tensor* t, mrk_plan** out) {
    MRK_NONNULL(t);
    MRK_NONNULL(out);
    std::unique_ptr<ExecutionPlan> p;
    MRK_TRY(t->t.prepare(&p));
    *out = new mrk_plan{std::move(p)};
    return kOk;
}
int mrk_hip_tensor_to_bytes(const mrk_tensor* t, void* dst, size_t nbytes) {
    MRK_NONNULL(t);
    if (nbytes) MRK_NONNULL(dst);
    return t->t.to_bytes(dst, nbytes);
}
int mrk_hip_tensor_buffer(const mrk_tensor* t, mrk_buffer** out) {
    MRK_NONNULL(t);
    MRK_NONNULL(out);
    auto b = t->t.buffer();
    if (!b) return fail(kInvalidArgument, "tensor is not realized");
    *out = new mrk_buffer{std::unique_ptr<Buffer>(new Buffer(*b))};
    return kOk;
}
void mrk_hip_tensor_set_fusion(int enabled) { set_fusion_enabled(enabled != 0); }
size_t mrk_hip_tensor_last_kernel_count(void) { return last_realize_stats().kernel_names.size(); }
const char* mrk_hip_tensor_last_kernel_name(size_t i) {
    const auto& n = last_realize_stats().kernel_names;
    return i < n.size() ? n[i].c_str() : nullptr;
}
const char* mrk_hip_tensor_last_kernel_source(size_t i) {
    const auto& n = last_realize_stats().kernel_sources;
    return i < n.size() ? n[i].c_str() : nullptr;
}
size_t mrk_hip_tensor_last_cached_count(void) { return last_realize_stats().cached_kernels; }
double mrk_hip_tensor_last_elapsed_ms(void) { return last_realize_stats().elapsed_ms; }
size_t mrk_hip_tensor_last_buffers_reused(void) { return last_realize_stats().buffers_reused; }
size_t mrk_hip_tensor_last_memory_saved(void) { return last_realize_stats().memory_saved; }
size_t mrk_hip_tensor_last_intermediate_bytes(void) { return last_realize_stats().intermediate_bytes; }
size_t mrk_hip_tensor_last_beam_candidates(void) { return last_realize_stats().beam_candidates; }
size_t mrk_hip_tensor_last_beam_cache_hits(void) { return last_realize_stats().beam_cache_hits; }

}  // extern "C"
