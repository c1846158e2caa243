// Native driver of the host runtime for sanitizer builds (AddressSanitizer + UBSan, or
// ThreadSanitizer): four threads create buffers and tensors, realize and prepare graphs, replay
// plans eagerly, profiled and as graphs, and use queues and signals, all through the C ABI and
// against the host-memory stand-ins of this directory.  TEST INFRASTRUCTURE ONLY.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#include "morok_hip.h"
#define CK(x) do { int rc_ = (x); if (rc_ != 0) { printf("FAIL line %d rc %d: %s\n", __LINE__, rc_, mrk_hip_last_error()); return 1; } } while (0)
#include <thread>
static int work(int id);
int main() {
    if (mrk_hip_device_create(0)) return 1;
    std::vector<std::thread> th; int rcs[4] = {0,0,0,0};
    for (int i = 0; i < 4; i++) th.emplace_back([i, &rcs] { for (int r = 0; r < 5; r++) rcs[i] |= work(i); });
    for (auto& t : th) t.join();
    for (int i = 0; i < 4; i++) if (rcs[i]) return 1;
    printf("threads ok\n");
    return 0;
}
static int work(int id) {
    CK(mrk_hip_device_create(0));
    // buffers and views
    mrk_buffer *b = nullptr, *v = nullptr;
    CK(mrk_hip_buffer_new(0, 4096, 1, 0, &b));
    CK(mrk_hip_buffer_ensure_allocated(b));
    CK(mrk_hip_buffer_view(b, 1024, 1024, &v));
    std::vector<float> h(256, 1.5f), o(256);
    CK(mrk_hip_buffer_copyin(v, h.data(), 1024));
    CK(mrk_hip_buffer_copyout(v, o.data(), 1024));
    mrk_hip_buffer_release(v);
    mrk_hip_buffer_release(b);
    // tensors: elementwise + reduce + matmul + softmax + cat, realize and prepare, graph replay
    int64_t shp[2] = {64, 64};
    std::vector<float> x(64 * 64, 0.25f);
    mrk_tensor *t = nullptr, *u = nullptr, *w = nullptr, *s = nullptr, *m = nullptr;
    CK(mrk_hip_tensor_from_bytes(0, x.data(), x.size() * 4, shp, 2, 11 /*f32*/, &t));
    CK(mrk_hip_tensor_binary(t, 0 /*add*/, t, &u));
    int64_t axes[1] = {1};
    CK(mrk_hip_tensor_reduce(u, 0 /*add*/, axes, 1, 0, 1, &w));
    CK(mrk_hip_tensor_softmax(u, -1, &s));
    CK(mrk_hip_tensor_matmul(t, u, &m));
    CK(mrk_hip_tensor_realize(w));
    CK(mrk_hip_tensor_realize(s));
    mrk_plan* plan = nullptr;
    CK(mrk_hip_tensor_prepare(m, &plan));
    CK(mrk_hip_plan_execute(plan));
    CK(mrk_hip_plan_execute_graph(plan));
    CK(mrk_hip_plan_execute_graph(plan));
    std::vector<double> prof(16); size_t n = 0;
    CK(mrk_hip_plan_execute_profiled(plan, prof.data(), 16, &n));
    mrk_hip_plan_release(plan);
    for (mrk_tensor* p : {t, u, w, s, m}) mrk_hip_tensor_release(p);
    // queues and signals
    mrk_queue* q = nullptr; mrk_signal* sig = nullptr;
    CK(mrk_hip_queue_create(0, 0, &q));
    CK(mrk_hip_signal_create(0, &sig));
    CK(mrk_hip_queue_signal(q, sig, 1));
    CK(mrk_hip_queue_submit(q, 1000));
    CK(mrk_hip_queue_synchronize(q));
    mrk_hip_queue_destroy(q);
    mrk_hip_signal_destroy(sig);
    // error paths
    mrk_tensor* bad = nullptr;
    int64_t shp2[2] = {3, 5};
    std::vector<float> y(15, 1.0f);
    mrk_tensor* t2 = nullptr;
    CK(mrk_hip_tensor_from_bytes(0, y.data(), 60, shp2, 2, 11, &t2));
    if (mrk_hip_tensor_matmul(t2, t2, &bad) == 0) { printf("expected a shape error\n"); return 1; }
    mrk_hip_tensor_release(t2);
    mrk_hip_kernel_cache_clear();
    CK(mrk_hip_lru_clear(0));
    printf("driver ok\n");
    return 0;
}
