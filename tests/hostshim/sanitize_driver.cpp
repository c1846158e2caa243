// Native driver of the host runtime for sanitizer builds (AddressSanitizer + UBSan, or
// ThreadSanitizer): four threads create buffers and tensors, realize and prepare graphs (among
// them attention over strided views, masked attention, rotary embeddings, vector products),
// replay plans eagerly, profiled and as graphs, build tensor-core kernels over the whole tile
// search space, and use queues and signals, all through the C ABI and against the host-memory
// stand-ins of this directory.  TEST INFRASTRUCTURE ONLY.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#include "morok_hip.h"
#define CK(x) do { int rc_ = (x); if (rc_ != 0) { printf("FAIL line %d rc %d: %s\n", __LINE__, rc_, mrk_hip_last_error()); return 1; } } while (0)
#include <thread>
static int work(int id);
// Four threads realize four different roots built over ONE shared lazy subgraph (a reduce over an
// elementwise chain, so the shared nodes are kernel boundaries that receive provisional buffers
// while a root is scheduled), several times over, and read the results back.
static int shared_subgraph() {
    int64_t shp[2] = {48, 80};
    std::vector<float> x(48 * 80, 0.5f);
    mrk_tensor *t = nullptr, *u = nullptr, *mid = nullptr;
    CK(mrk_hip_tensor_from_bytes(0, x.data(), x.size() * 4, shp, 2, 11 /*f32*/, &t));
    CK(mrk_hip_tensor_binary(t, 0 /*add*/, t, &u));
    int64_t axes[1] = {1};
    CK(mrk_hip_tensor_reduce(u, 0 /*add*/, axes, 1, 1, 1, &mid));  // shared, lazy
    int rcs[4] = {0, 0, 0, 0};
    std::vector<std::thread> th;
    for (int i = 0; i < 4; i++)
        th.emplace_back([i, u, mid, &rcs] {
            rcs[i] = [&]() -> int {
                for (int r = 0; r < 6; r++) {
                    mrk_tensor *a = nullptr, *root = nullptr;
                    CK(mrk_hip_tensor_binary(u, i % 2 ? 2 /*mul*/ : 1 /*sub*/, mid, &a));
                    int64_t ax[1] = {0};
                    CK(mrk_hip_tensor_reduce(a, i < 2 ? 0 : 2 /*add | max*/, ax, 1, 0, 1, &root));
                    if (r % 2) {
                        mrk_plan* plan = nullptr;
                        CK(mrk_hip_tensor_prepare(root, &plan));
                        CK(mrk_hip_plan_execute(plan));
                        mrk_hip_plan_release(plan);
                    } else {
                        CK(mrk_hip_tensor_realize(root));
                    }
                    std::vector<float> out(80);
                    CK(mrk_hip_tensor_to_bytes(root, out.data(), out.size() * 4));
                    mrk_hip_tensor_release(a);
                    mrk_hip_tensor_release(root);
                }
                return 0;
            }();
        });
    for (auto& thr : th) thr.join();
    for (int rc : rcs)
        if (rc) return 1;
    CK(mrk_hip_tensor_realize(mid));  // the shared node itself is still realizable afterwards
    for (mrk_tensor* p : {t, u, mid}) mrk_hip_tensor_release(p);
    return 0;
}
// Four threads realize graphs that share nothing and whose kernels nobody has compiled yet (every
// thread and round has a shape of its own): the graph lock is released while a thread compiles, so
// the compiles of unrelated graphs overlap and the schedules interleave around them.
static int unrelated_graphs_compile_concurrently() {
    int rcs[4] = {0, 0, 0, 0};
    std::vector<std::thread> th;
    for (int i = 0; i < 4; i++)
        th.emplace_back([i, &rcs] {
            rcs[i] = [&]() -> int {
                for (int r = 0; r < 3; r++) {
                    int64_t shp[2] = {16 + 8 * i + r, 24 + 4 * r + i};
                    std::vector<float> x(shp[0] * shp[1], 0.25f);
                    mrk_tensor *t = nullptr, *u = nullptr, *root = nullptr;
                    CK(mrk_hip_tensor_from_bytes(0, x.data(), x.size() * 4, shp, 2, 11 /*f32*/, &t));
                    CK(mrk_hip_tensor_binary(t, 2 /*mul*/, t, &u));
                    int64_t ax[1] = {1};
                    CK(mrk_hip_tensor_reduce(u, 0 /*add*/, ax, 1, 0, 1, &root));
                    if (r == 1) {
                        mrk_plan* plan = nullptr;
                        CK(mrk_hip_tensor_prepare(root, &plan));
                        CK(mrk_hip_plan_execute(plan));
                        mrk_hip_plan_release(plan);
                    }
                    std::vector<float> out(shp[0]);
                    CK(mrk_hip_tensor_to_bytes(root, out.data(), out.size() * 4));
                    CK(mrk_hip_tensor_realize(root));   // already realized: no second schedule
                    for (mrk_tensor* p : {t, u, root}) mrk_hip_tensor_release(p);
                }
                return 0;
            }();
        });
    for (auto& thr : th) thr.join();
    for (int rc : rcs)
        if (rc) return 1;
    return 0;
}
int main() {
    if (mrk_hip_device_create(0)) return 1;
    std::vector<std::thread> th; int rcs[4] = {0,0,0,0};
    for (int i = 0; i < 4; i++) th.emplace_back([i, &rcs] { for (int r = 0; r < 5; r++) rcs[i] |= work(i); });
    for (auto& t : th) t.join();
    for (int i = 0; i < 4; i++) if (rcs[i]) return 1;
    if (shared_subgraph()) return 1;
    if (unrelated_graphs_compile_concurrently()) return 1;
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
    // the scheduler's view analysis and kernel splitting: attention over slices of a packed bf16
    // product with the result permuted back (strided kernel), masked attention (composed graph),
    // rotary embedding in both layouts (per-part regions, split upcast groups), vector matmul
    {
        const int64_t B = 1, S = 128, H = 2, D = 128, hid = H * D;
        int64_t ps[2] = {B * S, 3 * hid};
        std::vector<uint16_t> packed(static_cast<size_t>(ps[0] * ps[1]), 0x3f80);
        mrk_tensor* pk = nullptr;
        CK(mrk_hip_tensor_from_bytes(0, packed.data(), packed.size() * 2, ps, 2, 10 /*bf16*/, &pk));
        mrk_tensor* qkv[3] = {nullptr, nullptr, nullptr};
        std::vector<mrk_tensor*> tmp;
        for (int i = 0; i < 3; i++) {
            int64_t b0[2] = {0, i * hid}, e0[2] = {B * S, (i + 1) * hid}, r4[4] = {B, S, H, D}, perm[4] = {0, 2, 1, 3};
            mrk_tensor *a = nullptr, *b4 = nullptr;
            CK(mrk_hip_tensor_shrink(pk, b0, e0, 2, &a));
            CK(mrk_hip_tensor_reshape(a, r4, 4, &b4));
            CK(mrk_hip_tensor_permute(b4, perm, 4, &qkv[i]));
            tmp.push_back(a);
            tmp.push_back(b4);
        }
        mrk_tensor *att = nullptr, *back = nullptr, *flat = nullptr;
        CK(mrk_hip_tensor_sdpa(qkv[0], qkv[1], qkv[2], 0.0, 1, &att));
        int64_t perm[4] = {0, 2, 1, 3}, r2[2] = {B * S, hid};
        CK(mrk_hip_tensor_permute(att, perm, 4, &back));
        CK(mrk_hip_tensor_reshape(back, r2, 2, &flat));
        CK(mrk_hip_tensor_realize(flat));
        if (mrk_hip_tensor_last_kernel_count() != 1 || !strstr(mrk_hip_tensor_last_kernel_name(0), "strided")) {
            printf("attention over views did not take the strided kernel\n");
            return 1;
        }
        // x + a @ w in bf16: the product kernel with the residual epilogue, through contiguous()
        {
            int64_t as[2] = {B * S, hid}, wsh[2] = {hid, hid};
            std::vector<uint16_t> av(static_cast<size_t>(as[0] * as[1]), 0x3f80), wv(static_cast<size_t>(hid * hid), 0x3c00);
            mrk_tensor *ta = nullptr, *tw = nullptr, *mm = nullptr, *sum = nullptr, *cont = nullptr;
            CK(mrk_hip_tensor_from_bytes(0, av.data(), av.size() * 2, as, 2, 10, &ta));
            CK(mrk_hip_tensor_from_bytes(0, wv.data(), wv.size() * 2, wsh, 2, 10, &tw));
            CK(mrk_hip_tensor_matmul(ta, tw, &mm));
            CK(mrk_hip_tensor_binary(ta, 0 /*add*/, mm, &sum));
            CK(mrk_hip_tensor_contiguous(sum, &cont));
            CK(mrk_hip_tensor_realize(cont));
            if (mrk_hip_tensor_last_kernel_count() != 1 || !strstr(mrk_hip_tensor_last_kernel_name(0), "residual")) {
                printf("x + a @ w did not take the residual epilogue\n");
                return 1;
            }
            for (mrk_tensor* p : {ta, tw, mm, sum, cont}) mrk_hip_tensor_release(p);
        }
        int64_t ms[2] = {S, S};
        std::vector<float> maskv(static_cast<size_t>(S * S), 0.0f);
        mrk_tensor *mask = nullptr, *att2 = nullptr;
        CK(mrk_hip_tensor_from_bytes(0, maskv.data(), maskv.size() * 4, ms, 2, 11, &mask));
        CK(mrk_hip_tensor_sdpa_ex(qkv[0], qkv[1], qkv[2], mask, 0.0, 0, 2.0, &att2));
        CK(mrk_hip_tensor_realize(att2));
        int64_t xs[4] = {2, 16, 4, 128}, cs[4] = {1, 16, 1, 64};
        std::vector<float> xv(2 * 16 * 4 * 128, 0.5f), cv(16 * 64, 1.0f);
        mrk_tensor *xr = nullptr, *c = nullptr, *r0 = nullptr, *r1 = nullptr;
        CK(mrk_hip_tensor_from_bytes(0, xv.data(), xv.size() * 4, xs, 4, 11, &xr));
        CK(mrk_hip_tensor_from_bytes(0, cv.data(), cv.size() * 4, cs, 4, 11, &c));
        CK(mrk_hip_tensor_rotary(xr, c, c, 0, &r0));
        CK(mrk_hip_tensor_rotary(xr, c, c, 1, &r1));
        CK(mrk_hip_tensor_realize(r0));
        CK(mrk_hip_tensor_realize(r1));
        int64_t vs[1] = {64};
        mrk_tensor *vec = nullptr, *dot = nullptr, *mv = nullptr, *lin = nullptr;
        CK(mrk_hip_tensor_from_bytes(0, x.data(), 64 * 4, vs, 1, 11, &vec));
        CK(mrk_hip_tensor_matmul(vec, vec, &dot));
        CK(mrk_hip_tensor_matmul(t, vec, &mv));
        CK(mrk_hip_tensor_linear(t, t, vec, -1, &lin));
        CK(mrk_hip_tensor_realize(dot));
        CK(mrk_hip_tensor_realize(mv));
        CK(mrk_hip_tensor_realize(lin));
        for (mrk_tensor* p : {pk, qkv[0], qkv[1], qkv[2], att, back, flat, mask, att2, xr, c, r0, r1, vec, dot, mv, lin}) mrk_hip_tensor_release(p);
        for (mrk_tensor* p : tmp) mrk_hip_tensor_release(p);
        // tensor-core kernel builders: every tile choice of the search space on a padded shape
        for (int wm : {1, 2, 4})
            for (int wn : {1, 2, 4})
                for (int um : {1, 4, 8}) {
                    int opts[6] = {wm, wn, um, 2, id % 3, 0};
                    uint8_t* kern = nullptr;
                    size_t len = 0;
                    if (mrk_hip_sched_build_wmma_matmul_lds_opts(3, 200 + id, 136, 72, 10, opts, &kern, &len) == 0) mrk_hip_sched_free(kern);
                }
        // and the variant with direct global -> local copies on shapes its tiles divide
        for (int um : {2, 4, 8}) {
            int opts[6] = {2, 2 << (id % 2), um, 4, 0, 2};
            uint8_t* kern = nullptr;
            size_t len = 0;
            if (mrk_hip_sched_build_wmma_matmul_lds_opts(3, 1024, 1024, 64 * (1 + id), 10, opts, &kern, &len) == 0) mrk_hip_sched_free(kern);
        }
    }
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
