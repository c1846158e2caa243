// Host-memory stand-in for morok_amd/csrc/hip_ffi.cpp.  TEST INFRASTRUCTURE ONLY: linked with
// the product's host sources into libmorok_hostshim.so so that allocator, buffer, kernel
// cache, renderer/compiler plumbing, scheduling and error paths can be exercised on a machine
// without a GPU.  "Device" memory is host memory, launches are recorded and compute nothing.
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "hip_ffi.h"

namespace {
std::mutex g_mu;
std::unordered_map<void*, size_t> g_allocs;
size_t g_in_use = 0, g_limit = ~size_t(0), g_alloc_calls = 0, g_free_calls = 0, g_launches = 0, g_syncs = 0;
int g_devices = 1;
unsigned g_last_grid[3], g_last_block[3];
std::string g_last_kernel;
struct FakeModule {
    std::string image;
};
struct FakeFunction {
    std::string name;
};
struct FakeEvent {
    int no = 0;
    std::chrono::steady_clock::time_point t;
    bool recorded = false;
};
constexpr int kOutOfMemory = 2, kInvalidValue = 1, kNotFound = 500, kInvalidDevice = 101, kInvalidImage = 200;
// stream capture: launches made while capturing are recorded, not run; a graph launch runs them
struct FakeGraph {
    size_t launches = 0;
};
std::map<void*, size_t> g_capturing;  // stream -> launches recorded so far
size_t g_graph_launches = 0, g_graphs_alive = 0;
bool g_events_pending = false;  // event_query answers "not ready" while set
// trace of stream operations ("memset:S", "record:E:S", "wait:S:E", "launch:S", "dtod:S", "htod:S", "dtoh:S"; S = stream
// number in creation order, E = event number), kept while enabled
bool g_trace_on = false;
std::string g_trace;
int g_next_stream = 0, g_next_event = 0;
int stream_no(void* s) { return s ? *static_cast<int*>(s) : -1; }
void trace(const std::string& what) {
    if (g_trace_on) g_trace += what + " ";
}
long g_fail_module_load_in = -1;  // >= 0: that many further module loads succeed, the next one fails once
// one launch seen by the stand-in: counted as run, or as recorded while its stream is capturing (g_mu held)
void count_launch(void* stream) {
    auto it = g_capturing.find(stream);
    if (it != g_capturing.end()) it->second++;
    else g_launches++;
}
}  // namespace

extern "C" {
void mrk_shim_reset() {
    std::lock_guard<std::mutex> l(g_mu);
    g_limit = ~size_t(0);
    g_alloc_calls = g_free_calls = g_launches = g_syncs = 0;
    g_graph_launches = 0;
    g_fail_module_load_in = -1;
    g_events_pending = false;
    g_trace_on = false;
    g_trace.clear();
    g_last_kernel.clear();
}
// failure injection: after `n` more successful module loads the next one reports an invalid image, once
void mrk_shim_fail_module_load_after(long n) { g_fail_module_load_in = n; }
void mrk_shim_set_events_pending(int on) { g_events_pending = on != 0; }
void mrk_shim_trace(int on) {
    std::lock_guard<std::mutex> l(g_mu);
    g_trace_on = on != 0;
    g_trace.clear();
}
// copies the trace (NUL-terminated, truncated to cap) and returns its full length
size_t mrk_shim_trace_get(char* out, size_t cap) {
    std::lock_guard<std::mutex> l(g_mu);
    if (out && cap) {
        size_t n = g_trace.size() < cap - 1 ? g_trace.size() : cap - 1;
        std::memcpy(out, g_trace.data(), n);
        out[n] = 0;
    }
    return g_trace.size();
}
size_t mrk_shim_graph_launches() { return g_graph_launches; }
size_t mrk_shim_graphs_alive() { return g_graphs_alive; }
void mrk_shim_set_memory_limit(size_t bytes) { g_limit = bytes; }
void mrk_shim_set_device_count(int n) { g_devices = n; }
size_t mrk_shim_bytes_in_use() { return g_in_use; }
size_t mrk_shim_alloc_calls() { return g_alloc_calls; }
size_t mrk_shim_free_calls() { return g_free_calls; }
size_t mrk_shim_launches() { return g_launches; }
size_t mrk_shim_syncs() { return g_syncs; }
const char* mrk_shim_last_kernel() { return g_last_kernel.c_str(); }
void mrk_shim_last_dims(unsigned* grid, unsigned* block) {
    std::memcpy(grid, g_last_grid, sizeof g_last_grid);
    std::memcpy(block, g_last_block, sizeof g_last_block);
}
// called by the recording launchers of fake_kernels.cpp
void mrk_shim_note_launch(void* stream, const char* name) {
    std::lock_guard<std::mutex> l(g_mu);
    count_launch(stream);
    trace("launch:" + std::to_string(stream_no(stream)));
    g_last_kernel = name;
}
}

namespace mrk::ffi {

const int kNotReady = 600;

int device_count(int* out) {
    *out = g_devices;
    return g_devices > 0 ? 0 : 100;  // hipErrorNoDevice
}
int set_device(int device_id) { return device_id >= 0 && device_id < g_devices ? 0 : kInvalidDevice; }

int malloc_device(void** out, size_t bytes) {
    std::lock_guard<std::mutex> l(g_mu);
    g_alloc_calls++;
    if (g_in_use + bytes > g_limit) return kOutOfMemory;
    void* p = std::malloc(bytes ? bytes : 1);
    if (!p) return kOutOfMemory;
    std::memset(p, 0xCD, bytes);  // fresh device memory is not zero
    g_allocs[p] = bytes;
    g_in_use += bytes;
    *out = p;
    return 0;
}
int malloc_managed(void** out, size_t bytes) { return malloc_device(out, bytes); }
int free_device(void* ptr) {
    std::lock_guard<std::mutex> l(g_mu);
    auto it = g_allocs.find(ptr);
    if (it == g_allocs.end()) return kInvalidValue;
    g_free_calls++;
    g_in_use -= it->second;
    g_allocs.erase(it);
    std::free(ptr);
    return 0;
}
int mem_info(size_t* free_bytes, size_t* total_bytes) {
    *total_bytes = g_limit == ~size_t(0) ? (size_t(288) << 30) : g_limit;
    *free_bytes = *total_bytes - g_in_use;
    return 0;
}

int memset_async(void* dst, int value, size_t bytes, Stream s) {
    { std::lock_guard<std::mutex> l(g_mu); trace("memset:" + std::to_string(stream_no(s))); }
    std::memset(dst, value, bytes);
    return 0;
}
int memcpy_htod_async(void* dst, const void* src, size_t bytes, Stream s) {
    { std::lock_guard<std::mutex> l(g_mu); trace("htod:" + std::to_string(stream_no(s))); }
    std::memcpy(dst, src, bytes);
    return 0;
}
int memcpy_dtoh_async(void* dst, const void* src, size_t bytes, Stream s) {
    { std::lock_guard<std::mutex> l(g_mu); trace("dtoh:" + std::to_string(stream_no(s))); }
    std::memcpy(dst, src, bytes);
    return 0;
}
int memcpy_dtod_async(void* dst, const void* src, size_t bytes, Stream s) {
    { std::lock_guard<std::mutex> l(g_mu); trace("dtod:" + std::to_string(stream_no(s))); }
    std::memmove(dst, src, bytes);
    return 0;
}

int stream_create(Stream* out) {
    std::lock_guard<std::mutex> l(g_mu);
    *out = new int(g_next_stream++);
    return 0;
}
int stream_destroy(Stream s) {
    delete static_cast<int*>(s);
    return 0;
}
int stream_synchronize(Stream) {
    { std::lock_guard<std::mutex> l(g_mu); g_syncs++; }
    return 0;
}
int stream_wait_event(Stream s, Event e) {
    std::lock_guard<std::mutex> l(g_mu);
    trace("wait:" + std::to_string(stream_no(s)) + ":" + std::to_string(static_cast<FakeEvent*>(e)->no));
    return 0;
}
int device_synchronize() {
    { std::lock_guard<std::mutex> l(g_mu); g_syncs++; }
    return 0;
}

int event_create(Event* out) {
    std::lock_guard<std::mutex> l(g_mu);
    auto* ev = new FakeEvent();
    ev->no = g_next_event++;
    *out = ev;
    return 0;
}
int event_destroy(Event e) {
    delete static_cast<FakeEvent*>(e);
    return 0;
}
int event_record(Event e, Stream s) {
    auto* ev = static_cast<FakeEvent*>(e);
    { std::lock_guard<std::mutex> l(g_mu); trace("record:" + std::to_string(ev->no) + ":" + std::to_string(stream_no(s))); }
    ev->t = std::chrono::steady_clock::now();
    ev->recorded = true;
    return 0;
}
int event_query(Event) { return g_events_pending ? kNotReady : 0; }
int event_synchronize(Event) { return 0; }
int event_elapsed_ms(float* ms, Event start, Event stop) {
    auto *a = static_cast<FakeEvent*>(start), *b = static_cast<FakeEvent*>(stop);
    if (!a->recorded || !b->recorded) return kInvalidValue;
    *ms = std::chrono::duration<float, std::milli>(b->t - a->t).count();
    return 0;
}

int module_load_data(Module* out, const void* image) {
    // a gfx950 code object is an ELF; its length is recovered from the section header table
    const unsigned char* p = static_cast<const unsigned char*>(image);
    if (!p || std::memcmp(p, "\x7f" "ELF", 4) != 0) return kInvalidImage;
    {
        std::lock_guard<std::mutex> l(g_mu);
        if (g_fail_module_load_in == 0) {
            g_fail_module_load_in = -1;
            return kInvalidImage;
        }
        if (g_fail_module_load_in > 0) g_fail_module_load_in--;
    }
    uint64_t shoff;
    uint16_t shentsize, shnum;
    std::memcpy(&shoff, p + 0x28, 8);
    std::memcpy(&shentsize, p + 0x3A, 2);
    std::memcpy(&shnum, p + 0x3C, 2);
    auto* m = new FakeModule();
    m->image.assign(reinterpret_cast<const char*>(p), shoff + size_t(shentsize) * shnum);
    *out = m;
    return 0;
}
int module_unload(Module m) {
    delete static_cast<FakeModule*>(m);
    return 0;
}
int module_get_function(Function* out, Module m, const char* name) {
    auto* mod = static_cast<FakeModule*>(m);
    std::string needle(name);
    needle.push_back('\0');  // the symbol name as it sits in the string table
    if (mod->image.find(needle) == std::string::npos) return kNotFound;
    static std::vector<std::unique_ptr<FakeFunction>> functions;  // owned here, freed at process exit
    std::lock_guard<std::mutex> l(g_mu);
    functions.emplace_back(new FakeFunction{name});
    *out = functions.back().get();
    return 0;
}
int module_launch(Function f, const unsigned grid[3], const unsigned block[3], unsigned, Stream stream, void**) {
    for (int i = 0; i < 3; i++)
        if (grid[i] == 0 || block[i] == 0) return kInvalidValue;
    if (size_t(block[0]) * block[1] * block[2] > 1024) return kInvalidValue;
    std::lock_guard<std::mutex> l(g_mu);
    std::memcpy(g_last_grid, grid, sizeof g_last_grid);
    std::memcpy(g_last_block, block, sizeof g_last_block);
    g_last_kernel = static_cast<FakeFunction*>(f)->name;
    count_launch(stream);
    trace("launch:" + std::to_string(stream_no(stream)));
    return 0;
}

int stream_begin_capture(Stream s) {
    std::lock_guard<std::mutex> l(g_mu);
    if (g_capturing.count(s)) return kInvalidValue;
    g_capturing[s] = 0;
    return 0;
}
int stream_end_capture(Stream s, Graph* out) {
    std::lock_guard<std::mutex> l(g_mu);
    *out = nullptr;
    auto it = g_capturing.find(s);
    if (it == g_capturing.end()) return kInvalidValue;
    *out = new FakeGraph{it->second};
    g_capturing.erase(it);
    return 0;
}
int graph_instantiate(GraphExec* out, Graph g) {
    std::lock_guard<std::mutex> l(g_mu);
    *out = new FakeGraph{static_cast<FakeGraph*>(g)->launches};
    g_graphs_alive++;
    return 0;
}
int graph_launch(GraphExec e, Stream) {
    std::lock_guard<std::mutex> l(g_mu);
    g_launches += static_cast<FakeGraph*>(e)->launches;
    g_graph_launches++;
    return 0;
}
int graph_exec_destroy(GraphExec e) {
    std::lock_guard<std::mutex> l(g_mu);
    delete static_cast<FakeGraph*>(e);
    g_graphs_alive--;
    return 0;
}
int graph_destroy(Graph g) {
    delete static_cast<FakeGraph*>(g);
    return 0;
}

const char* error_name(int code) {
    switch (code) {
        case 0: return "hipSuccess";
        case 1: return "hipErrorInvalidValue";
        case 2: return "hipErrorOutOfMemory";
        case 100: return "hipErrorNoDevice";
        case 101: return "hipErrorInvalidDevice";
        case 200: return "hipErrorInvalidImage";
        case 500: return "hipErrorNotFound";
        case 600: return "hipErrorNotReady";
        default: return "hipErrorUnknown";
    }
}
void clear_last_error() {}

}  // namespace mrk::ffi
