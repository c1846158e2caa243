#include "hip_ffi.h"

#include <hip/hip_runtime_api.h>

namespace mrk::ffi {

const int kNotReady = static_cast<int>(hipErrorNotReady);

int device_count(int* out) { return hipGetDeviceCount(out); }
int set_device(int device_id) { return hipSetDevice(device_id); }

int malloc_device(void** out, size_t bytes) { return hipMalloc(out, bytes); }
int malloc_managed(void** out, size_t bytes) { return hipMallocManaged(out, bytes, hipMemAttachGlobal); }
int free_device(void* ptr) { return hipFree(ptr); }
int mem_info(size_t* free_bytes, size_t* total_bytes) { return hipMemGetInfo(free_bytes, total_bytes); }

int memset_async(void* dst, int value, size_t bytes, Stream s) {
    return hipMemsetAsync(dst, value, bytes, static_cast<hipStream_t>(s));
}
int memcpy_htod_async(void* dst, const void* src, size_t bytes, Stream s) {
    return hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(s));
}
int memcpy_dtoh_async(void* dst, const void* src, size_t bytes, Stream s) {
    return hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(s));
}
int memcpy_dtod_async(void* dst, const void* src, size_t bytes, Stream s) {
    return hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(s));
}

int stream_create(Stream* out) {
    hipStream_t s = nullptr;
    // Default priority on purpose: every stream of this runtime has the same priority.
    int rc = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
    *out = s;
    return rc;
}
int stream_destroy(Stream s) { return hipStreamDestroy(static_cast<hipStream_t>(s)); }
int stream_synchronize(Stream s) { return hipStreamSynchronize(static_cast<hipStream_t>(s)); }
int stream_wait_event(Stream s, Event e) {
    return hipStreamWaitEvent(static_cast<hipStream_t>(s), static_cast<hipEvent_t>(e), 0);
}
int device_synchronize() { return hipDeviceSynchronize(); }

int event_create(Event* out) {
    hipEvent_t e = nullptr;
    int rc = hipEventCreate(&e);
    *out = e;
    return rc;
}
int event_destroy(Event e) { return hipEventDestroy(static_cast<hipEvent_t>(e)); }
int event_record(Event e, Stream s) { return hipEventRecord(static_cast<hipEvent_t>(e), static_cast<hipStream_t>(s)); }
int event_query(Event e) { return hipEventQuery(static_cast<hipEvent_t>(e)); }
int event_synchronize(Event e) { return hipEventSynchronize(static_cast<hipEvent_t>(e)); }
int event_elapsed_ms(float* ms, Event start, Event stop) {
    return hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop));
}

int module_load_data(Module* out, const void* image) {
    hipModule_t m = nullptr;
    int rc = hipModuleLoadData(&m, image);
    *out = m;
    return rc;
}
int module_unload(Module m) { return hipModuleUnload(static_cast<hipModule_t>(m)); }
int module_get_function(Function* out, Module m, const char* name) {
    hipFunction_t f = nullptr;
    int rc = hipModuleGetFunction(&f, static_cast<hipModule_t>(m), name);
    *out = f;
    return rc;
}
int module_launch(Function f, const unsigned grid[3], const unsigned block[3], unsigned shared_bytes, Stream s,
                  void** kernel_params) {
    return hipModuleLaunchKernel(static_cast<hipFunction_t>(f), grid[0], grid[1], grid[2], block[0], block[1],
                                 block[2], shared_bytes, static_cast<hipStream_t>(s), kernel_params, nullptr);
}

int stream_begin_capture(Stream s) {
    return static_cast<int>(hipStreamBeginCapture(static_cast<hipStream_t>(s), hipStreamCaptureModeThreadLocal));
}
int stream_end_capture(Stream s, Graph* out) {
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(static_cast<hipStream_t>(s), &g);
    *out = g;
    return static_cast<int>(e);
}
int graph_instantiate(GraphExec* out, Graph g) {
    hipGraphExec_t x = nullptr;
    hipError_t e = hipGraphInstantiate(&x, static_cast<hipGraph_t>(g), nullptr, nullptr, 0);
    *out = x;
    return static_cast<int>(e);
}
int graph_launch(GraphExec e, Stream s) {
    return static_cast<int>(hipGraphLaunch(static_cast<hipGraphExec_t>(e), static_cast<hipStream_t>(s)));
}
int graph_exec_destroy(GraphExec e) { return static_cast<int>(hipGraphExecDestroy(static_cast<hipGraphExec_t>(e))); }
int graph_destroy(Graph g) { return static_cast<int>(hipGraphDestroy(static_cast<hipGraph_t>(g))); }

const char* error_name(int code) { return hipGetErrorName(static_cast<hipError_t>(code)); }
void clear_last_error() { (void)hipGetLastError(); }

}  // namespace mrk::ffi
