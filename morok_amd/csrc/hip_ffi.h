// Thin hand-written FFI over the HIP runtime: the only place the host runtime touches
// HIP entry points (hipMalloc / hipMemcpyAsync / hipModuleLoadData /
// hipModuleLaunchKernel / hipEvent*).  It replaces what the reference reaches through
// the `cudarc` crate (device/src/allocator.rs:265-300, device/src/buffer.rs:351-366,
// 390-407,444-532, device/src/sync.rs:212-229,261-282), the custom ELF loader
// (runtime/src/jit_loader.rs:171-323) and the libffi dispatch
// (runtime/src/dispatch.rs:45-80).
//
// Every function returns the raw hipError_t as int (0 = hipSuccess).  Handles are opaque
// pointers so that host code above this layer includes no HIP header; a host-memory
// implementation of the same interface is linked in place of hip_ffi.cpp by the
// CPU-only test shim to exercise allocator, buffer and error-path logic without a GPU.
#pragma once
#include <cstddef>
#include <cstdint>

namespace mrk::ffi {

using Stream = void*;
using Event = void*;
using Module = void*;
using Function = void*;
using Graph = void*;
using GraphExec = void*;

int device_count(int* out);
int set_device(int device_id);

int malloc_device(void** out, size_t bytes);
int malloc_managed(void** out, size_t bytes);
int free_device(void* ptr);
int mem_info(size_t* free_bytes, size_t* total_bytes);

int memset_async(void* dst, int value, size_t bytes, Stream s);
int memcpy_htod_async(void* dst, const void* src, size_t bytes, Stream s);
int memcpy_dtoh_async(void* dst, const void* src, size_t bytes, Stream s);
int memcpy_dtod_async(void* dst, const void* src, size_t bytes, Stream s);

int stream_create(Stream* out);
int stream_destroy(Stream s);
int stream_synchronize(Stream s);
int device_synchronize();
// Makes all work queued on `s` after this call wait for `e` (hipStreamWaitEvent).
int stream_wait_event(Stream s, Event e);

int event_create(Event* out);
int event_destroy(Event e);
int event_record(Event e, Stream s);
int event_query(Event e);  // 0 = complete, kNotReady = still running
int event_synchronize(Event e);
int event_elapsed_ms(float* ms, Event start, Event stop);
extern const int kNotReady;

int module_load_data(Module* out, const void* image);
int module_unload(Module m);
int module_get_function(Function* out, Module m, const char* name);
// kernel_params: array of pointers to each argument (hipModuleLaunchKernel convention).
int module_launch(Function f, const unsigned grid[3], const unsigned block[3], unsigned shared_bytes, Stream s,
                  void** kernel_params);

// Stream capture into a graph (thread-local capture mode: other threads' calls are unaffected)
// and replay.  Only kernel launches are ever recorded by this library.
int stream_begin_capture(Stream s);
int stream_end_capture(Stream s, Graph* out);
int graph_instantiate(GraphExec* out, Graph g);
int graph_launch(GraphExec e, Stream s);
int graph_exec_destroy(GraphExec e);
int graph_destroy(Graph g);

const char* error_name(int code);
// Clears the sticky per-thread error state of the runtime after a failed call.
void clear_last_error();

}  // namespace mrk::ffi
