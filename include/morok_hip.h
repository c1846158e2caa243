/*
 * morok_hip.h - C ABI of libmorok_hip.so, the MI355X (gfx950) device backend for morok.
 *
 * The library sits behind morok's device boundary
 *     Device { Renderer, Compiler, RuntimeFactory -> Program, Allocator }
 * (device/src/device.rs) and exports one C entry point per trait method a Rust shim
 * would bind.  Each declaration cites the reference interface it stands for; paths are
 * relative to the morok workspace root.
 *
 * Conventions
 *   - every function returning int returns 0 on success, otherwise one of MRK_ERR_*;
 *     the message is available from mrk_hip_last_error() (thread-local, valid until the
 *     next failing call on the same thread).  No call panics or aborts across the ABI.
 *   - all device work of one device id is queued on a single in-order HIP stream
 *     (the execution loop of runtime/src/execution_plan.rs:168-181 relies on in-order
 *     execution and never synchronises between kernels); copyout synchronises.
 *   - launch dimensions: global_size = grid extent in workgroups, local_size = workgroup
 *     extent in work-items (the gidx/lidx extents of schedule/src/gpudims.rs:153-156).
 *   - all entry points are thread-safe (Renderer/Compiler are Send + Sync in the
 *     reference, device.rs:142,186; kernels are shared across threads by the kernel cache,
 *     runtime/src/kernel_cache.rs:46-50).
 */
#ifndef MOROK_HIP_H
#define MOROK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes: variants of device/src/error.rs:5-51 ---- */
#define MRK_OK 0
#define MRK_ERR_SIZE_MISMATCH 1      /* Error::SizeMismatch */
#define MRK_ERR_COPY_FAILED 2        /* Error::CopyFailed */
#define MRK_ERR_INVALID_DEVICE 3     /* Error::InvalidDevice */
#define MRK_ERR_NOT_ALLOCATED 4      /* Error::NotAllocated */
#define MRK_ERR_NOT_CPU_ACCESSIBLE 5 /* Error::NotCpuAccessible */
#define MRK_ERR_INVALID_VIEW 6       /* Error::InvalidView */
#define MRK_ERR_RUNTIME 7            /* Error::Runtime */
#define MRK_ERR_HIP 8                /* backend variant, cf. Error::CudaError (error.rs:47-50) */
#define MRK_ERR_RENDER 9             /* RenderKernel context, tensor/src/realize.rs:42-46 */
#define MRK_ERR_COMPILE 10           /* CompileKernel context */
#define MRK_ERR_INVALID_ARGUMENT 11
#define MRK_ERR_TIMEOUT 12           /* TimelineSignal::wait timeout, device/src/sync.rs:118-168 */
#define MRK_ERR_UNSUPPORTED_DEVICE 13 /* runtime/src/device_registry.rs:114-120 */

const char* mrk_hip_last_error(void);

/* ---- opaque handles ---- */
typedef struct mrk_buffer mrk_buffer;               /* device::Buffer        (device/src/buffer.rs:97-110) */
typedef struct mrk_program_spec mrk_program_spec;   /* device::ProgramSpec   (device/src/device.rs:327-367) */
typedef struct mrk_compiled_spec mrk_compiled_spec; /* device::CompiledSpec  (device/src/device.rs:72-100) */
typedef struct mrk_program mrk_program;             /* Box<dyn Program>      (device/src/device.rs:34-60) */
typedef struct mrk_kernel mrk_kernel;               /* Arc<CachedKernel>     (runtime/src/kernel_cache.rs:27-44) */
typedef struct mrk_plan mrk_plan;                   /* ExecutionPlan         (runtime/src/execution_plan.rs:84-106) */
typedef struct mrk_signal mrk_signal;               /* TimelineSignal        (device/src/sync.rs:44-71) */
typedef struct mrk_event mrk_event;                 /* hipEvent pair member for timing */

/* =====================================================================================
 * Device registry and factory
 * ===================================================================================== */

/* DeviceSpecExt::parse (device/src/registry.rs:26-81) with the HIP arm: accepts
 * "HIP", "HIP:n", "AMD[:n]", "GPU[:n]" (case-insensitive); anything else -> INVALID_DEVICE. */
int mrk_hip_device_parse(const char* spec, int* device_id);
/* Number of visible HIP devices. */
int mrk_hip_device_count(int* count);
/* DEVICE_FACTORIES.device(spec, registry) (runtime/src/device_registry.rs:99-127): creates
 * (once) the device bundle - allocator, renderer, compiler, runtime factory - for the id.
 * Registered under the base type string "HIP" (register_factory, device_registry.rs:81-83). */
int mrk_hip_device_create(int device_id);
/* Looks a factory up by base type string; unknown types -> UNSUPPORTED_DEVICE
 * (device_registry.rs:114-120). */
int mrk_hip_device_create_by_type(const char* device_type, int device_id);
/* Allocator::name (device/src/allocator.rs:186) / Device::base_device_key (device.rs:310-312). */
const char* mrk_hip_name(void);
/* The device's HIP stream (hipStream_t) for interop with caller-side HIP code. */
int mrk_hip_device_stream(int device_id, void** stream);

/* =====================================================================================
 * Allocator (device/src/allocator.rs:180-190) behind the LRU cache (allocator.rs:330-442)
 * ===================================================================================== */

/* Allocator::alloc(size, &BufferOptions{zero_init, cpu_accessible}).
 * cpu_accessible = 0 -> hipMalloc; 1 -> hipMallocManaged (as CudaUnified, allocator.rs:278-286). */
int mrk_hip_alloc(int device_id, size_t size, int zero_init, int cpu_accessible, void** out);
/* Allocator::free: parks the allocation in the LRU cache (<= 32 per (size, cpu_accessible)). */
int mrk_hip_free(int device_id, void* ptr, size_t size, int cpu_accessible);
/* Allocator::synchronize (allocator.rs:183-185). */
int mrk_hip_sync(int device_id);
/* LruAllocator::cache_count / total_cached (allocator.rs:350-363) and cache clear. */
int mrk_hip_lru_cache_count(int device_id, size_t size, int cpu_accessible, size_t* count);
int mrk_hip_lru_total_cached(int device_id, size_t* count);
int mrk_hip_lru_clear(int device_id);
/* Raw copies for callers that hold device pointers from mrk_hip_alloc
 * (device/src/buffer.rs:351-366,390-407,444-532).  copyout waits for everything queued on the
 * device's own stream first; work submitted through an mrk_queue runs on that queue's stream
 * and needs mrk_hip_queue_synchronize (or a signal wait) before its results are copied out. */
int mrk_hip_copyin(int device_id, void* dst, size_t dst_offset, const void* src_host, size_t size);
int mrk_hip_copyout(int device_id, void* dst_host, const void* src, size_t src_offset, size_t size);
int mrk_hip_copy_dd(int device_id, void* dst, size_t dst_offset, const void* src, size_t src_offset, size_t size);

/* =====================================================================================
 * Buffer (device/src/buffer.rs)
 * ===================================================================================== */

/* Buffer::new (buffer.rs:112-121): lazy, nothing is allocated until first use. */
int mrk_hip_buffer_new(int device_id, size_t size, int zero_init, int cpu_accessible, mrk_buffer** out);
/* Buffer::ensure_allocated / is_allocated (buffer.rs:153-160). */
int mrk_hip_buffer_ensure_allocated(mrk_buffer* b);
int mrk_hip_buffer_is_allocated(const mrk_buffer* b);
/* Buffer::view (buffer.rs:136-150): shares the allocation and the id; INVALID_VIEW when
 * offset + size exceeds the buffer. */
int mrk_hip_buffer_view(const mrk_buffer* b, size_t offset, size_t size, mrk_buffer** out);
/* Buffer::copyin / copyout / copy_from (buffer.rs:332-368,371-408,411-534): SIZE_MISMATCH
 * unless the byte counts match exactly. */
int mrk_hip_buffer_copyin(mrk_buffer* b, const void* src, size_t size);
int mrk_hip_buffer_copyout(const mrk_buffer* b, void* dst, size_t size);
int mrk_hip_buffer_copy_from(mrk_buffer* dst, const mrk_buffer* src);
/* Buffer::as_raw_ptr (buffer.rs:554-574): device address + view offset; NOT_ALLOCATED before
 * allocation (the reference panics). */
int mrk_hip_buffer_raw_ptr(const mrk_buffer* b, void** out);
/* Buffer::id / size (buffer.rs:327-329). */
uint64_t mrk_hip_buffer_id(const mrk_buffer* b);
size_t mrk_hip_buffer_size(const mrk_buffer* b);
/* Buffer::synchronize (buffer.rs:537-539). */
int mrk_hip_buffer_synchronize(const mrk_buffer* b);
/* Drop: the allocation returns to the allocator when the last view is released
 * (buffer.rs:86-93). */
void mrk_hip_buffer_release(mrk_buffer* b);

/* =====================================================================================
 * Compiler (device/src/device.rs:142-177) and ProgramSpec / CompiledSpec accessors
 * ===================================================================================== */

/* Renderer::render(&Arc<UOp>, Option<&str>) -> ProgramSpec (device/src/device.rs:186-222;
 * reference implementation CRenderer::render, codegen/src/c/mod.rs:47-270).  `kernel` is the
 * serialized linearized stream - the Vec<Arc<UOp>> after linearize_with_cfg +
 * line_rewrite_cleanups (schedule/src/linearize/mod.rs:172-177,308-310) - in the wire format
 * documented in morok_amd/csrc/uop.h; `name` may be NULL (falls back to "kernel",
 * device.rs:192-193).  Emits HIP-C for gfx950: SPECIAL -> blockIdx/threadIdx with the launch
 * dims taken from the extents, DEFINE_LOCAL -> __shared__, BARRIER -> __syncthreads(),
 * WMMA -> MFMA builtin.  Works without a GPU.  Renderer::decompositor is None for this
 * backend (all transcendental ops map to device math functions, cf. c/mod.rs:276-280). */
int mrk_hip_render(int device_id, const uint8_t* kernel, size_t len, const char* name, mrk_program_spec** out);

/* Builds a ProgramSpec from already-rendered HIP-C source (what Renderer::render returns).
 * var_is_i64[i] != 0 -> scalar argument i is `long long`, else `int`.  global/local may be
 * NULL when the launch sizes are supplied at execute time. */
int mrk_hip_program_spec_from_source(const char* name, const char* src, size_t buf_count, const char* const* var_names,
                                     const uint8_t* var_is_i64, size_t nvars, const size_t global_size[3],
                                     const size_t local_size[3], mrk_program_spec** out);
const char* mrk_hip_program_spec_name(const mrk_program_spec* s);
const char* mrk_hip_program_spec_src(const mrk_program_spec* s);
size_t mrk_hip_program_spec_buf_count(const mrk_program_spec* s);
size_t mrk_hip_program_spec_var_count(const mrk_program_spec* s);
const char* mrk_hip_program_spec_var_name(const mrk_program_spec* s, size_t i);
/* Returns 1 and fills the arrays if the spec carries launch sizes, else 0. */
int mrk_hip_program_spec_sizes(const mrk_program_spec* s, size_t global_size[3], size_t local_size[3]);
/* globals / outs / ins PARAM slot lists (device.rs:353-363): which = 0,1,2. */
size_t mrk_hip_program_spec_slots(const mrk_program_spec* s, int which, size_t* out, size_t cap);
void mrk_hip_program_spec_release(mrk_program_spec* s);

/* Compiler::compile (device.rs:170): HIP-C -> gfx950 code object, in process.  AOT
 * convention (device.rs:118-120,153-169): bytes populated, src absent. */
int mrk_hip_compile(const mrk_program_spec* spec, mrk_compiled_spec** out);
/* Compiler::cache_key (device.rs:176): "hip-gfx950". */
const char* mrk_hip_cache_key(void);
const char* mrk_hip_compiled_spec_name(const mrk_compiled_spec* c);
size_t mrk_hip_compiled_spec_bytes(const mrk_compiled_spec* c, const uint8_t** bytes);
int mrk_hip_compiled_spec_has_src(const mrk_compiled_spec* c);
void mrk_hip_compiled_spec_release(mrk_compiled_spec* c);

/* =====================================================================================
 * RuntimeFactory and Program (device/src/device.rs:34-60,234)
 * ===================================================================================== */

/* RuntimeFactory(&CompiledSpec) -> Box<dyn Program>: hipModuleLoadData +
 * hipModuleGetFunction(spec.name). */
int mrk_hip_program_create(int device_id, const mrk_compiled_spec* spec, mrk_program** out);
/* Program::execute(buffers, vals, global_size, local_size) (device.rs:50-56):
 * hipModuleLaunchKernel with the buffer pointers first, then vals in var_names order
 * (same positional order as runtime/src/dispatch.rs:67-69).  global/local may be NULL to
 * use the sizes recorded in the spec.  Asynchronous: returns once the launch is queued. */
int mrk_hip_program_execute(mrk_program* p, void* const* buffers, size_t nbufs, const int64_t* vals, size_t nvals,
                            const size_t global_size[3], const size_t local_size[3]);
/* Program::name (device.rs:59). */
const char* mrk_hip_program_name(const mrk_program* p);
void mrk_hip_program_destroy(mrk_program* p);

/* Hand-written gfx950 kernels exposed as Programs, so that an ExecutionPlan can hold them
 * next to generated kernels.  `kind` and the meaning of `params`:
 *   "softmax_f32"     params = {rows, cols}                         buffers = {y, x}
 *   "gemm_bf16"       params = {M, N, K} or {M, N, K, batch}        buffers = {c, a, b}
 *                     (batch: that many products over matrices stored back to back)
 *                     params = {M, N, K, batch, workspace bytes}    buffers = {c, a, b, workspace}
 *                     (split-K for shapes with few output tiles; size from mrk_hip_gemm_bf16_workspace_bytes)
 *   "gemm_bf16_residual"  params = {M, N, K} or {M, N, K, batch}  buffers = {c, a, b, r}   (c = a b + r)
 *   "gemm_bf16_bias"      params = {M, N, K} or {M, N, K, batch}  buffers = {c, a, b, bias} (c = a b + bias, bias [N])
 *   "gemm_bf16_swiglu"    params = {M, F, K}                      buffers = {c, a, w}      (w = gate | up, [K, 2F])
 *   "gemm_bf16_nt", "gemm_bf16_nt_residual", "gemm_bf16_nt_bias", "gemm_bf16_nt_swiglu": the same with the second operand
 *                     stored transposed, [N, K] ([2F, K], gate rows first), as a Linear layer holds its
 *                     weight (tensor/src/nn/linear.rs:9-14: y = x @ weight.T + bias); the same bits as
 *                     the [K, N] kinds.  No split-K form: shapes with a workspace size > 0 are refused.
 *   "flash_fwd_bf16"  params = {B*H, Sq, Sk, D, causal, f32 bits of scale}   buffers = {o, q, k, v}
 *   "flash_fwd_bf16_strided"  params = {B, H, Sq, Sk, D, causal, f32 bits of scale, element offsets
 *                     of q k v o into their buffers (4), (batch, head, row) element strides of
 *                     q k v o (12)}                                  buffers = {o, q, k, v}
 *                     (both: optionally one more parameter, the bytes of a scratch buffer that follows v:
 *                     mrk_hip_flash_attn_workspace_bytes, for a key sequence split over workgroups)
 * Buffer order follows the reference's PARAM numbering: outputs first. */
int mrk_hip_program_builtin(int device_id, const char* kind, const int64_t* params, size_t nparams, mrk_program** out);

/* =====================================================================================
 * Kernel cache (runtime/src/kernel_cache.rs) and execution plan (runtime/src/execution_plan.rs)
 * ===================================================================================== */

/* get_or_compile_kernel(ast_id, device, || render; compile; runtime) (kernel_cache.rs:87-118;
 * call site tensor/src/realize.rs:1052-1070): the kernel is looked up by the content hash of
 * the linearized stream, the device string and the compiler's cache_key; on a miss it goes
 * through the three boundary hooks.  *was_cached (may be NULL) tells which happened. */
int mrk_hip_kernel_get_or_compile(int device_id, const uint8_t* kernel, size_t len, const char* name, mrk_kernel** out,
                                  int* was_cached);
/* Same cache for a hand-written kernel (kinds and params as for mrk_hip_program_builtin). */
int mrk_hip_kernel_builtin(int device_id, const char* kind, const int64_t* params, size_t nparams, mrk_kernel** out);
/* CachedKernel fields (kernel_cache.rs:27-44). */
const char* mrk_hip_kernel_entry_point(const mrk_kernel* k);
const char* mrk_hip_kernel_code(const mrk_kernel* k);
size_t mrk_hip_kernel_var_count(const mrk_kernel* k);
const char* mrk_hip_kernel_var_name(const mrk_kernel* k, size_t i);
/* 1 if both handles share one cached kernel (Arc pointer identity). */
int mrk_hip_kernel_same(const mrk_kernel* a, const mrk_kernel* b);
void mrk_hip_kernel_release(mrk_kernel* k);
size_t mrk_hip_kernel_cache_size(void);
/* clear_all (kernel_cache.rs:124-130). */
void mrk_hip_kernel_cache_clear(void);

/* ExecutionPlanBuilder (execution_plan.rs:330-411): buffers are owned by the plan; kernels
 * refer to them by index in the order the kernel expects (outputs first). */
int mrk_hip_plan_create(int device_id, mrk_plan** out);
int mrk_hip_plan_add_buffer(mrk_plan* plan, const mrk_buffer* b, size_t* index);
int mrk_hip_plan_add_kernel(mrk_plan* plan, const mrk_kernel* k, const size_t* buffer_indices, size_t nbufs,
                            const int64_t* vals, size_t nvals);
/* ensure_allocated on every buffer and precompute the raw pointers (execution_plan.rs:391-397). */
int mrk_hip_plan_build(mrk_plan* plan);
/* ExecutionPlan::execute (execution_plan.rs:168-181): launches every kernel in order on the
 * device stream; no synchronisation between kernels. */
int mrk_hip_plan_execute(mrk_plan* plan);
/* The launches of mrk_hip_plan_execute replayed as one HIP graph: the first call records them
 * on the device's stream and instantiates the graph, later calls are one hipGraphLaunch.  No
 * counterpart in the reference (its CPU kernels are plain function calls); for plans of many
 * short kernels, where per-launch submission cost dominates.  The plan must be rebuilt-free:
 * mrk_hip_plan_execute_with_vars or adding kernels drops the recorded graph. */
int mrk_hip_plan_execute_graph(mrk_plan* plan);
/* ExecutionPlan::execute_profiled (execution_plan.rs:200-221): per-kernel elapsed time in ms,
 * measured with HIP events (the reference uses Instant around blocking CPU calls). */
int mrk_hip_plan_execute_profiled(mrk_plan* plan, double* elapsed_ms, size_t cap, size_t* count);
/* ExecutionPlan::execute_with_vars (execution_plan.rs:239-250): rebind variables by name. */
int mrk_hip_plan_execute_with_vars(mrk_plan* plan, const char* const* names, const int64_t* vals, size_t n);
size_t mrk_hip_plan_kernel_count(const mrk_plan* plan);
const char* mrk_hip_plan_kernel_name(const mrk_plan* plan, size_t i);
void mrk_hip_plan_release(mrk_plan* plan);

/* benchmark_kernel (runtime/src/benchmark.rs:64-91; protocol 23-27: warm-up runs, timed runs,
 * minimum), timed with HIP events so that asynchronous launches are measured correctly - the
 * hook beam search needs (tensor/src/realize.rs:1190-1242). */
int mrk_hip_benchmark_kernel(int device_id, mrk_program* p, void* const* buffers, size_t nbufs, const int64_t* vals,
                             size_t nvals, const size_t global_size[3], const size_t local_size[3], int warmup, int runs,
                             double* min_ms, double* mean_ms);

/* benchmark_kernel_with_cutoff (runtime/src/benchmark.rs:100-137): as above, but when the first timed
 * run takes more than three times cutoff_ms the candidate is given up at once: *skipped = 1 and the
 * times are those of that one run.  cutoff_ms <= 0 disables the check. */
int mrk_hip_benchmark_kernel_with_cutoff(int device_id, mrk_program* p, void* const* buffers, size_t nbufs, const int64_t* vals,
                                         size_t nvals, const size_t global_size[3], const size_t local_size[3], int warmup,
                                         int runs, double cutoff_ms, double* min_ms, double* mean_ms, int* skipped);

/* TimelineSignal::{set, value, wait(value, timeout_ms)} (device/src/sync.rs:44-71), modelled on
 * CudaTimelineSignal (sync.rs:192-310): one event per recorded value, the last 16 kept.
 * wait returns MRK_ERR_TIMEOUT when the value is not reached in time (sync.rs:118-168). */
int mrk_hip_signal_create(int device_id, mrk_signal** out);
int mrk_hip_signal_set(mrk_signal* s, uint64_t value);
uint64_t mrk_hip_signal_value(mrk_signal* s);
int mrk_hip_signal_wait(mrk_signal* s, uint64_t value, uint64_t timeout_ms);
void mrk_hip_signal_destroy(mrk_signal* s);

/* =====================================================================================
 * Hardware queues (device/src/queue.rs:76-161) over HIP streams of default priority.
 * Commands are batched and reach the queue's stream on submit; ordering between queues is
 * expressed with timeline signals, which become hipStreamWaitEvent dependencies on the GPU
 * (QueueFactory::create_compute_queue / create_copy_queue / create_signal, queue.rs:136-161).
 * ===================================================================================== */
typedef struct mrk_queue mrk_queue;
int mrk_hip_queue_create(int device_id, int copy_queue, mrk_queue** out);
/* HardwareQueue::wait / signal (queue.rs:93-105). */
int mrk_hip_queue_wait(mrk_queue* q, mrk_signal* s, uint64_t value);
int mrk_hip_queue_signal(mrk_queue* q, mrk_signal* s, uint64_t value);
/* HardwareQueue::exec (queue.rs:107-121): global/local may be null (sizes recorded at compile
 * time are used, ExecParams default). */
int mrk_hip_queue_exec(mrk_queue* q, const mrk_kernel* k, mrk_buffer* const* buffers, size_t nbufs, const int64_t* vals,
                       size_t nvals, const size_t* global, const size_t* local);
/* HardwareQueue::copy (queue.rs:123-128): device-to-device, SIZE_MISMATCH at submit unless
 * the sizes are equal. */
int mrk_hip_queue_copy(mrk_queue* q, mrk_buffer* dst, const mrk_buffer* src);
/* HardwareQueue::memory_barrier (queue.rs:130-134): a HIP stream executes in order; records nothing. */
int mrk_hip_queue_memory_barrier(mrk_queue* q);
/* HardwareQueue::submit (queue.rs:136-141): hands the batch to the stream without waiting for it.
 * A wait on a value that no queue has signalled yet is retried for wait_timeout_ms, then TIMEOUT. */
int mrk_hip_queue_submit(mrk_queue* q, uint64_t wait_timeout_ms);
int mrk_hip_queue_synchronize(mrk_queue* q);
size_t mrk_hip_queue_pending(const mrk_queue* q);
void mrk_hip_queue_destroy(mrk_queue* q);

/* =====================================================================================
 * Scheduling helpers for the gfx950 target (what morok's `schedule` crate supplies per backend)
 * ===================================================================================== */

/* Renderer::amd_cdna4() capability descriptor (schedule/src/optimizer/renderer.rs:290-303) as
 * "key=value;..." text: device, has_local, has_shared, has_threads, shared_max, global_max,
 * local_max, upcast_max, tensor_cores (WMMA names in table order). */
const char* mrk_hip_sched_caps(void);
/* select_tensor_core (schedule/src/optimizer/tc.rs:126-168) over cdna4_tensor_cores()
 * (renderer.rs:724-733): scalar dtype tags as in morok_amd/csrc/uop.h; -1 if none matches.
 * The table holds the reference's six entries in its order (indices 0-5: fp8e5m2, fp8e4m3, f16,
 * bf16 as 16x16x32; f16, bf16 as 16x16x16) and, behind them, two that the reference does not
 * have: f16 and bf16 as 32x32x16 (indices 6, 7), reachable by index only. */
int mrk_hip_sched_tc_select(int in0_scalar, int in1_scalar, int acc_scalar);
/* TensorCore fields (renderer.rs:358-417): dims (N, M, K), threads, elements per lane (A, B, C). */
int mrk_hip_sched_tc_info(int tc_index, int dims[3], int* threads, int elements_per_thread[3]);
/* Which matrix element a lane's operand element is, derived from the table's opts and
 * swizzle (tc.rs:175-215): operand 0 = A -> (m, k), 1 = B -> (n, k), 2 = C -> (m, n). */
int mrk_hip_sched_tc_operand_element(int tc_index, int operand, int lane, int elem, int* mn, int* k);
/* gpudims helpers (schedule/src/gpudims.rs:387-463,529-584). group_dims / get_contraction return 1
 * on success and 0 when no grouping / contraction exists. */
size_t mrk_hip_sched_find_smallest_divisor(size_t n);
int mrk_hip_sched_group_dims(const size_t* dims, size_t n, const size_t* max_sizes, size_t nmax, size_t* out, size_t cap,
                             size_t* nout);
int mrk_hip_sched_split_dims(const size_t* dims, size_t n, const size_t* max_sizes, size_t nmax, size_t* out, size_t cap,
                             size_t* nout);
int mrk_hip_sched_limit_dims(const size_t* dims, size_t n, const size_t* max_sizes, size_t nmax, size_t* out, size_t cap,
                             size_t* nout);
int mrk_hip_sched_get_contraction(const size_t* original, size_t n, const size_t* limited, size_t nl, size_t* group_of_dim);
/* get_grouped_dims (gpudims.rs:331-382): launch extents for `dims` under `max_sizes` (NULL = no
 * limit) and, when raw/index_per_dim are given, the index of every original dimension for one
 * tuple of hardware indices.  reverse: 0 = local indices (dims as given); 1 = global indices as
 * this backend launches them: the dims are reversed before limiting and the indices after it, so
 * the innermost axis is gidx0 whatever regrouping happened (tinygrad's order); 2 = the reference's
 * literal code, which limits the dims as given and reverses only the index list.  Modes 1 and 2
 * agree exactly when the dims read the same in both directions (one dim, [a, a], [a, b, a] ...);
 * for every other dims list mode 2 gives dimension i an index that runs over the extent of
 * dimension n-1-i (for [3, 5]: dimension 0 gets an index in [0, 5)), which is why generated
 * kernels use mode 1.  A caller comparing with the reference's unit tests wants mode 2. */
int mrk_hip_sched_grouped_dims(const size_t* dims, size_t n, const size_t* max_sizes, size_t nmax, int reverse,
                               size_t* launch, size_t cap, size_t* nlaunch, const size_t* raw, size_t* index_per_dim);
/* Linearized kernels for the matmul shapes on the hot path, serialized in the wire format
 * (free with mrk_hip_sched_free): the f32 matmul kernel (LOCAL 16x16, UPCAST 4x4) and the
 * tensor-core matmul that tc::apply produces (tc.rs:358-674) with post-TC upcasts
 * (schedule/src/optimizer/heuristics.rs:787-821). */
int mrk_hip_sched_build_matmul_f32(int64_t m, int64_t n, int64_t k, uint8_t** kernel, size_t* len);
int mrk_hip_sched_build_wmma_matmul(int tc_index, int64_t m, int64_t n, int64_t k, int out_scalar, uint8_t** kernel,
                                    size_t* len);
/* The same product with both operands staged through local memory by a workgroup of 2 x 2 waves
 * (128 x 128 output tile): the GROUP / LOCAL step of the optimizer
 * (schedule/src/optimizer/heuristics.rs:37-82) applied after the tensor-core rewrite.  Extents
 * the tile does not divide are padded (PADTO, tc.rs:400-432: gated loads, guarded stores); N and
 * K must be multiples of 8 (16-byte copies). */
int mrk_hip_sched_build_wmma_matmul_lds(int tc_index, int64_t m, int64_t n, int64_t k, int out_scalar, uint8_t** kernel,
                                        size_t* len);
/* The same with the choices explicit: opts = {waves_m, waves_n (LOCAL: the grid of waves in a
 * workgroup), tiles_m, tiles_n (UPCAST: 16x16 tensor-core tiles per wave), K steps per barrier
 * pair (UNROLL; 0 = as many as divide K, up to 64 elements), stages}.  stages = 0: tiles travel
 * global -> registers -> local memory; stages = 2: two stages per tile filled by direct
 * global -> local copies, B fragments through the transposing local load, one barrier per
 * 64-deep K step, workgroups mapped to tiles per XCD (16x16x32 tensor cores; m, n, k must be
 * multiples of the workgroup tile and of 64).  All powers of two; INVALID_ARGUMENT for choices
 * whose tiles do not split into whole copies per work-item / wave or exceed local memory. */
int mrk_hip_sched_build_wmma_matmul_lds_opts(int tc_index, int64_t m, int64_t n, int64_t k, int out_scalar, const int opts[6],
                                             uint8_t** kernel, size_t* len);
void mrk_hip_sched_free(void* p);
/* The f32 matmul kernel with the optimisation choices explicit: opts = {LOCAL x, LOCAL y,
 * UPCAST of N (vector width 1/2/4), UPCAST of M (rows per work-item 1..8), UNROLL of K,
 * GROUP depth}.  GROUP depth 0: operands straight from global memory.  8 / 16 / 32: the
 * workgroup stages A and B tiles of that K depth through local memory (UPCAST 4 or 8 each way,
 * UNROLL ignored; schedule/src/optimizer/heuristics.rs:37-82).  INVALID_ARGUMENT when the choices
 * do not divide the shape (the action space of schedule/src/optimizer/beam.rs:36-120 restricted
 * to this kernel). */
int mrk_hip_sched_build_matmul_f32_opts(int64_t m, int64_t n, int64_t k, const int opts[6], uint8_t** kernel, size_t* len);

/* =====================================================================================
 * Beam-search support (tensor/src/realize.rs:1190-1242, schedule/src/optimizer/beam.rs)
 * ===================================================================================== */
/* compile_and_time: render + compile + load (not timed), then warm-up and `runs` timed
 * launches with HIP events on the device stream; *min_ms is the minimum
 * (runtime/src/benchmark.rs:23-27,64-91).  Candidates are timed one at a time however many
 * threads call this.  A candidate that does not render / compile / launch returns a status,
 * it never aborts the process. */
int mrk_hip_compile_and_time(int device_id, const void* kernel, size_t len, const char* name, mrk_buffer* const* buffers,
                             size_t nbufs, const int64_t* vals, size_t nvals, int warmup, int runs, double* min_ms);
/* On-disk result cache keyed (ast_hash, beam_width, device string) (beam.rs:390-440; sled in the
 * reference, one file per key here, under $MOROK_CACHE_DIR | $XDG_CACHE_HOME/morok |
 * $HOME/.cache/morok, in beam_cache_hip/).  get: *len = 0 on a miss (and always when
 * IGNORE_BEAM_CACHE is set); INVALID_ARGUMENT if the value exceeds capacity. */
int mrk_hip_beam_cache_get(uint64_t ast_hash, int width, const char* device, void* value, size_t capacity, size_t* len);
int mrk_hip_beam_cache_put(uint64_t ast_hash, int width, const char* device, const void* value, size_t len);
/* Beam search of width `width` over LOCAL / UPCAST / UNROLL / GROUP for the f32 matmul of this
 * shape; result in opts (same six-entry layout as above), its time in *best_ms, *from_cache = 1
 * when the disk cache answered, *timed = number of candidates compiled and timed. */
int mrk_hip_beam_search_matmul_f32(int device_id, int64_t m, int64_t n, int64_t k, int width, int opts[6],
                                   double* best_ms, int* from_cache, int* timed);
/* The same search over the LDS-staged tensor-core matmul of mrk_hip_sched_build_wmma_matmul_lds_opts
 * (bf16 / f16 in and out, tensor core `tc_index` of mrk_hip_sched_tensor_cores): the TC action
 * of tc.rs:358-674 first, then LOCAL / UPCAST / UNROLL as above.  opts = {waves_m, waves_n,
 * tiles_m per wave, tiles_n per wave, K steps per barrier pair, stages}. */
int mrk_hip_beam_search_wmma_matmul(int device_id, int tc_index, int64_t m, int64_t n, int64_t k, int width, int opts[6],
                                    double* best_ms, int* from_cache, int* timed);

/* =====================================================================================
 * Hand-written kernels, direct entry points (device pointers, queued on the device stream)
 * ===================================================================================== */

/* Fused row softmax over the last axis, f32 [rows, cols] row-major: the lazy graph of
 * Tensor::softmax (tensor/src/activation.rs:90-101) in one kernel instead of the
 * reference's three (tensor/src/test/unit/fusion.rs:83-88). */
int mrk_hip_softmax_f32(int device_id, const void* x, void* y, int64_t rows, int64_t cols);
/* Same with an explicit implementation variant (0 default, 1 one-wave-per-row); tuning only. */
int mrk_hip_softmax_f32_variant(int device_id, const void* x, void* y, int64_t rows, int64_t cols, int variant);

/* C[M,N] = A[M,K] @ B[K,N], row-major bf16, f32 accumulation on MFMA, bf16 result: the
 * lazy graph of Tensor::matmul on bf16 operands (tensor/src/matmul.rs:82-110; accumulator
 * promotion tensor/src/reduce.rs:101-117) as the tensor-core rewrite leaves it
 * (schedule/src/optimizer/tc.rs:36-94).  Any shape; shapes with M,N % 256 == 0 and
 * K % 64 == 0 take the LDS-tiled kernel. */
int mrk_hip_gemm_bf16(int device_id, const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k);
/* Bytes of f32 scratch with which the product of this shape is spread over the chip along K
 * (few output tiles, long K: a handful of rows against a weight matrix; up to 16 rows, and up to
 * 64 against a weight of at most 4096 columns, stream the weight once into partial sums instead
 * of running the tiled kernels); 0 when the shape has enough tiles by itself or one streaming
 * launch does.  mrk_hip_gemm_bf16 takes that scratch from the device allocator by
 * itself; a "gemm_bf16" builtin Program takes it as its fourth buffer. */
size_t mrk_hip_gemm_bf16_workspace_bytes(int64_t m, int64_t n, int64_t k, int64_t batch);
/* c[M,N] = a[M,K] * bt[N,K]^T: the product with the second operand as it is stored by a Linear
 * layer (weight [out_features, in_features], tensor/src/nn/linear.rs:9-14, 39-41), read in place
 * instead of through a transposed copy.  K a multiple of 8, 16-byte aligned operands.  More than
 * 64 rows with N a multiple of 8: the tiled kernels, the same products in the same order as
 * mrk_hip_gemm_bf16 on the transposed matrix, so the same bits (split-K shapes included; the
 * scratch comes from the device allocator).  Up to 64 rows (a decode step, a batch of them) with
 * any N: one streaming pass over the weight, no scratch: one or two rows with packed dot products
 * on the vector ALUs, 3 to 64 on the matrix pipes from 16-row blocks staged through LDS; f32
 * accumulation in another order than the tiled kernels' (results agree with them to the rounding
 * of the result), the same bits on every run.  More than 64 rows with N not a multiple of 8, or K
 * not a multiple of 8: INVALID_ARGUMENT.  Builtin Program kind "gemm_bf16_nt"
 * ({M, N, K[, batch[, workspace bytes]]}; the workspace is used by split-K shapes of more than 64
 * rows, which without one run the plain tiled kernel). */
int mrk_hip_gemm_bf16_nt(int device_id, const void* a, const void* bt, void* c, int64_t m, int64_t n, int64_t k);
/* The same two products on IEEE half precision (f16) operands and result, f32 accumulate: the f16
 * 16x16x32 entry of the reference's CDNA4 tensor-core table
 * (schedule/src/optimizer/renderer.rs:724-733, listed ahead of the bf16 one) as a hand-written
 * kernel; what Tensor::matmul computes for f16 inputs (tensor/src/matmul.rs:82-110 with the
 * tensor-core rewrite).  Same shapes, fallbacks and argument rules as the bf16 entry points; the
 * fused residual / gated epilogues are bf16 only.  Builtin Program kinds "gemm_f16", "gemm_f16_nt". */
int mrk_hip_gemm_f16(int device_id, const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k);
int mrk_hip_gemm_f16_nt(int device_id, const void* a, const void* bt, void* c, int64_t m, int64_t n, int64_t k);
/* Same with an explicit kernel variant (0 choose by shape, 2 any-shape kernel, 3 / 4 tiled kernel
 * with the 256-row / 128-row tile); tuning/tests. */
int mrk_hip_gemm_bf16_variant(int device_id, const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k,
                               int variant);

/* mrk_hip_gemm_bf16 for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same kernels and the same bits as mrk_hip_gemm_bf16, but the split-K partials go
 * to a fixed 32 MiB device array inside the library (resolved per device by
 * mrk_hip_device_create) instead of a block from the allocator, and the call performs no
 * allocation or free of any kind.  The device must have been created before
 * (INVALID_ARGUMENT otherwise: creating it allocates).  A shape whose partials would exceed
 * mrk_hip_gemm_bf16_noalloc_capacity() bytes is refused with INVALID_ARGUMENT and nothing is
 * launched.  All calls on one device share the array: calls that may overlap on one device
 * (different streams or threads without ordering between them) race; calls queued on the
 * device's own in-order stream, as this entry point does, do not. */
int mrk_hip_gemm_bf16_noalloc(int device_id, const void* a, const void* b, void* c, int64_t m, int64_t n, int64_t k);
size_t mrk_hip_gemm_bf16_noalloc_capacity(void);

/* c = bf16(float(bf16(a b)) + float(r)): the product above with a bf16 matrix r of c's shape added
 * in the kernel's epilogue - the bits of mrk_hip_gemm_bf16 followed by an elementwise add
 * (Tensor::matmul + try_add, tensor/src/matmul.rs:82-110), without the round trip of the product
 * through memory.  The product takes the route mrk_hip_gemm_bf16 takes and r joins where its result is
 * written: the tiled kernels' epilogue, the sum of the partial results of a product spread along K (scratch
 * from the device allocator), the streaming kernels for a handful of rows.  INVALID_ARGUMENT for shapes
 * outside the tiled kernels' (N or K not a multiple of 8, K = 0).  Builtin Program kinds
 * "gemm_bf16_residual" / "gemm_bf16_nt_residual" / "gemm_bf16_bias" / "gemm_bf16_nt_bias" take
 * {M, N, K[, batch[, workspace bytes]]} and buffers {c, a, b, r[, scratch]}. */
int mrk_hip_gemm_bf16_residual(int device_id, const void* a, const void* b, const void* r, void* c, int64_t m, int64_t n,
                               int64_t k);
/* y[M, N] = x[M, K] * w[N, K]^T + bias[N]: a Linear layer's forward pass on its parameters as it stores them
 * (tensor/src/nn/linear.rs:9-14 weight [out_features, in_features] and bias [out_features]; :39-41
 * x.linear(weight, bias) = x @ weight.T + bias), bf16 operands and result, f32 accumulation.  The bias is added in
 * the product kernel's epilogue: y = bf16(float(bf16(x w^T)) + float(bias)), the bits of the product followed by
 * the elementwise add.  bias may be NULL (the plain product, mrk_hip_gemm_bf16_nt).  Shapes as for
 * mrk_hip_gemm_bf16_nt; up to 64 rows run the streaming kernels, more rows the tiled kernels (a shape that the plain
 * product would spread along K runs unsplit here, on the workgroups its tiles make).  Builtin Program kinds
 * "gemm_bf16_nt_bias" and, for a weight stored [K, N], "gemm_bf16_bias" ({M, N, K[, batch]}, buffers {y, x, w, bias}). */
int mrk_hip_linear_bf16(int device_id, const void* x, const void* w, const void* bias, void* y, int64_t m, int64_t n, int64_t k);

/* Gated-MLP pair of products: c[M, F] = bf16(silu(float(bf16(a wg))) * float(bf16(a wu))) with
 * w = [wg | wu] stored side by side as one row-major [K, 2F] matrix: what
 * (x.matmul(w)[:, :F]).silu() * x.matmul(w)[:, F:] computes (Tensor::matmul, tensor/src/matmul.rs:82-110;
 * Tensor::silu / swish, tensor/src/activation.rs:309-318; the products rounded to bf16 first, then
 * x * sigmoid(x) * y in f32 and one rounding), with the gate applied in the product kernel's
 * epilogue so that the [M, 2F] product is never written.  The epilogue evaluates sigmoid(x) as
 * rcp(1 + exp2(-x log2 e)) with the hardware reciprocal (1 ulp in f32) where the separate
 * elementwise kernel divides exactly, so about 2 % of the results differ from the unfused
 * sequence by one bf16 ulp: fusing changes output bits within that bound.  No test of the
 * reference covers the gated product (parity unpinned by reference tests; pinned against
 * float64 and the oracle within 2e-2).  F and K multiples of 8, K > 0;
 * INVALID_ARGUMENT otherwise.  Builtin Program kind "gemm_bf16_swiglu", params {M, F, K},
 * buffers {c, a, w}. */
int mrk_hip_gemm_bf16_swiglu(int device_id, const void* a, const void* w, void* c, int64_t m, int64_t f, int64_t k);

/* A packed projection with the rotary embedding in its epilogue: for w [K, N] whose first `split`
 * columns are attention heads of 128 columns each (Wq | Wk of a fused QKV projection; split a
 * multiple of 256), c_rot[M, split] = apply_rotary_emb(bf16(a w)[:, :split] seen as heads, cos, sin)
 * in the reference's non-interleaved form (tensor/src/transformer.rs:32-69: x1 cos - x2 sin |
 * x1 sin + x2 cos over the two halves of a head), computed in f32 on the rounded product and
 * rounded once, as Tensor::matmul followed by apply_rotary_emb and a cast computes it; row r has
 * position r % seq, cos / sin are [seq, 64] f32.  The remaining columns go, unrotated, to
 * c_rest[M, N - split] (NULL when split == N).  The rotated product is never written and read
 * again in between.  K a multiple of 64, N of 8, cos / sin 32-byte aligned; INVALID_ARGUMENT
 * otherwise.  Builtin Program kind "gemm_bf16_rope", params {M, N, K, split, seq}, buffers
 * {c_rot, a, w, c_rest, cos, sin}; "gemm_bf16_nt_rope" is the same over a weight stored [N, K]
 * (a Linear layer's), with the same bits.  The reference holds no value test of this composition: parity
 * unpinned by reference tests, pinned against the oracle's product followed by its rotary stage. */
int mrk_hip_gemm_bf16_rope(int device_id, const void* a, const void* b, const void* cos, const void* sin, void* c_rot, void* c_rest,
                           int64_t m, int64_t n, int64_t k, int64_t split, int64_t seq);

/* Scaled dot-product attention forward in one kernel (online softmax, f32 scores and
 * statistics, P rounded to bf16 before the second product, bf16 output):
 * Tensor::scaled_dot_product_attention (tensor/src/transformer.rs:78-137) with is_causal as
 * given and no attn_mask / softcap.  q [B,H,Sq,D], k and v [B,H,Sk,D], o [B,H,Sq,D], row-major
 * bf16, D = 256, 128 or 64 (other head dims: INVALID_ARGUMENT here, the composed graph through the tensor
 * API), scale > 0 (the reference default is 1/sqrt(D), transformer.rs:90-91).
 * Causal rule of the reference: key j is visible to query i iff j <= i (transformer.rs:103-109).
 * Up to 32 queries without the causal rule against 256 keys and more (the decode step of a model that keeps
 * its keys and values: the same function of the reference, called with a short q) take a kernel that streams
 * K and V once and splits the key sequence over workgroups where (batch, head) pairs alone would not fill the
 * chip; the ranges' partial results (f32) are merged by a second kernel in a fixed order.  This call and the
 * strided one take that scratch from the device's allocator; a builtin Program gets it as a fifth buffer of
 * mrk_hip_flash_attn_workspace_bytes (0: the shape needs none), its size as one more parameter, and runs the
 * shape as one key range per pair without it. */
int mrk_hip_flash_attn_fwd_bf16(int device_id, const void* q, const void* k, const void* v, void* o, int64_t batch,
                                int64_t heads, int64_t sq, int64_t sk, int64_t d, float scale, int causal);
size_t mrk_hip_flash_attn_workspace_bytes(int64_t batch, int64_t heads, int64_t sq, int64_t sk, int64_t d, int causal);
/* The same over operands given as views of larger buffers, the way the reference's movement
 * ops hand them over without a copy (tensor/src/transformer.rs:78-137 takes any view; permute /
 * shrink / expand never move data there): strides = (batch, head, row) element strides of q, k,
 * v and o, 12 values; the D elements of a row are contiguous.  All strides are non-negative
 * multiples of 8 elements and the pointers 16-byte aligned; a zero batch or head stride of k / v
 * shares one set of keys between batches or heads; output rows, heads and batches must not
 * overlap.  (rows - 1) * row stride * 2 bytes must stay below 4 GiB per operand.
 * In a decode shape (above) heads whose k and v head strides are both zero are served by one pass over their
 * shared keys, up to 32 query rows (runs of consecutive heads) per pass (multi-query attention; grouped-query
 * attention with batch = batch x key heads and heads = query heads per key head). */
int mrk_hip_flash_attn_fwd_bf16_strided(int device_id, const void* q, const void* k, const void* v, void* o, int64_t batch,
                                        int64_t heads, int64_t sq, int64_t sk, int64_t d, float scale, int causal,
                                        const int64_t* strides);

/* The same attention with attn_mask and / or softcap inside the fused kernel
 * (Tensor::scaled_dot_product_attention, tensor/src/transformer.rs:112-132), in the reference's
 * order: scale, causal where(-inf), mask, softcap, softmax.  `strides` as in the call above, or
 * NULL for dense [batch, heads, rows, d] operands.  mask_kind 0: none (mask, mask_strides unused);
 * 1: Bool, one byte per element, nonzero = attend, false adds -inf (transformer.rs:114-121);
 * 2: additive bf16 (transformer.rs:122-124).  The mask is a [batch, heads, sq, sk] view with
 * contiguous keys; mask_strides holds its element strides per batch, head and query row (0 =
 * broadcast over that axis), each a multiple of 4, and sk must be a multiple of 4 when a mask is
 * given.  softcap 0: none; > 0: scores become softcap * tanh(score / softcap) AFTER the masks
 * (transformer.rs:128-132), so a masked score (causal ones included) becomes -softcap and still
 * takes part in the softmax, exactly as the reference's graph computes it; the kernel then visits
 * every key tile.  A row whose keys are all masked out (no softcap) is NaN, as softmax over -inf
 * only is.  Without mask and softcap this is mrk_hip_flash_attn_fwd_bf16_strided.
 * Without the causal rule a decode shape (up to 32 queries, 256 keys and more: a batch of sequences of different
 * lengths decoding under a key-padding mask [batch, 1, 1, sk]) takes the kernel that splits the key sequence, like
 * the unmasked call, mask and softcap inside it; key ranges without a visible key weigh nothing.
 * Builtin Program kind "flash_fwd_bf16_ext" (29 params, buffers {o, q, k, v, mask}; optionally a 30th, the bytes
 * of a scratch buffer that follows the mask: mrk_hip_flash_attn_workspace_bytes). */
int mrk_hip_flash_attn_fwd_bf16_ex(int device_id, const void* q, const void* k, const void* v, void* o, int64_t batch,
                                   int64_t heads, int64_t sq, int64_t sk, int64_t d, float scale, int causal,
                                   const int64_t* strides, const void* mask, int mask_kind, const int64_t* mask_strides,
                                   float softcap);

/* =====================================================================================
 * Synthetic inputs for benchmarks (no counterpart in the reference, whose tensor API has no
 * RNG, tensor/src/nn/mod.rs:304): counter-based SplitMix64 values written on the device.
 * dtype 0 = f32, 1 = bf16; mode 0 = uniform [a, b), mode 1 = normal(0, sigma = a).
 * ===================================================================================== */
int mrk_hip_fill(int device_id, void* out, size_t n, int dtype, int mode, uint64_t seed, uint64_t tensor_id, float a,
                 float b);
/* Streaming copy kernel over `bytes` (multiple of 16): the kernel of known traffic that
 * FETCH_SIZE / WRITE_SIZE counter readings are scaled against (no reference counterpart). */
int mrk_hip_copy_kernel(int device_id, const void* src, void* dst, size_t bytes);
/* MFMA-only calibration kernel (no reference counterpart): `workgroups` workgroups of four
 * waves, each wave issuing the matrix-instruction stream of one 256 x 256 x (64 * k_steps) bf16
 * GEMM tile from registers, without memory traffic: 2 * 256 * 256 * 64 * k_steps flops per
 * workgroup.  The rate it sustains is the ceiling GEMM kernels are compared with next to the
 * published peak.  random_operands: 0 = smooth small operand values, 1 = hashed values in
 * [-1.7, 1.7) as in a product of random matrices (the pipes' power draw, and with it the sustained
 * clock, depends on how much the operand bits toggle), 2 = the same hashed values rounded to IEEE
 * half precision and issued as the f16 instruction.  `scratch`: any device allocation of >= 4 bytes. */
int mrk_hip_mfma_ceiling(int device_id, void* scratch, int64_t workgroups, int64_t k_steps, int random_operands);
/* int32 values uniform over [0, high). */
int mrk_hip_fill_randint(int device_id, void* out, size_t n, uint64_t seed, uint64_t tensor_id, int high);

/* =====================================================================================
 * Events (hipEvent timing; stands where benchmark_kernel / execute_profiled use Instant,
 * runtime/src/benchmark.rs:64-91, runtime/src/execution_plan.rs:200-221)
 * ===================================================================================== */
int mrk_hip_event_create(int device_id, mrk_event** out);
int mrk_hip_event_record(mrk_event* e);
int mrk_hip_event_synchronize(mrk_event* e);
int mrk_hip_event_elapsed_ms(mrk_event* start, mrk_event* stop, float* ms);
void mrk_hip_event_destroy(mrk_event* e);

/* =====================================================================================
 * Lazy tensors: the caller side of the boundary.  Ops build a graph; realize splits it into
 * kernels (a reduce is a kernel boundary, movement ops become index arithmetic), obtains each
 * through the kernel cache and runs them as one execution plan
 * (tensor/src/realize.rs:83-127,299-357,937-1117).  With fusion on (the default) the composed
 * graphs of softmax / matmul / scaled_dot_product_attention run as the hand-written kernels
 * when dtype and layout qualify; with fusion off every op runs through generated kernels.
 * dtype and op tags are those of the linearized-kernel wire format (morok_amd/csrc/uop.h).
 * Every constructor returns a new handle the caller releases; handles are immutable.
 * ===================================================================================== */
typedef struct mrk_tensor mrk_tensor;
/* Tensor::from_raw_bytes / from_slice (tensor/src/data.rs:23-96): data is copied to the device
 * at creation; nbytes must equal numel * sizeof(dtype) (MRK_ERR_SIZE_MISMATCH otherwise). */
int mrk_hip_tensor_from_bytes(int device_id, const void* data, size_t nbytes, const int64_t* shape, size_t ndim,
                              int dtype, mrk_tensor** out);
/* Tensor::from_slice / from_raw_bytes without a device (data.rs:27-36,81-96): the tensor lives on
 * the CPU device, its bytes are copied into host memory owned by the tensor and no GPU is
 * touched.  This backend does not compute on the CPU: such a tensor can be read back, reshaped,
 * and moved with mrk_hip_tensor_to; realizing a computation over it is UNSUPPORTED_DEVICE. */
int mrk_hip_tensor_from_host_bytes(const void* data, size_t nbytes, const int64_t* shape, size_t ndim, int dtype,
                                   mrk_tensor** out);
/* Tensor::to (tensor/src/lib.rs:479-486).  device: "CPU", "HIP", "HIP:0", "AMD:0", "GPU"...  Same
 * device: a new handle to the same tensor.  Otherwise a lazy COPY: nothing moves until the result
 * (or something computed from it) is realized; the execution plan then carries a copy item that
 * runs in order with its kernels on every execute (tensor/src/realize.rs:1002-1011), so a prepared
 * plan re-uploads the host data each time it runs.  A copy to "CPU" must be the last step of a
 * realization.  Plans with copy items cannot be replayed through mrk_hip_plan_execute_graph. */
int mrk_hip_tensor_to(const mrk_tensor* t, const char* device, mrk_tensor** out);
/* Tensor::device (lib.rs:464-466): writes "CPU" or "HIP:<n>" (NUL-terminated) into out[cap]. */
int mrk_hip_tensor_device(const mrk_tensor* t, char* out, size_t cap);
/* Wraps an existing device buffer (shared, not copied). */
int mrk_hip_tensor_from_buffer(const mrk_buffer* b, const int64_t* shape, size_t ndim, int dtype, mrk_tensor** out);
int mrk_hip_tensor_const(int device_id, double value, int dtype, mrk_tensor** out);          /* lib.rs:432 */
int mrk_hip_tensor_full(int device_id, const int64_t* shape, size_t ndim, double value, int dtype,
                        mrk_tensor** out);                                                    /* lib.rs:251 */
void mrk_hip_tensor_release(mrk_tensor* t);
size_t mrk_hip_tensor_ndim(const mrk_tensor* t);
int mrk_hip_tensor_shape(const mrk_tensor* t, int64_t* shape_out, size_t capacity);
int mrk_hip_tensor_dtype(const mrk_tensor* t);
/* movement */
int mrk_hip_tensor_reshape(const mrk_tensor* t, const int64_t* shape, size_t ndim, mrk_tensor** out);
int mrk_hip_tensor_permute(const mrk_tensor* t, const int64_t* perm, size_t ndim, mrk_tensor** out);
int mrk_hip_tensor_transpose(const mrk_tensor* t, int64_t a, int64_t b, mrk_tensor** out);
int mrk_hip_tensor_expand(const mrk_tensor* t, const int64_t* shape, size_t ndim, mrk_tensor** out);
int mrk_hip_tensor_shrink(const mrk_tensor* t, const int64_t* begin, const int64_t* end, size_t ndim,
                          mrk_tensor** out);
int mrk_hip_tensor_contiguous(const mrk_tensor* t, mrk_tensor** out);                         /* lib.rs:548 */
int mrk_hip_tensor_cat(const mrk_tensor* const* parts, size_t nparts, int64_t axis, mrk_tensor** out);
/* elementwise, with broadcasting and dtype promotion (dtype/src/cast.rs:88) */
int mrk_hip_tensor_cast(const mrk_tensor* t, int dtype, mrk_tensor** out);                    /* lib.rs:495 */
int mrk_hip_tensor_unary(const mrk_tensor* t, int unary_op, mrk_tensor** out);
int mrk_hip_tensor_binary(const mrk_tensor* a, int binary_op, const mrk_tensor* b, mrk_tensor** out);
/* cond ? a : b */
int mrk_hip_tensor_where(const mrk_tensor* cond, const mrk_tensor* a, const mrk_tensor* b, mrk_tensor** out);
int mrk_hip_tensor_sigmoid(const mrk_tensor* t, mrk_tensor** out);                            /* activation.rs:42-52 */
int mrk_hip_tensor_silu(const mrk_tensor* t, mrk_tensor** out);                               /* activation.rs:309-318 */
/* reductions (reduce.rs:620-692); promote != 0 accumulates half types in f32 and small ints
 * in 32 bits (reduce.rs:101-117) */
int mrk_hip_tensor_reduce(const mrk_tensor* t, int reduce_op, const int64_t* axes, size_t naxes, int keepdim,
                          int promote, mrk_tensor** out);
int mrk_hip_tensor_mean(const mrk_tensor* t, const int64_t* axes, size_t naxes, int keepdim, mrk_tensor** out);
/* composite ops of the hot path */
/* 1-D x 1-D (scalar result), 1-D x 2-D, 2-D x 1-D, 2-D x 2-D, batched with broadcast batch axes */
int mrk_hip_tensor_matmul(const mrk_tensor* a, const mrk_tensor* b, mrk_tensor** out);        /* matmul.rs:82-110 */
/* matmul_with().dtype(): accumulate in and return `acc_dtype` (a dtype tag; -1 = the default rule) */
int mrk_hip_tensor_matmul_with(const mrk_tensor* a, const mrk_tensor* b, int acc_dtype, mrk_tensor** out);
/* alpha * op(A) @ op(B) + beta * C, c may be NULL (matmul.rs:112-135) */
int mrk_hip_tensor_gemm(const mrk_tensor* a, const mrk_tensor* b, float alpha, float beta, int trans_a, int trans_b,
                        const mrk_tensor* c, mrk_tensor** out);
/* x @ weight^T + bias, weight [out, in] (1-D weight: elementwise product), bias may be NULL (matmul.rs:160-190) */
int mrk_hip_tensor_linear(const mrk_tensor* x, const mrk_tensor* weight, const mrk_tensor* bias, int acc_dtype, mrk_tensor** out);
int mrk_hip_tensor_softmax(const mrk_tensor* t, int64_t axis, mrk_tensor** out);              /* activation.rs:90-101 */
int mrk_hip_tensor_log_softmax(const mrk_tensor* t, int64_t axis, mrk_tensor** out);          /* activation.rs:117-128 */
int mrk_hip_tensor_logsumexp(const mrk_tensor* t, int64_t axis, mrk_tensor** out);            /* activation.rs:143-157 */
int mrk_hip_tensor_rms_norm(const mrk_tensor* t, int64_t axis, double eps, mrk_tensor** out); /* nn/norm.rs:92-111 */
int mrk_hip_tensor_embedding(const mrk_tensor* weight, const mrk_tensor* indices, mrk_tensor** out); /* transformer.rs:12-25 */
int mrk_hip_tensor_rotary(const mrk_tensor* x, const mrk_tensor* cos, const mrk_tensor* sin, int interleaved,
                          mrk_tensor** out);                                                  /* transformer.rs:32-69 */
/* scale <= 0 selects 1/sqrt(head_dim) (transformer.rs:90-91) */
int mrk_hip_tensor_sdpa(const mrk_tensor* q, const mrk_tensor* k, const mrk_tensor* v, double scale, int is_causal,
                        mrk_tensor** out);                                                    /* transformer.rs:78-137 */
/* The same with the remaining options of the reference's builder: attn_mask (NULL for none; Bool:
 * true = attend, otherwise added to the scores; broadcastable to [.., Sq, Sk], transformer.rs:112-125)
 * and softcap (<= 0 for none; cap * tanh(scores / cap), transformer.rs:128-132).  With either of them
 * the composed graph runs; the fused attention kernel covers neither. */
int mrk_hip_tensor_sdpa_ex(const mrk_tensor* q, const mrk_tensor* k, const mrk_tensor* v, const mrk_tensor* attn_mask,
                           double scale, int is_causal, double softcap, mrk_tensor** out);
int mrk_hip_tensor_tanh(const mrk_tensor* t, mrk_tensor** out);                               /* activation.rs:64-74 */
/* realization (realize.rs:83-127) and extraction (data.rs:211-236) */
int mrk_hip_tensor_realize(const mrk_tensor* t);
/* Tensor::prepare (realize.rs:299-357): schedule + compile into an execution plan without
 * running it; the plan may be executed repeatedly (mrk_hip_plan_execute*), the tensor holds
 * valid data once it has run.  Release with mrk_hip_plan_release. */
int mrk_hip_tensor_prepare(const mrk_tensor* t, mrk_plan** out);
int mrk_hip_tensor_to_bytes(const mrk_tensor* t, void* dst, size_t nbytes);
/* Device buffer of a realized tensor (new handle sharing the allocation). */
int mrk_hip_tensor_buffer(const mrk_tensor* t, mrk_buffer** out);
/* Per-thread: hand-written fused kernels on/off; what the last realize on this thread ran
 * (Tensor::kernels(), tensor/src/lib.rs:213). */
void mrk_hip_tensor_set_fusion(int enabled);
size_t mrk_hip_tensor_last_kernel_count(void);
const char* mrk_hip_tensor_last_kernel_name(size_t i);
/* Rendered HIP C of that kernel; "" for a hand-written kernel (CachedKernel::code,
 * runtime/src/kernel_cache.rs:27-44). */
const char* mrk_hip_tensor_last_kernel_source(size_t i);
size_t mrk_hip_tensor_last_cached_count(void);
double mrk_hip_tensor_last_elapsed_ms(void);
/* Memory planner result of the last realize / prepare on this thread: intermediates that were
 * given an already used block, and the bytes that saved (tensor/src/memory_planner.rs:84-96).
 * Intermediates share blocks by liveness; MOROK_NO_MEMORY_PLANNER=1 turns that off. */
size_t mrk_hip_tensor_last_buffers_reused(void);
size_t mrk_hip_tensor_last_memory_saved(void);
/* Device bytes the intermediates of that plan occupy: the planner's pool after reuse, or one
 * block per intermediate with the planner off (MemoryPlannerResult::memory_planned,
 * tensor/src/memory_planner.rs:84-96). */
size_t mrk_hip_tensor_last_intermediate_bytes(void);
/* With MOROK_BEAM=<width> in the environment, realize / prepare searches the choices of every
 * generated elementwise and reduce kernel of at least 65536 elements of work as well
 * (tensor/src/realize.rs:1190-1242, schedule/src/optimizer/beam.rs:36-120): UPCAST then LOCAL for
 * elementwise kernels, GROUP / split then LOCAL for wave reductions; winners are cached on disk
 * (mrk_hip_beam_cache_*).  Candidates compiled and timed, and kernels answered by the cache,
 * in the last realize / prepare on this thread. */
size_t mrk_hip_tensor_last_beam_candidates(void);
size_t mrk_hip_tensor_last_beam_cache_hits(void);

#ifdef __cplusplus
}
#endif
#endif /* MOROK_HIP_H */
