"""ctypes binding of libmorok_hip.so (the C ABI declared in include/morok_hip.h).

The library is loaded from the package directory; there is no fallback of any kind: if
the shared object is missing, importing this module raises.
"""
import ctypes as C
import os
import re

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmorok_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "morok_hip.h")


class MorokHipError(RuntimeError):
    """An entry point returned a non-zero status; `code` is one of the MRK_ERR_* values."""

    def __init__(self, code, message):
        super().__init__(f"[{code}] {message}")
        self.code = code
        self.message = message


if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
        "or `make -C morok_amd/csrc` (there is no CPU fallback)"
    )

lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)

c_size_p = C.POINTER(C.c_size_t)
c_void_pp = C.POINTER(C.c_void_p)
c_i64_p = C.POINTER(C.c_int64)

_SIGS = {
    "mrk_hip_last_error": (C.c_char_p, []),
    "mrk_hip_device_parse": (C.c_int, [C.c_char_p, C.POINTER(C.c_int)]),
    "mrk_hip_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "mrk_hip_device_create": (C.c_int, [C.c_int]),
    "mrk_hip_device_create_by_type": (C.c_int, [C.c_char_p, C.c_int]),
    "mrk_hip_name": (C.c_char_p, []),
    "mrk_hip_device_stream": (C.c_int, [C.c_int, c_void_pp]),
    "mrk_hip_alloc": (C.c_int, [C.c_int, C.c_size_t, C.c_int, C.c_int, c_void_pp]),
    "mrk_hip_free": (C.c_int, [C.c_int, C.c_void_p, C.c_size_t, C.c_int]),
    "mrk_hip_sync": (C.c_int, [C.c_int]),
    "mrk_hip_lru_cache_count": (C.c_int, [C.c_int, C.c_size_t, C.c_int, c_size_p]),
    "mrk_hip_lru_total_cached": (C.c_int, [C.c_int, c_size_p]),
    "mrk_hip_lru_clear": (C.c_int, [C.c_int]),
    "mrk_hip_copyin": (C.c_int, [C.c_int, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t]),
    "mrk_hip_copyout": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t]),
    "mrk_hip_copy_dd": (C.c_int, [C.c_int, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t]),
    "mrk_hip_buffer_new": (C.c_int, [C.c_int, C.c_size_t, C.c_int, C.c_int, c_void_pp]),
    "mrk_hip_buffer_ensure_allocated": (C.c_int, [C.c_void_p]),
    "mrk_hip_buffer_is_allocated": (C.c_int, [C.c_void_p]),
    "mrk_hip_buffer_view": (C.c_int, [C.c_void_p, C.c_size_t, C.c_size_t, c_void_pp]),
    "mrk_hip_buffer_copyin": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "mrk_hip_buffer_copyout": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "mrk_hip_buffer_copy_from": (C.c_int, [C.c_void_p, C.c_void_p]),
    "mrk_hip_buffer_raw_ptr": (C.c_int, [C.c_void_p, c_void_pp]),
    "mrk_hip_buffer_id": (C.c_uint64, [C.c_void_p]),
    "mrk_hip_buffer_size": (C.c_size_t, [C.c_void_p]),
    "mrk_hip_buffer_synchronize": (C.c_int, [C.c_void_p]),
    "mrk_hip_buffer_release": (None, [C.c_void_p]),
    "mrk_hip_render": (C.c_int, [C.c_int, C.c_char_p, C.c_size_t, C.c_char_p, c_void_pp]),
    "mrk_hip_program_spec_from_source": (
        C.c_int,
        [C.c_char_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_char_p), C.POINTER(C.c_uint8), C.c_size_t, c_size_p,
         c_size_p, c_void_pp],
    ),
    "mrk_hip_program_spec_name": (C.c_char_p, [C.c_void_p]),
    "mrk_hip_program_spec_src": (C.c_char_p, [C.c_void_p]),
    "mrk_hip_program_spec_buf_count": (C.c_size_t, [C.c_void_p]),
    "mrk_hip_program_spec_var_count": (C.c_size_t, [C.c_void_p]),
    "mrk_hip_program_spec_var_name": (C.c_char_p, [C.c_void_p, C.c_size_t]),
    "mrk_hip_program_spec_sizes": (C.c_int, [C.c_void_p, c_size_p, c_size_p]),
    "mrk_hip_program_spec_slots": (C.c_size_t, [C.c_void_p, C.c_int, c_size_p, C.c_size_t]),
    "mrk_hip_program_spec_release": (None, [C.c_void_p]),
    "mrk_hip_compile": (C.c_int, [C.c_void_p, c_void_pp]),
    "mrk_hip_cache_key": (C.c_char_p, []),
    "mrk_hip_compiled_spec_name": (C.c_char_p, [C.c_void_p]),
    "mrk_hip_compiled_spec_bytes": (C.c_size_t, [C.c_void_p, C.POINTER(C.POINTER(C.c_uint8))]),
    "mrk_hip_compiled_spec_has_src": (C.c_int, [C.c_void_p]),
    "mrk_hip_compiled_spec_release": (None, [C.c_void_p]),
    "mrk_hip_program_create": (C.c_int, [C.c_int, C.c_void_p, c_void_pp]),
    "mrk_hip_program_execute": (C.c_int, [C.c_void_p, c_void_pp, C.c_size_t, c_i64_p, C.c_size_t, c_size_p, c_size_p]),
    "mrk_hip_program_name": (C.c_char_p, [C.c_void_p]),
    "mrk_hip_program_destroy": (None, [C.c_void_p]),
    "mrk_hip_program_builtin": (C.c_int, [C.c_int, C.c_char_p, c_i64_p, C.c_size_t, c_void_pp]),
    "mrk_hip_kernel_get_or_compile": (C.c_int, [C.c_int, C.c_char_p, C.c_size_t, C.c_char_p, c_void_pp,
                                                C.POINTER(C.c_int)]),
    "mrk_hip_kernel_builtin": (C.c_int, [C.c_int, C.c_char_p, c_i64_p, C.c_size_t, c_void_pp]),
    "mrk_hip_kernel_entry_point": (C.c_char_p, [C.c_void_p]),
    "mrk_hip_kernel_code": (C.c_char_p, [C.c_void_p]),
    "mrk_hip_kernel_var_count": (C.c_size_t, [C.c_void_p]),
    "mrk_hip_kernel_var_name": (C.c_char_p, [C.c_void_p, C.c_size_t]),
    "mrk_hip_kernel_same": (C.c_int, [C.c_void_p, C.c_void_p]),
    "mrk_hip_kernel_release": (None, [C.c_void_p]),
    "mrk_hip_kernel_cache_size": (C.c_size_t, []),
    "mrk_hip_kernel_cache_clear": (None, []),
    "mrk_hip_plan_create": (C.c_int, [C.c_int, c_void_pp]),
    "mrk_hip_plan_add_buffer": (C.c_int, [C.c_void_p, C.c_void_p, c_size_p]),
    "mrk_hip_plan_add_kernel": (C.c_int, [C.c_void_p, C.c_void_p, c_size_p, C.c_size_t, c_i64_p, C.c_size_t]),
    "mrk_hip_plan_build": (C.c_int, [C.c_void_p]),
    "mrk_hip_plan_execute": (C.c_int, [C.c_void_p]),
    "mrk_hip_plan_execute_graph": (C.c_int, [C.c_void_p]),
    "mrk_hip_plan_execute_profiled": (C.c_int, [C.c_void_p, C.POINTER(C.c_double), C.c_size_t, c_size_p]),
    "mrk_hip_plan_execute_with_vars": (C.c_int, [C.c_void_p, C.POINTER(C.c_char_p), c_i64_p, C.c_size_t]),
    "mrk_hip_plan_kernel_count": (C.c_size_t, [C.c_void_p]),
    "mrk_hip_plan_kernel_name": (C.c_char_p, [C.c_void_p, C.c_size_t]),
    "mrk_hip_plan_release": (None, [C.c_void_p]),
    "mrk_hip_benchmark_kernel": (C.c_int, [C.c_int, C.c_void_p, c_void_pp, C.c_size_t, c_i64_p, C.c_size_t, c_size_p,
                                           c_size_p, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "mrk_hip_benchmark_kernel_with_cutoff": (C.c_int, [C.c_int, C.c_void_p, c_void_pp, C.c_size_t, c_i64_p, C.c_size_t,
                                                       c_size_p, c_size_p, C.c_int, C.c_int, C.c_double,
                                                       C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_int)]),
    "mrk_hip_signal_create": (C.c_int, [C.c_int, c_void_pp]),
    "mrk_hip_signal_set": (C.c_int, [C.c_void_p, C.c_uint64]),
    "mrk_hip_signal_value": (C.c_uint64, [C.c_void_p]),
    "mrk_hip_signal_wait": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint64]),
    "mrk_hip_signal_destroy": (None, [C.c_void_p]),
    "mrk_hip_sched_caps": (C.c_char_p, []),
    "mrk_hip_sched_tc_select": (C.c_int, [C.c_int, C.c_int, C.c_int]),
    "mrk_hip_sched_tc_info": (C.c_int, [C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "mrk_hip_sched_tc_operand_element": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int),
                                                   C.POINTER(C.c_int)]),
    "mrk_hip_sched_find_smallest_divisor": (C.c_size_t, [C.c_size_t]),
    "mrk_hip_sched_group_dims": (C.c_int, [c_size_p, C.c_size_t, c_size_p, C.c_size_t, c_size_p, C.c_size_t, c_size_p]),
    "mrk_hip_sched_split_dims": (C.c_int, [c_size_p, C.c_size_t, c_size_p, C.c_size_t, c_size_p, C.c_size_t, c_size_p]),
    "mrk_hip_sched_limit_dims": (C.c_int, [c_size_p, C.c_size_t, c_size_p, C.c_size_t, c_size_p, C.c_size_t, c_size_p]),
    "mrk_hip_sched_get_contraction": (C.c_int, [c_size_p, C.c_size_t, c_size_p, C.c_size_t, c_size_p]),
    "mrk_hip_sched_grouped_dims": (C.c_int, [c_size_p, C.c_size_t, c_size_p, C.c_size_t, C.c_int, c_size_p, C.c_size_t,
                                             c_size_p, c_size_p, c_size_p]),
    "mrk_hip_sched_build_matmul_f32": (C.c_int, [C.c_int64, C.c_int64, C.c_int64, C.POINTER(C.POINTER(C.c_uint8)),
                                                 c_size_p]),
    "mrk_hip_sched_build_wmma_matmul": (C.c_int, [C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int,
                                                  C.POINTER(C.POINTER(C.c_uint8)), c_size_p]),
    "mrk_hip_sched_build_wmma_matmul_lds": (C.c_int, [C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int,
                                                      C.POINTER(C.POINTER(C.c_uint8)), c_size_p]),
    "mrk_hip_sched_build_wmma_matmul_lds_opts": (C.c_int, [C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int,
                                                           C.POINTER(C.c_int), C.POINTER(C.POINTER(C.c_uint8)), c_size_p]),
    "mrk_hip_sched_free": (None, [C.c_void_p]),
    "mrk_hip_softmax_f32": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64]),
    "mrk_hip_softmax_f32_variant": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int]),
    "mrk_hip_gemm_bf16": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64]),
    "mrk_hip_gemm_bf16_nt": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64]),
    "mrk_hip_gemm_f16": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64]),
    "mrk_hip_gemm_f16_nt": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64]),
    "mrk_hip_gemm_bf16_swiglu": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64]),
    "mrk_hip_gemm_bf16_noalloc": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64]),
    "mrk_hip_gemm_bf16_noalloc_capacity": (C.c_size_t, []),
    "mrk_hip_gemm_bf16_workspace_bytes": (C.c_size_t, [C.c_int64, C.c_int64, C.c_int64, C.c_int64]),
    "mrk_hip_flash_attn_workspace_bytes": (C.c_size_t, [C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int]),
    "mrk_hip_gemm_bf16_variant": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64,
                                            C.c_int64, C.c_int]),
    "mrk_hip_gemm_bf16_residual": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64,
                                             C.c_int64]),
    "mrk_hip_linear_bf16": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64]),
    "mrk_hip_gemm_bf16_rope": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                         C.c_int64, C.c_int64, C.c_int64, C.c_int64]),
    "mrk_hip_flash_attn_fwd_bf16": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                              C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_float, C.c_int]),
    "mrk_hip_flash_attn_fwd_bf16_strided": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                                      C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_float, C.c_int,
                                                      C.POINTER(C.c_int64)]),
    "mrk_hip_flash_attn_fwd_bf16_ex": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                                 C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_float, C.c_int,
                                                 C.POINTER(C.c_int64), C.c_void_p, C.c_int, C.POINTER(C.c_int64), C.c_float]),
    "mrk_hip_fill": (C.c_int, [C.c_int, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_uint64, C.c_uint64, C.c_float,
                               C.c_float]),
    "mrk_hip_mfma_ceiling": (C.c_int, [C.c_int, C.c_void_p, C.c_int64, C.c_int64, C.c_int]),
    "mrk_hip_copy_kernel": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t]),
    "mrk_hip_fill_randint": (C.c_int, [C.c_int, C.c_void_p, C.c_size_t, C.c_uint64, C.c_uint64, C.c_int]),
    "mrk_hip_event_create": (C.c_int, [C.c_int, c_void_pp]),
    "mrk_hip_event_record": (C.c_int, [C.c_void_p]),
    "mrk_hip_event_synchronize": (C.c_int, [C.c_void_p]),
    "mrk_hip_event_elapsed_ms": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "mrk_hip_event_destroy": (None, [C.c_void_p]),
    "mrk_hip_sched_build_matmul_f32_opts": (C.c_int, [C.c_int64, C.c_int64, C.c_int64, C.POINTER(C.c_int), C.POINTER(C.POINTER(C.c_uint8)), c_size_p]),
    "mrk_hip_compile_and_time": (C.c_int, [C.c_int, C.c_void_p, C.c_size_t, C.c_char_p, c_void_pp, C.c_size_t, c_i64_p, C.c_size_t, C.c_int, C.c_int, C.POINTER(C.c_double)]),
    "mrk_hip_beam_cache_get": (C.c_int, [C.c_uint64, C.c_int, C.c_char_p, C.c_void_p, C.c_size_t, c_size_p]),
    "mrk_hip_beam_cache_put": (C.c_int, [C.c_uint64, C.c_int, C.c_char_p, C.c_void_p, C.c_size_t]),
    "mrk_hip_beam_search_matmul_f32": (C.c_int, [C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_double), C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "mrk_hip_beam_search_wmma_matmul": (C.c_int, [C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.POINTER(C.c_int),
                                                  C.POINTER(C.c_double), C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "mrk_hip_queue_create": (C.c_int, [C.c_int, C.c_int, c_void_pp]),
    "mrk_hip_queue_wait": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint64]),
    "mrk_hip_queue_signal": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint64]),
    "mrk_hip_queue_exec": (C.c_int, [C.c_void_p, C.c_void_p, c_void_pp, C.c_size_t, c_i64_p, C.c_size_t, c_size_p, c_size_p]),
    "mrk_hip_queue_copy": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "mrk_hip_queue_memory_barrier": (C.c_int, [C.c_void_p]),
    "mrk_hip_queue_submit": (C.c_int, [C.c_void_p, C.c_uint64]),
    "mrk_hip_queue_synchronize": (C.c_int, [C.c_void_p]),
    "mrk_hip_queue_pending": (C.c_size_t, [C.c_void_p]),
    "mrk_hip_queue_destroy": (None, [C.c_void_p]),
    # lazy tensors
    "mrk_hip_tensor_from_bytes": (C.c_int, [C.c_int, C.c_void_p, C.c_size_t, c_i64_p, C.c_size_t, C.c_int, c_void_pp]),
    "mrk_hip_tensor_from_host_bytes": (C.c_int, [C.c_void_p, C.c_size_t, c_i64_p, C.c_size_t, C.c_int, c_void_pp]),
    "mrk_hip_tensor_to": (C.c_int, [C.c_void_p, C.c_char_p, c_void_pp]),
    "mrk_hip_tensor_device": (C.c_int, [C.c_void_p, C.c_char_p, C.c_size_t]),
    "mrk_hip_tensor_from_buffer": (C.c_int, [C.c_void_p, c_i64_p, C.c_size_t, C.c_int, c_void_pp]),
    "mrk_hip_tensor_const": (C.c_int, [C.c_int, C.c_double, C.c_int, c_void_pp]),
    "mrk_hip_tensor_full": (C.c_int, [C.c_int, c_i64_p, C.c_size_t, C.c_double, C.c_int, c_void_pp]),
    "mrk_hip_tensor_release": (None, [C.c_void_p]),
    "mrk_hip_tensor_ndim": (C.c_size_t, [C.c_void_p]),
    "mrk_hip_tensor_shape": (C.c_int, [C.c_void_p, c_i64_p, C.c_size_t]),
    "mrk_hip_tensor_dtype": (C.c_int, [C.c_void_p]),
    "mrk_hip_tensor_reshape": (C.c_int, [C.c_void_p, c_i64_p, C.c_size_t, c_void_pp]),
    "mrk_hip_tensor_permute": (C.c_int, [C.c_void_p, c_i64_p, C.c_size_t, c_void_pp]),
    "mrk_hip_tensor_transpose": (C.c_int, [C.c_void_p, C.c_int64, C.c_int64, c_void_pp]),
    "mrk_hip_tensor_expand": (C.c_int, [C.c_void_p, c_i64_p, C.c_size_t, c_void_pp]),
    "mrk_hip_tensor_shrink": (C.c_int, [C.c_void_p, c_i64_p, c_i64_p, C.c_size_t, c_void_pp]),
    "mrk_hip_tensor_contiguous": (C.c_int, [C.c_void_p, c_void_pp]),
    "mrk_hip_tensor_cat": (C.c_int, [c_void_pp, C.c_size_t, C.c_int64, c_void_pp]),
    "mrk_hip_tensor_cast": (C.c_int, [C.c_void_p, C.c_int, c_void_pp]),
    "mrk_hip_tensor_unary": (C.c_int, [C.c_void_p, C.c_int, c_void_pp]),
    "mrk_hip_tensor_binary": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, c_void_pp]),
    "mrk_hip_tensor_where": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, c_void_pp]),
    "mrk_hip_tensor_sigmoid": (C.c_int, [C.c_void_p, c_void_pp]),
    "mrk_hip_tensor_silu": (C.c_int, [C.c_void_p, c_void_pp]),
    "mrk_hip_tensor_reduce": (C.c_int, [C.c_void_p, C.c_int, c_i64_p, C.c_size_t, C.c_int, C.c_int, c_void_pp]),
    "mrk_hip_tensor_mean": (C.c_int, [C.c_void_p, c_i64_p, C.c_size_t, C.c_int, c_void_pp]),
    "mrk_hip_tensor_matmul": (C.c_int, [C.c_void_p, C.c_void_p, c_void_pp]),
    "mrk_hip_tensor_matmul_with": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int, c_void_pp]),
    "mrk_hip_tensor_gemm": (C.c_int, [C.c_void_p, C.c_void_p, C.c_float, C.c_float, C.c_int, C.c_int, C.c_void_p, c_void_pp]),
    "mrk_hip_tensor_linear": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, c_void_pp]),
    "mrk_hip_tensor_softmax": (C.c_int, [C.c_void_p, C.c_int64, c_void_pp]),
    "mrk_hip_tensor_log_softmax": (C.c_int, [C.c_void_p, C.c_int64, c_void_pp]),
    "mrk_hip_tensor_logsumexp": (C.c_int, [C.c_void_p, C.c_int64, c_void_pp]),
    "mrk_hip_tensor_rms_norm": (C.c_int, [C.c_void_p, C.c_int64, C.c_double, c_void_pp]),
    "mrk_hip_tensor_embedding": (C.c_int, [C.c_void_p, C.c_void_p, c_void_pp]),
    "mrk_hip_tensor_rotary": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, c_void_pp]),
    "mrk_hip_tensor_sdpa": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_double, C.c_int, c_void_pp]),
    "mrk_hip_tensor_sdpa_ex": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_double, C.c_int, C.c_double,
                                         c_void_pp]),
    "mrk_hip_tensor_tanh": (C.c_int, [C.c_void_p, c_void_pp]),
    "mrk_hip_tensor_realize": (C.c_int, [C.c_void_p]),
    "mrk_hip_tensor_prepare": (C.c_int, [C.c_void_p, c_void_pp]),
    "mrk_hip_tensor_to_bytes": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "mrk_hip_tensor_buffer": (C.c_int, [C.c_void_p, c_void_pp]),
    "mrk_hip_tensor_set_fusion": (None, [C.c_int]),
    "mrk_hip_tensor_last_kernel_count": (C.c_size_t, []),
    "mrk_hip_tensor_last_kernel_name": (C.c_char_p, [C.c_size_t]),
    "mrk_hip_tensor_last_kernel_source": (C.c_char_p, [C.c_size_t]),
    "mrk_hip_tensor_last_cached_count": (C.c_size_t, []),
    "mrk_hip_tensor_last_elapsed_ms": (C.c_double, []),
    "mrk_hip_tensor_last_buffers_reused": (C.c_size_t, []),
    "mrk_hip_tensor_last_memory_saved": (C.c_size_t, []),
    "mrk_hip_tensor_last_intermediate_bytes": (C.c_size_t, []),
    "mrk_hip_tensor_last_beam_candidates": (C.c_size_t, []),
    "mrk_hip_tensor_last_beam_cache_hits": (C.c_size_t, []),
}


def declared_symbols(header_path=HEADER_PATH):
    """Names of every function declared in the public header."""
    text = open(header_path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mrk_\w+)\s*\(", text)))


def _bind():
    for name, (res, args) in _SIGS.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args


_bind()


def check(rc):
    """Raises MorokHipError for a non-zero status."""
    if rc != 0:
        raise MorokHipError(rc, lib.mrk_hip_last_error().decode("utf-8", "replace"))
    return rc
