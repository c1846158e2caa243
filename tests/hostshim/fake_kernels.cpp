// Recording stand-ins for the launchers of the hand-written gfx950 kernels
// (morok_amd/csrc/kernels/kernels.h).  TEST INFRASTRUCTURE ONLY: they compute nothing.
#include "kernels/kernels.h"

extern "C" void mrk_shim_note_launch(void* stream, const char* name);

namespace mrk {
int launch_softmax_f32(void* stream, const void*, void*, long, long, int) {
    mrk_shim_note_launch(stream, "softmax_f32");
    return 0;
}
size_t gemm_bf16_workspace_bytes(long, long, long, long) { return 0; }
size_t gemm_bf16_nt_workspace_bytes(long, long, long, long) { return 0; }
int launch_gemm_bf16(void* stream, const void*, const void*, void*, long, long, long, int, long, void*, size_t, bool b_transposed, bool f16) {
    mrk_shim_note_launch(stream, f16 ? (b_transposed ? "gemm_f16_nt" : "gemm_f16") : b_transposed ? "gemm_bf16_nt" : "gemm_bf16");
    return 0;
}
bool gemm_bf16_nt_supported(long M, long N, long K, long batch) {
    return M > 0 && N > 0 && K > 0 && batch > 0 && N % 8 == 0 && K % 8 == 0;
}
bool gemm_nt_skinny_supported(long M, long N, long K, long batch) { return M >= 1 && M <= 2 && N >= 1 && K >= 8 && K % 8 == 0 && batch >= 1; }
int launch_gemm_nt_skinny(void* stream, const void*, const void*, void*, long, long, long, long, bool f16) {
    mrk_shim_note_launch(stream, f16 ? "gemm_f16_nt" : "gemm_bf16_nt");
    return 0;
}
bool gemm_nt_rows_supported(long M, long N, long K, long batch) { return M >= 1 && M <= 64 && N >= 1 && K >= 8 && K % 8 == 0 && batch >= 1; }
int launch_gemm_nt_rows(void* stream, const void*, const void*, void*, long, long, long, long, bool f16) {
    mrk_shim_note_launch(stream, f16 ? "gemm_f16_nt" : "gemm_bf16_nt");
    return 0;
}
bool gemm_kn_skinny_plan(long, long, long, long, long*, long*) { return false; }
bool gemm_kn_rows_plan(long, long, long, long, long*, long*) { return false; }
int launch_gemm_kn_rows(void* stream, const void*, const void*, void*, void*, long, long, long, long, long, bool) {
    mrk_shim_note_launch(stream, "gemm_bf16");
    return 0;
}
int launch_gemm_kn_skinny(void* stream, const void*, const void*, void*, void*, long, long, long, long, long, bool) {
    mrk_shim_note_launch(stream, "gemm_bf16");
    return 0;
}
int gemm_bf16_static_workspace_init(int) { return 0; }
size_t gemm_bf16_static_workspace_capacity() { return size_t(32) << 20; }
int launch_gemm_bf16_static_ws(void* stream, int, const void*, const void*, void*, long, long, long) {
    mrk_shim_note_launch(stream, "gemm_bf16");
    return 0;
}
bool gemm_nt_swiglu_streamed(long M, long F, long K) { return M >= 1 && M <= 64 && F >= 1 && K >= 8 && K % 8 == 0; }
bool gemm_nt_bias_streamed(long M, long N, long K, long batch) { return batch == 1 && M >= 1 && M <= 64 && N >= 1 && K >= 8 && K % 8 == 0; }
bool gemm_bf16_bias_supported(long M, long N, long K, long batch, bool) { return M > 0 && N > 0 && K > 0 && batch > 0 && N % 8 == 0 && K % 8 == 0; }
bool gemm_bf16_bias_launchable(long M, long N, long K, long batch, bool t) { return gemm_bf16_bias_supported(M, N, K, batch, t); }
int launch_gemm_bf16_bias(void* stream, const void*, const void*, const void*, void*, long, long, long, long, bool b_transposed, void*, size_t) {
    mrk_shim_note_launch(stream, b_transposed ? "gemm_bf16_nt_bias" : "gemm_bf16_bias");
    return 0;
}
bool gemm_bf16_residual_supported(long M, long N, long K, long batch) {
    return M > 0 && N > 0 && K > 0 && batch > 0 && N % 8 == 0 && K % 8 == 0;
}
int launch_gemm_bf16_residual(void* stream, const void*, const void*, const void*, void*, long, long, long, long, bool b_transposed, bool r_is_row, void*, size_t) {
    if (r_is_row) {
        mrk_shim_note_launch(stream, b_transposed ? "gemm_bf16_nt_bias" : "gemm_bf16_bias");
        return 0;
    }
    mrk_shim_note_launch(stream, b_transposed ? "gemm_bf16_nt_residual" : "gemm_bf16_residual");
    return 0;
}
bool gemm_bf16_swiglu_supported(long M, long F, long K, bool) { return M > 0 && F > 0 && K > 0 && F % 8 == 0 && K % 8 == 0; }
int launch_gemm_bf16_swiglu(void* stream, const void*, const void*, void*, long, long, long, bool b_transposed) {
    mrk_shim_note_launch(stream, b_transposed ? "gemm_bf16_nt_swiglu" : "gemm_bf16_swiglu");
    return 0;
}
bool gemm_bf16_rope_supported(long M, long N, long K, long split, long seq) {
    return M > 0 && N > 0 && K > 0 && seq > 0 && K % 64 == 0 && N % 8 == 0 && split > 0 && split <= N && split % 256 == 0;
}
int launch_gemm_bf16_rope(void* stream, const void*, const void*, void*, void*, long, long, long, long, const void*, const void*, long, bool b_transposed) {
    mrk_shim_note_launch(stream, b_transposed ? "gemm_bf16_nt_rope" : "gemm_bf16_rope");
    return 0;
}
// a handful of queries against many keys with few (batch, head) pairs: scratch for a split key sequence
size_t flash_fwd_workspace_bytes(long BH, long Sq, long Sk, long D, int causal) {
    return !causal && Sq >= 1 && Sq <= 16 && Sk >= 1024 && BH >= 1 && BH <= 96 ? (size_t)2 * BH * 16 * (D + 2) * 4 : 0;
}
int launch_flash_fwd_bf16(void* stream, const void*, const void*, const void*, void*, long, long, long, long, float, int, void* ws, size_t) {
    mrk_shim_note_launch(stream, ws ? "flash_fwd_bf16_splitkv" : "flash_fwd_bf16");
    return 0;
}
int launch_flash_fwd_bf16_strided(void* stream, const void*, const void*, const void*, void*, long, long, long, long, long, float,
                                  int, const long*, void* ws, size_t) {
    mrk_shim_note_launch(stream, ws ? "flash_fwd_bf16_strided_splitkv" : "flash_fwd_bf16_strided");
    return 0;
}
int launch_flash_fwd_bf16_ext(void* stream, const void*, const void*, const void*, void*, long, long, long, long, long, float, int,
                              const long*, const void*, int mask_kind, const long*, float softcap, void* ws, size_t) {
    mrk_shim_note_launch(stream, mask_kind == 0 && !(softcap > 0.0f) ? "flash_fwd_bf16_strided" : ws ? "flash_fwd_bf16_ext_splitkv" : "flash_fwd_bf16_ext");
    return 0;
}
int launch_fill(void* stream, void*, size_t, int, int, unsigned long long, unsigned long long, float, float) {
    mrk_shim_note_launch(stream, "fill");
    return 0;
}
int launch_fill_randint(void* stream, void*, size_t, unsigned long long, unsigned long long, int) {
    mrk_shim_note_launch(stream, "fill_randint");
    return 0;
}
int launch_copy(void* stream, const void*, void*, size_t) {
    mrk_shim_note_launch(stream, "copy");
    return 0;
}
int launch_mfma_ceiling(void* stream, void*, long, long, int) {
    mrk_shim_note_launch(stream, "mfma_ceiling");
    return 0;
}
}  // namespace mrk
