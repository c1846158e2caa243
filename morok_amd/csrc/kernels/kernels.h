// Host-callable launchers of the hand-written gfx950 kernels.  Each returns the raw
// hipError_t (0 = success) of the launch; all work is queued on `stream`.
#pragma once
#include <cstddef>
#include <cstdint>

namespace mrk {

// y = softmax(x, axis=-1), x and y f32 [rows, cols] row-major.  variant 0 = default.
int launch_softmax_f32(void* stream, const void* x, void* y, long rows, long cols, int variant);


// C[M,N] = A[M,K] * B[K,N]; bf16 row-major operands, f32 accumulate, bf16 result.
// variant 0 = choose by shape, 2 = force the any-shape kernel, 3 / 4 = force the 256-row /
// 128-row tile of the tiled kernel (where the shape allows the tiled kernel at all), 5 = as 0.  batch > 1: that many
// independent products over matrices stored back to back (A [batch,M,K], B [batch,K,N],
// C [batch,M,N]), one launch.
// b_transposed: B is stored as B^T [N, K] (k contiguous: the layout of a Linear layer's weight;
// [batch, N, K] for batch > 1).  Same products in the same order, so the same bits as the [K, N]
// form (split-K included, given the workspace).  Up to 64 rows with K a multiple of 8 take the
// streaming kernels below (any N, no workspace), whose sums run in another order.  Shapes outside
// gemm_bf16_nt_supported (K not a multiple of 8; N not a multiple of 8 with more than 64 rows)
// are refused with hipErrorInvalidValue.
// f16: operands and result are IEEE half precision instead of bf16 (the same kernels around
// v_mfma_f32_16x16x32_f16; plain product only, the fused epilogues are bf16).
int launch_gemm_bf16(void* stream, const void* A, const void* B, void* C, long M, long N, long K, int variant,
                     long batch = 1, void* workspace = nullptr, size_t workspace_bytes = 0, bool b_transposed = false,
                     bool f16 = false);
bool gemm_bf16_nt_supported(long M, long N, long K, long batch);
// Scratch bytes launch_gemm_bf16 wants for the Bt[N, K] form: 0 for up to 64 rows (streamed), else the split-K
// plan's as for the [K, N] form.
size_t gemm_bf16_nt_workspace_bytes(long M, long N, long K, long batch);
// C[M, N] = A[M, K] @ Bt[N, K]^T for one or two rows (a decode step against a Linear layer's weight): one
// pass over the weight with packed dot products, no matrix pipe, no scratch memory.  K a multiple
// of 8, any N; bf16 or (f16) IEEE half operands and result, f32 accumulation.  Summation order
// differs from the tiled kernels', so results agree with them to rounding, not bit for bit.
bool gemm_nt_skinny_supported(long M, long N, long K, long batch);
int launch_gemm_nt_skinny(void* stream, const void* A, const void* Bt, void* C, long M, long N, long K, long batch, bool f16);
// The same for up to 64 rows on the matrix pipes: 16-row blocks of both operands go through LDS (direct
// copies, fragments read back), the waves of a workgroup split K and add their sums in a fixed order.  One
// launch, no scratch memory.  K a multiple of 8 (at most 2^23), any N.
bool gemm_nt_rows_supported(long M, long N, long K, long batch);
int launch_gemm_nt_rows(void* stream, const void* A, const void* Bt, void* C, long M, long N, long K, long batch, bool f16);
// The [K, N] form for one row (N <= 24576 and K multiples of 8, K >= 256, one product): the weight is
// streamed once into `splits` f32 partial results W[splits][M][N], which a second kernel adds up in a
// fixed order and rounds into C; gemm_kn_skinny_plan chooses the split and tells whether the shape is
// taken this way.  gemm_bf16_workspace_bytes reports splits * M * N * 4 for such shapes.
bool gemm_kn_skinny_plan(long M, long N, long K, long batch, long* splits, long* rows_per_group);
int launch_gemm_kn_skinny(void* stream, const void* A, const void* B, void* C, void* W, long M, long N, long K, long splits, long rows_per_group,
                          bool f16, const void* add = nullptr, bool add_is_row = false);
// The [K, N] form for up to 16 rows (up to 64 against a weight of at most 4096 columns and 8192 rows) on the matrix
// pipes (weight blocks through LDS and the transposing read), with the
// same split into f32 partial sums W[splits][M][N] and the same second kernel; with splits == 1 one launch writes C
// and W is not used.  N and K multiples of 8, K >= 256, one product.
bool gemm_kn_rows_plan(long M, long N, long K, long batch, long* splits, long* k_per_split);
int launch_gemm_kn_rows(void* stream, const void* A, const void* B, void* C, void* W, long M, long N, long K, long splits, long k_per_split,
                        bool f16, const void* add = nullptr, bool add_is_row = false);
// (`add`, for both: a matrix of C's shape or, add_is_row, one row [N] of C's type, added to the rounded result where the
// second kernel, or the single launch, writes it: the bits of the product followed by the elementwise add)
// c = bf16(float(bf16(a b)) + float(r)) with r of c's shape, or (r_is_row) one row [N] added to every row of c (a
// Linear layer's bias, tensor/src/nn/linear.rs:39-41): the same bits as the product followed by an elementwise add.  The
// product takes the route launch_gemm_bf16 would take (same workspace: gemm_bf16[_nt]_workspace_bytes) and r is added by
// whichever kernel writes the result: the tiled kernels' residual epilogue, the split-K reduction, the streaming kernels.
// gemm_bf16_residual_supported: N and K multiples of 8 (the tiled kernels' shapes); with the second operand stored
// [N, K] also every shape the streaming kernels take (gemm_bf16_bias_supported / _launchable tell, for either operand).
bool gemm_bf16_residual_supported(long M, long N, long K, long batch);
int launch_gemm_bf16_residual(void* stream, const void* a, const void* b, const void* r, void* c, long M, long N, long K, long batch,
                              bool b_transposed = false, bool r_is_row = false, void* workspace = nullptr, size_t workspace_bytes = 0);
bool gemm_bf16_bias_supported(long M, long N, long K, long batch, bool b_transposed);
bool gemm_bf16_bias_launchable(long M, long N, long K, long batch, bool b_transposed);
int launch_gemm_bf16_bias(void* stream, const void* a, const void* b, const void* bias, void* c, long M, long N, long K, long batch,
                          bool b_transposed, void* workspace = nullptr, size_t workspace_bytes = 0);
// y[M, N] = bf16(float(bf16(x wt^T)) + float(add)) with wt [N, K] as a Linear layer holds it and `add` either one row
// [N] (its bias) or a matrix [M, N] (a residual), for the shapes the streaming kernels take (up to 64 rows, K a
// multiple of 8, one product): added where the kernel writes its result.  Same bits as the product followed by the add.
// c[M, F] = silu(a gate) * (a up) over a weight [2 F, K] (gate rows first) with up to 64 rows of a, bf16: the gate applied where
// the matrix-pipe streaming kernel writes its result (the arithmetic of the generated elementwise kernel it replaces).
bool gemm_nt_swiglu_streamed(long M, long F, long K);
int launch_gemm_nt_swiglu_streamed(void* stream, const void* A, const void* Bt, void* C, long M, long F, long K);
bool gemm_nt_bias_streamed(long M, long N, long K, long batch);
int launch_gemm_nt_bias_streamed(void* stream, const void* A, const void* Bt, const void* add, void* C, long M, long N, long K, bool f16,
                                 bool add_is_row = true);
// C[M, F] = bf16(silu(float(bf16(A Wg))) * float(bf16(A Wu))) for W = [Wg | Wu] stored side by side as
// one [K, 2F] matrix: the gated-MLP pair of products with the gate applied in the product kernel's
// epilogue, so that the [M, 2F] product never reaches memory.  F and K multiples of 8.
// b_transposed: W is stored as [2F, K] (the rows of Wg^T, then the rows of Wu^T).
bool gemm_bf16_swiglu_supported(long M, long F, long K, bool b_transposed = false);
int launch_gemm_bf16_swiglu(void* stream, const void* a, const void* w, void* c, long M, long F, long K, bool b_transposed = false);
// A packed projection whose first `split` columns are attention heads of 128 columns (q | k of a
// fused QKV product, split a multiple of 256) with the rotary embedding applied in the product
// kernel's epilogue: c_rot [M, split] = rope(bf16(a b)[:, :split]) (non-interleaved halves, cos /
// sin [seq, 64] f32, 32-byte aligned, position = row % seq; f32 arithmetic on the rounded product,
// one rounding), c_rest [M, N - split] = bf16(a b)[:, split:] (may be null when split == N).
// K a multiple of 64, N of 8.
bool gemm_bf16_rope_supported(long M, long N, long K, long split, long seq);
int launch_gemm_bf16_rope(void* stream, const void* a, const void* b, void* c_rot, void* c_rest, long M, long N, long K, long split,
                          const void* cos, const void* sin, long seq, bool b_transposed = false);
// Bytes of f32 scratch with which launch_gemm_bf16 spreads the K loop of this shape over the
// chip (split-K: partial products per K range, added up in a fixed order by a second kernel);
// 0 when the shape has enough output tiles by itself.  Without the workspace the same shape
// runs unsplit.
size_t gemm_bf16_workspace_bytes(long M, long N, long K, long batch);
// The same product with the split-K partials in a file-scope device array instead of a
// caller's workspace, for callers that must not allocate.  gemm_bf16_static_workspace_init
// resolves the array's address on one device (that device current; once per device, at
// set-up); launch_gemm_bf16_static_ws launches nothing and returns hipErrorInvalidValue when
// the shape's partials exceed gemm_bf16_static_workspace_capacity(), hipErrorNotInitialized
// when the address has not been resolved for device_id.  Calls on one device share the array.
int gemm_bf16_static_workspace_init(int device_id);
size_t gemm_bf16_static_workspace_capacity();
int launch_gemm_bf16_static_ws(void* stream, int device_id, const void* A, const void* B, void* C, long M, long N, long K);

// The attention kernels form the byte offset of a row inside one (batch, head) in 32 bits:
// `rows` rows of `row_bytes` each (D elements of them used) must end below 4 GiB.
inline bool flash_fwd_rows_addressable(long rows, long row_bytes, long D) {
    return rows <= 0 || (rows - 1) * row_bytes + D * 2 <= 0xffffffffL;
}
// O = softmax(Q K^T * scale [causal]) V; Q [BH,Sq,D], K/V [BH,Sk,D], O [BH,Sq,D] bf16, D = 256, 128 or 64,
// scale > 0.  Causal: key j visible to query i iff j <= i.
// Up to 32 queries without the causal rule against 256 keys and more (a decode step over a key/value cache) take
// a kernel that also splits the key sequence over workgroups (flash_decode_plan tells how); with several key
// ranges their f32 partial results go through `workspace` (flash_fwd_workspace_bytes; 0 = one range), which a
// second kernel merges.  Without a workspace of that size such a shape runs in as many ranges as the workspace holds.
// Heads that share their keys and values (zero head strides of k and v: multi-query attention, or grouped-query
// attention with the groups as batches) are folded into one pair's query slots, as many consecutive heads as give at
// most 32 slots (a divisor of the head count), so that K and V are read once per such run instead of once per head.
bool flash_decode_plan(long BH, long Sq, long Sk, long D, int causal, long* splits, long* keys_per_split);
long flash_decode_slot_capacity(long slots);
size_t flash_fwd_workspace_bytes(long BH, long Sq, long Sk, long D, int causal);
int launch_flash_decode(void* stream, const void* q, const void* k, const void* v, void* o, long B, long H, long Sq, long Sk, long D,
                        float scale, const long* strides, long splits, long keys_per_split, void* W, const void* mask = nullptr,
                        int mask_kind = 0, const long* mask_strides = nullptr, float softcap = 0.0f, long group = 1);
int launch_flash_fwd_bf16(void* stream, const void* q, const void* k, const void* v, void* o, long BH, long Sq, long Sk,
                          long D, float scale, int causal, void* workspace = nullptr, size_t workspace_bytes = 0);
// The same kernel over operands given as views: strides holds (batch, head, row) element
// strides of q, k, v and o, in that order (12 values); the 128 elements of a row are
// contiguous.  Strides must be multiples of 8 elements and the pointers 16-byte aligned;
// zero batch / head strides broadcast an input.  Dense strides take the kernel above.
int launch_flash_fwd_bf16_strided(void* stream, const void* q, const void* k, const void* v, void* o, long B, long H, long Sq,
                                  long Sk, long D, float scale, int causal, const long* strides, void* workspace = nullptr,
                                  size_t workspace_bytes = 0);

// The same attention with an attn_mask and / or a softcap (transformer.rs:112-132), operands as
// views like the strided launcher.  mask_kind 0: none; 1: Bool, one byte per element, nonzero =
// attend; 2: additive bf16.  mask_strides: element strides of the mask per batch, head and query
// row (0 broadcasts; keys are contiguous), multiples of 4, and Sk a multiple of 4.  softcap 0:
// none; else scores become softcap * tanh(score / softcap) after masking, so masked scores
// (causal ones included) turn into -softcap and still take part, as in the reference.  A row
// whose keys are all masked out (no softcap) comes out as NaN, as the reference's softmax does.
// Without mask and softcap this is launch_flash_fwd_bf16_strided.
// Without the causal rule a decode shape (see flash_decode_plan) takes the split kernel here as well, mask and
// softcap inside it, with the same workspace.
int launch_flash_fwd_bf16_ext(void* stream, const void* q, const void* k, const void* v, void* o, long B, long H, long Sq, long Sk,
                              long D, float scale, int causal, const long* strides, const void* mask, int mask_kind,
                              const long* mask_strides, float softcap, void* workspace = nullptr, size_t workspace_bytes = 0);

// Synthetic benchmark inputs. dtype 0 = f32, 1 = bf16; mode 0 = uniform [a, b), 1 = normal(0, a).
int launch_fill(void* stream, void* out, size_t n, int dtype, int mode, unsigned long long seed,
                unsigned long long tensor_id, float a, float b);
int launch_fill_randint(void* stream, void* out, size_t n, unsigned long long seed, unsigned long long tensor_id,
                        int high);

// Streaming device-to-device copy kernel (bytes % 16 == 0): traffic-counter calibration.
int launch_copy(void* stream, const void* in, void* out, size_t bytes);


// MFMA-only calibration kernel: `workgroups` workgroups of four waves, each wave issuing
// k_steps x 128 v_mfma_f32_16x16x32_bf16 from registers (the instruction stream of one
// 256 x 256 x 64*k_steps GEMM tile without its memory traffic): 2 * 256 * 256 * 64 * k_steps
// flops per workgroup.  `out` (>= 4 bytes) is never written in practice.
// random_operands: 0 = smooth small operand values, 1 = hashed values in [-1.7, 1.7) like a product of
// random matrices (operand bit toggling costs power, and the sustained clock follows the power),
// 2 = the same hashed values rounded to IEEE half precision, issued as v_mfma_f32_16x16x32_f16.
int launch_mfma_ceiling(void* stream, void* out, long workgroups, long k_steps, int random_operands);

}  // namespace mrk
