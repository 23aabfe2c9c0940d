/*
 * C ABI of libanygpu_hip.so: the gfx950 (MI355X) kernels behind anyGPU's matmul, row softmax
 * and causal conv1d + SiLU entry points.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer into memory the caller owns; inputs are only read,
 *     outputs only written.  One kind of scratch exists: the GEMM entry points cut some products
 *     along K (few tiles and a deep K, few rows against a weight matrix) and pass the partial
 *     sums of such a launch through a workspace that belongs to the (device, stream) pair of the
 *     call; the same workspace takes the aligned copy of a GEMM operand that cannot be fetched
 *     in 16-byte pieces where it lies (an odd start or row pitch, a K or N that is no multiple
 *     of 8) and the partial results of the key-split blocks of the fused attention.  Who owns
 *     it is the caller's choice, see anygpu_set_workspace: by default the library
 *     allocates ANYGPU_WORKSPACE_BYTES (64 MiB) the first time an eager launch on a stream cuts a
 *     product and keeps them until anygpu_release_workspaces or the end of the process (operand
 *     copies that need more make that buffer grow, in steps of the same size, up to
 *     ANYGPU_WORKSPACE_MAX_BYTES: the old buffer is freed, which waits for the device); a caller
 *     that hands in its own workspace for a stream makes the library allocate nothing there.
 *     While a stream is being captured into a graph only a caller's workspace is used, never the
 *     library's: without one every captured product runs uncut and uncopied (a valid result,
 *     summed in another order than the cut one).  Nothing else allocates;
 *   - sizes, strides and leading dimensions are int64_t counts of ELEMENTS;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream, which is what the
 *     reference uses for every launch); calls are asynchronous with respect to the host;
 *   - the return value is 0 on success, a negative ANYGPU_ERR_* code when an argument is
 *     rejected before anything is launched, or a positive hipError_t value when the runtime
 *     refuses the launch.  The C++ `cu_*` wrappers turn any non-zero value into the
 *     reference's convention (log the error, exit(1); srcs/core/core.hpp:445-475).
 *   - fp16 values are IEEE binary16 stored as 2 bytes (what the reference calls float16,
 *     srcs/core/core.hpp:37).
 *
 * File and line citations name the interface of the reference (adamtiger/anyGPU) that each
 * entry point stands in for.
 */
#ifndef ANYGPU_HIP_H
#define ANYGPU_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ANYGPU_OK                 0
#define ANYGPU_ERR_NULL_POINTER  -1   /* a required buffer pointer is NULL */
#define ANYGPU_ERR_BAD_SHAPE     -2   /* a size is negative, or sizes are mutually inconsistent */
#define ANYGPU_ERR_BAD_STRIDE    -3   /* a stride / leading dimension is smaller than the extent it spans */
#define ANYGPU_ERR_UNSUPPORTED   -4   /* a value outside what the kernels implement (e.g. conv width > 4) */
#define ANYGPU_ERR_TOO_LARGE     -5   /* an extent exceeds what the launch geometry can index */
#define ANYGPU_ERR_SCRATCH_TOO_SMALL -6 /* the shape needs more scratch than the library's fixed device array holds */

/* Layout of the left-hand GEMM operand (fp32 entry point only). */
#define ANYGPU_A_ROW_MAJOR  0   /* A stored [M, K], element (r, l) at A[r * lda + l]  (reference layout) */
#define ANYGPU_A_COL_MAJOR  1   /* A stored [K, M], element (r, l) at A[l * lda + r]  (pre-transposed input) */

/* Layout of the right-hand GEMM operand. */
#define ANYGPU_B_ROW_MAJOR  0   /* B stored [K, N], element (l, c) at B[l * ldb + c]  (reference layout) */
#define ANYGPU_B_COL_MAJOR  1   /* B stored [N, K], element (l, c) at B[c * ldb + l]  ("weights as [out, in]") */

/* Library identification: ABI version (bumped on any signature change) and the code object target. */
int         anygpu_hip_abi_version(void);
const char* anygpu_hip_target(void);            /* "gfx950" */
const char* anygpu_hip_error_string(int code);  /* text for ANYGPU_ERR_* and for hipError_t values */

/*
 * The workspace of a (current device, stream) pair.  Who uses it: every anygpu_gemm_* entry point (partial sums of
 * products cut along K, aligned copies of operands that cannot be fetched where they lie) and the fused attention
 * anygpu_sdp_attention_fwd_f16 / _f32 (partial results of query blocks whose keys are walked in two halves).  The decode
 * attention takes its workspace as an argument instead.
 *
 * anygpu_set_workspace(stream, workspace, bytes) hands in `bytes` of device memory, 256-byte aligned, for the launches
 * made on `stream` from now on: the library then allocates nothing for that stream, plans its cuts along K within
 * `bytes` (too small for a shape: that shape runs uncut) and makes the same plan whether the stream is being captured
 * or not, so a captured product equals the eager one bit for bit.  The memory stays the caller's: it must outlive every
 * launch and every graph that used it, launches on the stream share it in stream order, and a graph that recorded
 * cut products owns it while it replays (no other work that uses the same workspace may overlap the replay, on
 * whatever stream).  workspace = NULL (bytes = 0) takes the registration back; a buffer the library had allocated for
 * the stream is freed by either call, so nothing on the stream may still be running.  The reference has no such
 * scratch: its ops layer allocates every buffer and its kernels none (srcs/core/tensor.hpp:56-57).
 *
 * anygpu_release_workspaces() frees every buffer the library itself allocated (on all devices) and forgets all
 * registrations; call it when no launch of this library is in flight.  A (device, stream) pair that needs a workspace
 * and has none from the caller takes ANYGPU_WORKSPACE_BYTES from the library at its first eager launch of that kind.
 * The library does not notice a stream being destroyed, so it bounds what it holds itself: at most
 * ANYGPU_MAX_OWN_WORKSPACES buffers; a further stream takes the place of the one used longest ago (whose buffer is
 * freed, which waits for the device).  A caller's registration is the caller's to take back: call
 * anygpu_set_workspace(stream, NULL, 0) before destroying a stream that has one, or a later stream that the runtime
 * gives the same handle would write into that memory.
 */
#define ANYGPU_WORKSPACE_BYTES (64 * 1024 * 1024)
#define ANYGPU_WORKSPACE_MAX_BYTES (1024 * 1024 * 1024)
#define ANYGPU_MAX_OWN_WORKSPACES 8

int anygpu_set_workspace(void* stream, void* workspace, int64_t bytes);
int anygpu_release_workspaces(void);

/*
 * C[M,N] = A[M,K] * B  with fp16 inputs, fp32 accumulation on the MFMA units, fp16 output.
 * Replaces opt2::cu_tensor_mm_f16 (srcs/kernels/cuda/mm_ops.cuh:60-63, the tensor_mm<float16, CUDA>
 * path of srcs/ops/mm_ops.hpp:62-65) and the cu_fast_mm_f16_* ladder
 * (srcs/kernels/cuda/fast_mm.cuh:70-98).  A is row-major with leading dimension lda >= K,
 * C row-major with ldc >= N, B as selected by b_layout (ldb >= N for row-major, >= K for
 * column-major).  Any M, N, K >= 0 are accepted; K a multiple of 64 with 16-byte aligned operand
 * rows takes the fastest kernels (whatever M, N and the alignment of C).
 */
int anygpu_gemm_f16_f32acc(const void* A, const void* B, void* C,
                           int64_t M, int64_t N, int64_t K,
                           int64_t lda, int64_t ldb, int64_t ldc,
                           int b_layout, void* stream);

/*
 * anygpu_gemm_f16_f32acc with the epilogues the models hang on their linear layers, applied to the fp32 sums before the
 * one rounding to fp16 (operands, layouts and leading dimensions as above):
 *   _bias      C = A * B + bias[N] (bias fp16)          tensor_gemm / tensor_linear with a bias (srcs/ops/mm_ops.hpp:102-171)
 *   _softcap   C = softcap * tanh((A * B) / softcap)    the Gemma2 output head, cu_tensor_gemma_linear_softcap_f32
 *                                                       (srcs/models/gemma2/gemma_linsoftcap.cu:11-33; weights [vocab, hidden]
 *                                                       = ANYGPU_B_COL_MAJOR), softcap > 0
 *   _gelu_mul  C = gelu_tanh(A * B_gate) (*) (A * B_up) the Gemma2 MLP up-projection (srcs/models/gemma2/gemma_mlp.hpp:85-90,
 *                                                       cu_mlp_gemma2_fused_upproj_f32_v1 / _v2); A is read once, B_gate and
 *                                                       B_up share b_layout and ldb
 * The reference runs these layers in float32 (anygpu_gemm_f32 and its _softcap / _gelu_mul forms); these are the same
 * operators for a model held in fp16.  K >= 1.  One exception to "before the one rounding": operands no tile kernel can
 * fetch and no copy is made of (K or N no multiple of 8 with fewer than 64 rows or without a workspace to copy into)
 * run the plain product, rounded to fp16, and a pass over it that adds the bias or applies the softcap and rounds
 * again; such results agree with the fused ones to the tolerance of the fp16 product (1e-2), not bit for bit.  _gelu_mul needs 16-byte aligned operand rows, K >= 64 and K a multiple
 * of 8 (with row-major B also N a multiple of 8) unless M <= 64; other shapes return ANYGPU_ERR_UNSUPPORTED.
 */
int anygpu_gemm_f16_f32acc_bias(const void* A, const void* B, const void* bias, void* C,
                                int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                int b_layout, void* stream);

int anygpu_gemm_f16_f32acc_softcap(const void* A, const void* B, void* C,
                                   int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                   int b_layout, float softcap, void* stream);

int anygpu_gemm_f16_f32acc_gelu_mul(const void* A, const void* B_gate, const void* B_up, void* C,
                                    int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                    int b_layout, void* stream);

/*
 * Measurement hook: anygpu_gemm_f16_f32acc through the kernel of the whole-tile case (M and N multiples of 256, K a
 * multiple of 64, B column-major, 16-byte aligned rows; anything else returns ANYGPU_ERR_UNSUPPORTED and launches
 * nothing), which additionally leaves four 64-bit counts per 256 x 256 tile in probe[4 * tile .. + 3] (device memory,
 * 4 * (M / 256) * (N / 256) values): the shader clock count at entry and at exit of that tile's main loop, then the
 * count of the constant 100 MHz clock at the same two points.  (exit - entry) of the first pair over 10 ns times
 * (exit - entry) of the second is the clock the part sustained under the kernel; K / 32 * 64 matrix instructions of 16
 * cycles over the first difference is the share of cycles its matrix cores were busy.  The result in C is that of
 * anygpu_gemm_f16_f32acc.  No counterpart in the reference.
 */
int anygpu_gemm_f16_f32acc_probe(const void* A, const void* B, void* C,
                                 int64_t M, int64_t N, int64_t K,
                                 int64_t lda, int64_t ldb, int64_t ldc,
                                 int b_layout, uint64_t* probe, void* stream);

/*
 * Measurement hook: a plain streaming kernel, dst[i] = src[i] over `bytes` bytes (a multiple of 16, both pointers
 * 16-byte aligned) in 16-byte accesses: blocks of `block` threads (256, 512 or 1024), `vectors_per_lane` (1, 2, 4 or 8)
 * accesses per lane all loaded before the first store, non-temporal loads / stores when the flags are non-zero, and,
 * with grid_limit > 0, at most that many blocks which walk the tiles in grid strides.  It states what read + write
 * bandwidth the box gives a streaming kernel in the geometry chosen, the yardstick for the memory-bound kernels of
 * this library (bytes read + bytes written = 2 * bytes).  No counterpart in the reference.
 */
int anygpu_stream_probe(const void* src, void* dst, int64_t bytes, int block, int vectors_per_lane,
                        int nt_load, int nt_store, int64_t grid_limit, void* stream);

/*
 * `batch` products of one shape in one launch: product i reads A + i * stride_a, B + i * stride_b and
 * writes C + i * stride_c (strides in elements, 0 shares an operand).  This is what the per-head host
 * loop of srcs/transformers/sdp.hpp:258-271 (one tensor_mm launch per head for Q K^T and again for P V)
 * collapses into.  batch <= 65535.
 */
int anygpu_gemm_f16_f32acc_batched(const void* A, const void* B, void* C,
                                   int64_t M, int64_t N, int64_t K,
                                   int64_t lda, int64_t ldb, int64_t ldc,
                                   int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                                   int b_layout, void* stream);

/*
 * C[M,N] = A[M,K] * B (+ bias[N] added to every row when bias != NULL), fp32 throughout, fp32 MFMA.
 * Replaces cu_tensor_mm_f32_opt0 and cu_tensor_gemm_f32_opt0 (srcs/kernels/cuda/mm_ops.cuh:10-25, the
 * tensor_mm / tensor_gemm <float32, CUDA> paths of srcs/ops/mm_ops.hpp:58-61,160-163) and the
 * cu_fast_mm_f32_* ladder (srcs/kernels/cuda/fast_mm.cuh:7-68), whose last rung takes the left operand
 * pre-transposed ([K, M], srcs/kernels/cuda/fast_mm_f32_v4.2.cu:190-199): a_layout selects that storage
 * (lda >= K for row-major A, >= M for column-major A).  Any shape.
 */
int anygpu_gemm_f32(const float* A, const float* B, const float* bias, float* C,
                    int64_t M, int64_t N, int64_t K,
                    int64_t lda, int64_t ldb, int64_t ldc,
                    int a_layout, int b_layout, void* stream);

/* Batched form of anygpu_gemm_f32 (no bias); see anygpu_gemm_f16_f32acc_batched. */
int anygpu_gemm_f32_batched(const float* A, const float* B, float* C,
                            int64_t M, int64_t N, int64_t K,
                            int64_t lda, int64_t ldb, int64_t ldc,
                            int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                            int a_layout, int b_layout, void* stream);

/*
 * C[M,N] = softcap * tanh((A[M,K] * B) / softcap), fp32.  The Gemma2 output head with its final logit
 * soft-capping in the GEMM's epilogue: replaces cu_tensor_gemma_linear_softcap_f32
 * (srcs/models/gemma2/gemma_linsoftcap.cu:3-60; the weight there is [vocab, hidden], i.e.
 * ANYGPU_B_COL_MAJOR with ldb = hidden, and M = batch * seq).  softcap must be > 0.  Any shape.
 */
int anygpu_gemm_f32_softcap(const float* A, const float* B, float* C,
                            int64_t M, int64_t N, int64_t K,
                            int64_t lda, int64_t ldb, int64_t ldc,
                            int b_layout, float softcap, void* stream);

/*
 * C[M,N] = gelu_tanh(A[M,K] * B_gate) (*) (A * B_up), (*) elementwise, fp32; gelu_tanh(z) =
 * z / 2 * (1 + tanh(sqrt(2 / pi) * (z + 0.044715 z^3))).  The Gemma2 MLP's gate and up projections with
 * the activation and the product in the epilogue of one kernel that reads A once: replaces
 * cu_mlp_gemma2_fused_upproj_f32_v1 / _v2 (srcs/kernels/cuda/mlp_gemma2_fused_upproj.cuh:6-16, weights
 * there are [hidden, intermediate] = ANYGPU_B_ROW_MAJOR) and the three-launch default path
 * tensor_gelu(tensor_linear(x, gate), true) * tensor_linear(x, up) of srcs/models/gemma2/gemma_mlp.hpp:85-90.
 * B_gate and B_up share b_layout and ldb.  Any shape.
 */
int anygpu_gemm_f32_gelu_mul(const float* A, const float* B_gate, const float* B_up, float* C,
                             int64_t M, int64_t N, int64_t K,
                             int64_t lda, int64_t ldb, int64_t ldc,
                             int b_layout, void* stream);

/*
 * Row softmax over the last axis of a [rows, cols] matrix, with the steps the attention caller
 * runs in front of it fused in, applied in this order to each element x[r, j]:
 *     s = x * alpha                                   (tensor_mul, srcs/ops/binary_ops.hpp:61-76)
 *     s = softcap * tanh(s / softcap)   if softcap != 0   (srcs/models/gemma2/gemma_linsoftcap.cu:3-9)
 *     masked if causal != 0 and j >  i + diag         (additive -inf above the diagonal)
 *     masked if window  > 0 and j <= i + diag - window (srcs/models/gemma2/gemma_slide_mask.cu:21)
 *     y = softmax over the row, masked elements are exactly 0  (srcs/ops/softmax_ops.hpp:15-82)
 * where i = r % q_len is the query index of row r (q_len <= 0 means i = r).  With alpha = 1,
 * softcap = 0, causal = 0, window = 0 this is cu_tensor_softmax_f32
 * (srcs/kernels/cuda/softmax_ops.cuh:6-8); the fused form replaces the mul -> add -> softmax
 * launches of srcs/transformers/sdp.hpp:267-269.  Rows are x_row_stride / y_row_stride elements
 * apart (>= cols), elements of a row are contiguous.  A row whose every element is masked is
 * written as zeros.  Internals are fp32 for both element types.
 */
int anygpu_softmax_rows_f16(const void* x, void* y,
                            int64_t rows, int64_t cols,
                            int64_t x_row_stride, int64_t y_row_stride,
                            int64_t q_len, int64_t diag,
                            float alpha, float softcap, int causal, int64_t window,
                            void* stream);

int anygpu_softmax_rows_f32(const float* x, float* y,
                            int64_t rows, int64_t cols,
                            int64_t x_row_stride, int64_t y_row_stride,
                            int64_t q_len, int64_t diag,
                            float alpha, float softcap, int causal, int64_t window,
                            void* stream);

/*
 * The same with the mask handed over as data, the way srcs/transformers/sdp.hpp:207-274 receives it:
 *     y[r, :] = softmax( softcap( x[r, :] * alpha ) + mask[r % q_len, :] )
 * mask is an additive [q_len, cols] matrix of the element type (0 = visible, -inf or the lowest finite
 * value = masked; masked outputs are exact zeros), rows mask_row_stride elements apart, shared by all
 * heads (q_len <= 0: one mask row per matrix row).  Every element of x and of the mask is read.
 */
int anygpu_softmax_rows_masked_f16(const void* x, const void* mask, void* y,
                                   int64_t rows, int64_t cols,
                                   int64_t x_row_stride, int64_t mask_row_stride, int64_t y_row_stride,
                                   int64_t q_len, float alpha, float softcap, void* stream);

int anygpu_softmax_rows_masked_f32(const float* x, const float* mask, float* y,
                                   int64_t rows, int64_t cols,
                                   int64_t x_row_stride, int64_t mask_row_stride, int64_t y_row_stride,
                                   int64_t q_len, float alpha, float softcap, void* stream);

/*
 * Scaled-dot-product attention, forward, in one kernel (the score matrix stays on chip):
 *     y[h] = softmax( mask( softcap( alpha * q[h] k[h / q_per_kv]^T ) ) ) v[h / q_per_kv]
 * q and y are [batch_heads, n_q, head_dim], k and v [batch_heads / q_per_kv, n_k, head_dim] (q_per_kv query
 * heads share one key / value head; 1 for ordinary multi-head attention), all fp16 and densely packed;
 * fp32 scores, sums and output accumulators.  The prologue steps and their order are those of
 * anygpu_softmax_rows_f16 with q_len = n_q and diag = n_k - n_q (the last query sees the last key):
 * causal != 0 hides key j from query i when j > i + diag, window > 0 also when j <= i + diag - window.
 * A query without a visible key gets zeros.  head_dim must be 64, 128 or 256, pointers 16-byte aligned.
 * Replaces the per-head loop of sdp_attention_masked_scaled_fwd (srcs/transformers/sdp.hpp:258-271: transpose,
 * tensor_mm, tensor_mul, tensor_add, tensor_softmax, tensor_mm per head) for masks that are index rules, and
 * is the half-precision counterpart of cu_flash_sdpa_fwd_d256_v1 (srcs/kernels/cuda/flash_sdpa_fwd.cuh:6-15,
 * fp32, head_dim 256, no mask).
 * Scratch: a launch with at least a block per compute unit whose longest query blocks would make the launch end
 * unevenly (long key ranges under a sliding window) walks the keys of those blocks in two halves and passes their
 * partial results through the stream's workspace (anygpu_set_workspace).  Without a caller's workspace the first such
 * eager launch on a stream makes the library allocate ANYGPU_WORKSPACE_BYTES; a stream under capture without a
 * caller's workspace runs whole blocks, whose sums are formed in another order (equal to the tolerance, not bit for
 * bit).  The same holds for anygpu_sdp_attention_fwd_f32.
 */
int anygpu_sdp_attention_fwd_f16(const void* q, const void* k, const void* v, void* y,
                                 int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                 float alpha, float softcap, int causal, int64_t window, void* stream);

/*
 * anygpu_sdp_attention_fwd_f16 in float32: operands, scores, sums and output are fp32 and both products run on the
 * fp32 matrix instruction, so results agree with the unfused float32 path to fp32 rounding.  Same arguments and
 * rules.  Replaces cu_flash_sdpa_fwd_d256_v1 (srcs/kernels/cuda/flash_sdpa_fwd.cuh:6-15: one head, head_dim 256,
 * no mask; here any number of heads, head_dim 64 / 128 / 256, the index-rule masks) and, for masks that are
 * index rules, the per-head loop of sdp_attention_masked_scaled_fwd (srcs/transformers/sdp.hpp:258-271).
 */
int anygpu_sdp_attention_fwd_f32(const float* q, const float* k, const float* v, float* y,
                                 int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                 float alpha, float softcap, int causal, int64_t window, void* stream);

/*
 * anygpu_sdp_attention_fwd_f32 with the mask as data: y = softmax(softcap(alpha q k^T) + mask) v, mask an additive
 * [n_q, n_k] float32 matrix (rows mask_stride >= n_k floats apart, any alignment) shared by all heads, -inf (or the
 * float lowest the reference's mask builders write) where a key is hidden; a query without a visible key gives zeros.
 * One kernel, no score matrix in memory: the fused counterpart of sdp_attention_masked_scaled_fwd
 * (srcs/transformers/sdp.hpp:207-274), whose mask argument is a tensor, in the precision the reference runs it in.
 * For masks of 4 M values and more, and for key ranges of 16384 keys and more whatever the queries (the environment variable
 * ANYGPU_ATTN_MASK_MAP_FROM, read at every call, replaces both by a number of mask values) a pass over the mask ahead of the kernel (once, not per head) notes which key tiles it hides from which
 * blocks of queries; those are neither loaded nor multiplied.  The note lives at the front of the stream's workspace;
 * under a capture without a caller's workspace there is none, every tile is loaded and the hidden ones cost no products.
 * The results are the same bit for bit either way, except where few query blocks go out in parts of their key range:
 * with the note the parts divide the visible tiles among them (a sliding window over a long cache leaves most equal
 * parts of the range empty), without it the range, and the sums are taken in another order.  With as many query blocks as
 * one to four rounds of the device's compute units the float32 form sends every block out in two such parts; for their
 * partial results an eager launch without a caller's workspace lets the library's own grow (as operand copies do, up to
 * 1 GiB; 192 MiB for 8 heads x 8192 queries x 256).  Callers whose mask is an index rule are still better served by
 * anygpu_sdp_attention_fwd_f32.  Same key splits through the stream's workspace as that entry point.
 */
int anygpu_sdp_attention_fwd_masked_f32(const float* q, const float* k, const float* v, const float* mask, float* y,
                                        int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                        int64_t mask_stride, float alpha, float softcap, void* stream);

/*
 * The same in half precision: q, k, v, y and the mask are halves (the mask 2-byte aligned, rows mask_stride >= n_k
 * halves apart), sums in fp32 on the matrix cores as in anygpu_sdp_attention_fwd_f16.  -inf hides a key; the half
 * lowest (-65504) is an ordinary, very negative bias, which hides a key wherever the row has a less negative one.
 * Hidden key tiles are left out as in the float32 form.
 */
int anygpu_sdp_attention_fwd_masked_f16(const void* q, const void* k, const void* v, const void* mask, void* y,
                                        int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                        int64_t mask_stride, float alpha, float softcap, void* stream);

/*
 * Decode form of anygpu_sdp_attention_fwd_f16 for generation steps: few queries per head, long key range.  Same
 * arguments, meaning and result; additionally q_per_kv * n_q <= 128 (the queries of the heads that share a key /
 * value head are processed together, sixteen rows to a wave, so k and v come from memory once per key / value head
 * and from the caches for the further groups of sixteen) and a workspace: the visible
 * key range is split over up to 256 waves per key / value head and group, whose partial results (running maximum, sum and
 * unnormalised accumulators, fp32) pass through `workspace` and are merged by a second kernel on the same stream.
 * anygpu_sdp_attention_decode_workspace_bytes returns the bytes needed for a shape (a negative error code for
 * arguments the decode form rejects); workspace must be 16-byte aligned device memory of at least that size and
 * may be reused by the next call on the same stream.  The reference has no decode kernel: its generation step
 * runs the per-head loop of srcs/transformers/sdp.hpp:258-271 against the cached keys.
 */
int64_t anygpu_sdp_attention_decode_workspace_bytes(int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k,
                                                    int64_t head_dim, int causal, int64_t window);

int anygpu_sdp_attention_decode_f16(const void* q, const void* k, const void* v, void* y,
                                    void* workspace, int64_t workspace_bytes,
                                    int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                    float alpha, float softcap, int causal, int64_t window, void* stream);

/*
 * anygpu_sdp_attention_decode_f16 without the workspace arguments, for callers that cannot allocate device memory
 * and have no workspace to hand in: code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation.  It has no counterpart in the reference.  The partial results pass through a fixed array of
 * ANYGPU_DECODE_STATIC_SCRATCH_BYTES of device memory that is part of the library's code object (every GPU the
 * library runs on holds its copy until the process ends); the call allocates and frees nothing.  Same kernels,
 * same split plan and bit-identical results to anygpu_sdp_attention_decode_f16.  A shape for which
 * anygpu_sdp_attention_decode_workspace_bytes exceeds the array is rejected with ANYGPU_ERR_SCRATCH_TOO_SMALL and
 * nothing is launched.  All calls on one GPU share the array: calls on one stream are ordered by the stream, calls
 * that overlap on different streams of one GPU race.  The first call on a device looks up the array's address
 * (hipGetSymbolAddress, which may load the code object): make it outside graph capture; a call with
 * batch_heads = 0 does that and nothing else.
 */
#define ANYGPU_DECODE_STATIC_SCRATCH_BYTES (8 * 1024 * 1024)

int anygpu_sdp_attention_decode_f16_static(const void* q, const void* k, const void* v, void* y,
                                           int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                           float alpha, float softcap, int causal, int64_t window, void* stream);

/*
 * The decode form in float32: anygpu_sdp_attention_decode_f16 with fp32 operands and the fp32 matrix instruction
 * (keys in tiles of 16, K and V straight from global memory into the MFMA operands).  Its workspace size comes
 * from anygpu_sdp_attention_decode_f32_workspace_bytes.  The reference has no counterpart: its generation loop
 * runs the per-head operator chain of sdp_attention_masked_scaled_fwd (srcs/transformers/sdp.hpp:258-271)
 * against the key / value cache (srcs/models/gemma2/gemma_kv_cache.hpp).
 */
int64_t anygpu_sdp_attention_decode_f32_workspace_bytes(int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k,
                                                        int64_t head_dim, int causal, int64_t window);

int anygpu_sdp_attention_decode_f32(const float* q, const float* k, const float* v, float* y,
                                    void* workspace, int64_t workspace_bytes,
                                    int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                    float alpha, float softcap, int causal, int64_t window, void* stream);

/*
 * Depthwise causal conv1d with bias and fused SiLU:
 *     y[b, d, s] = silu( bias[d] + sum_{k=0}^{width-1} w[d, k] * x[b, d, s + k - (width - 1)] ),
 * terms with a negative sequence index dropped (left zero padding of width-1).
 * x and y are [batch, chan, seqlen] with seqlen contiguous, w is [chan, width], bias [chan], all
 * densely packed and of the element type of the entry point; fp32 internals.  width must be 1..4,
 * the bound the reference asserts (srcs/fused/causal_conv1d.hpp:100).
 * Replaces cu_tensor_causal_conv1d_f32 (srcs/kernels/cuda/causal_conv1d.cuh:6-10).
 */
int anygpu_causal_conv1d_silu_f16(const void* x, const void* w, const void* bias, void* y,
                                  int64_t batch, int64_t chan, int64_t seqlen, int64_t width,
                                  void* stream);

int anygpu_causal_conv1d_silu_f32(const float* x, const float* w, const float* bias, float* y,
                                  int64_t batch, int64_t chan, int64_t seqlen, int64_t width,
                                  void* stream);

/*
 * One decode step of the same convolution: x is [batch, chan] (the new sample of every row), state is
 * [batch, chan, width - 1], the samples in front of it, oldest first, and is updated in place
 * (shifted by one, x appended); y[b, d] = silu(bias[d] + sum_{k < width-1} w[d, k] * state[b, d, k]
 * + w[d, width-1] * x[b, d]).  Starting from a zero state, seqlen calls reproduce
 * anygpu_causal_conv1d_silu_* column by column.  The reference has no decode path for its Mamba2
 * convolution (srcs/fused/causal_conv1d.hpp:24-117 is the whole-sequence form this step continues).
 * state may be NULL when width == 1.
 */
int anygpu_causal_conv1d_silu_update_f16(const void* x, void* state, const void* w, const void* bias, void* y,
                                         int64_t batch, int64_t chan, int64_t width, void* stream);

int anygpu_causal_conv1d_silu_update_f32(const float* x, float* state, const float* w, const float* bias, float* y,
                                         int64_t batch, int64_t chan, int64_t width, void* stream);

/*
 * Gated RMS normalisation over rows of `cols` contiguous elements:
 *     g = x * silu(z) (g = x when z == NULL);  y = g / sqrt(mean(g^2) + eps) * (w + (zero_centered ? 1 : 0))
 * x, z, y are [rows, cols], w is [cols]; fp32 internals.  One kernel for tensor_zamba_gated_rmsnorm
 * (srcs/models/zamba2/zamba_gated_rmsnorm.hpp:9-23: tensor_silu, tensor_mul, tensor_rms_norm, three
 * kernels there) and, with z == NULL, for cu_tensor_rms_norm_f32 / _v1 (srcs/kernels/cuda/norm_ops.cuh:14-37)
 * normalising over the last axis.
 */
int anygpu_gated_rmsnorm_f16(const void* x, const void* z, const void* w, void* y,
                             int64_t rows, int64_t cols, float eps, int zero_centered, void* stream);

int anygpu_gated_rmsnorm_f32(const float* x, const float* z, const float* w, float* y,
                             int64_t rows, int64_t cols, float eps, int zero_centered, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* ANYGPU_HIP_H */
