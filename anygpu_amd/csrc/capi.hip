// extern "C" layer of libanygpu_hip.so: argument validation, then the kernel launchers.
// Nothing is launched when an argument is rejected.
#include "anygpu_hip.h"
#include "launch.hpp"
#include "gemm_band.hpp"
#include "gemm_epilogue.hpp"
#include "device_utils.hpp"

#include <atomic>
#include <climits>
#include <cmath>

// Scratch of anygpu_sdp_attention_decode_f16_static: the per-split partial results of the decode attention, for
// callers that can hand in no workspace.  Every GPU holds its own copy of the array from the moment the code
// object is loaded until the process ends.  In host code the name is only a handle for hipGetSymbolAddress.
static __device__ __align__(256) unsigned char scratch[ANYGPU_DECODE_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kAbiVersion = 1;
constexpr int64_t kMaxIndex32 = 0x7FFFFFFFLL;

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

int check_gemm(const void* A, const void* B, const void* C, int64_t M, int64_t N, int64_t K,
               int64_t lda, int64_t ldb, int64_t ldc, int a_layout, int b_layout)
{
	if (M < 0 || N < 0 || K < 0) return ANYGPU_ERR_BAD_SHAPE;
	if (a_layout != ANYGPU_A_ROW_MAJOR && a_layout != ANYGPU_A_COL_MAJOR) return ANYGPU_ERR_UNSUPPORTED;
	if (b_layout != ANYGPU_B_ROW_MAJOR && b_layout != ANYGPU_B_COL_MAJOR) return ANYGPU_ERR_UNSUPPORTED;
	if (M == 0 || N == 0) return ANYGPU_OK;
	if (C == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if (K > 0 && (A == nullptr || B == nullptr)) return ANYGPU_ERR_NULL_POINTER;
	if (lda < (a_layout == ANYGPU_A_ROW_MAJOR ? K : M) || ldc < N) return ANYGPU_ERR_BAD_STRIDE;
	if (ldb < (b_layout == ANYGPU_B_ROW_MAJOR ? N : K)) return ANYGPU_ERR_BAD_STRIDE;
	// the grids index 64- or 128-wide tiles with 16-bit y and 31-bit x block numbers
	if (M > 65535LL * 64 || N > kMaxIndex32 || K > kMaxIndex32) return ANYGPU_ERR_TOO_LARGE;
	return ANYGPU_OK;
}

int check_softmax(const void* x, const void* y, int64_t rows, int64_t cols, int64_t xs, int64_t ys, int64_t window)
{
	if (rows < 0 || cols < 0 || window < 0) return ANYGPU_ERR_BAD_SHAPE;
	if (rows == 0 || cols == 0) return ANYGPU_OK;
	if (x == nullptr || y == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if (xs < cols || ys < cols) return ANYGPU_ERR_BAD_STRIDE;
	if (rows > kMaxIndex32 || cols > kMaxIndex32) return ANYGPU_ERR_TOO_LARGE;
	return ANYGPU_OK;
}

int check_conv(const void* x, const void* w, const void* b, const void* y,
               int64_t batch, int64_t chan, int64_t seqlen, int64_t width)
{
	if (batch < 0 || chan < 0 || seqlen < 0) return ANYGPU_ERR_BAD_SHAPE;
	if (width < 1 || width > 4) return ANYGPU_ERR_UNSUPPORTED;
	if (batch == 0 || chan == 0 || seqlen == 0) return ANYGPU_OK;
	if (x == nullptr || w == nullptr || b == nullptr || y == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if (chan > kMaxIndex32 || seqlen > kMaxIndex32) return ANYGPU_ERR_TOO_LARGE;
	if (batch > kMaxIndex32 / chan) return ANYGPU_ERR_TOO_LARGE;                 // rows fit 31 bits
	if (batch * chan > (kMaxIndex32 * 256) / seqlen) return ANYGPU_ERR_TOO_LARGE;  // element grid fits 31 bits of blocks
	return ANYGPU_OK;
}

template <typename T>
int softmax_entry(const void* x, void* y, int64_t rows, int64_t cols, int64_t xs, int64_t ys,
                  int64_t q_len, int64_t diag, float alpha, float softcap, int causal, int64_t window, void* stream)
{
	const int rc = check_softmax(x, y, rows, cols, xs, ys, window);
	if (rc != ANYGPU_OK) return rc;
	if (q_len > kMaxIndex32) return ANYGPU_ERR_TOO_LARGE;
	// keep i + diag and i + diag - window + 1 inside 64-bit range whatever the caller passes
	if (diag > kMaxIndex32 || diag < -kMaxIndex32) return ANYGPU_ERR_TOO_LARGE;
	return (int)anygpu::launch_softmax_rows<T>(x, y, rows, cols, xs, ys, q_len, diag, alpha, softcap, causal,
	                                            window, nullptr, 0, as_stream(stream));
}

template <typename T>
int softmax_masked_entry(const void* x, const void* mask, void* y, int64_t rows, int64_t cols,
                         int64_t xs, int64_t ms, int64_t ys, int64_t q_len, float alpha, float softcap, void* stream)
{
	const int rc = check_softmax(x, y, rows, cols, xs, ys, 0);
	if (rc != ANYGPU_OK) return rc;
	if (rows == 0 || cols == 0) return ANYGPU_OK;
	if (mask == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if (ms < cols) return ANYGPU_ERR_BAD_STRIDE;
	if (q_len > kMaxIndex32) return ANYGPU_ERR_TOO_LARGE;
	return (int)anygpu::launch_softmax_rows<T>(x, y, rows, cols, xs, ys, q_len, 0, alpha, softcap, 0, 0,
	                                            mask, ms, as_stream(stream));
}

int check_batch(int64_t batch, int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t M, int64_t N, int64_t ldc)
{
	if (batch < 0 || stride_a < 0 || stride_b < 0 || stride_c < 0) return ANYGPU_ERR_BAD_SHAPE;
	if (batch > 65535) return ANYGPU_ERR_TOO_LARGE;
	// results of different products must not overlap
	if (batch > 1 && M > 0 && N > 0 && stride_c < (M - 1) * ldc + N) return ANYGPU_ERR_BAD_STRIDE;
	return ANYGPU_OK;
}

int check_attention_shape(int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim, int64_t window)
{
	if (batch_heads < 0 || n_q < 0 || n_k < 0 || head_dim < 0 || window < 0) return ANYGPU_ERR_BAD_SHAPE;
	if (q_per_kv < 1 || batch_heads % q_per_kv != 0) return ANYGPU_ERR_BAD_SHAPE;
	if (!anygpu::sdp_attention_fwd_f16_supports(head_dim)) return ANYGPU_ERR_UNSUPPORTED;
	if (batch_heads > 65535) return ANYGPU_ERR_TOO_LARGE;                        // (the decode form: one grid row per head)
	// the fused form's grid: one block per (head, block of 64 queries at least), plus padding of its block walk
	if (batch_heads * (n_q / 64 + 32) > kMaxIndex32 / 2) return ANYGPU_ERR_TOO_LARGE;
	// query and key indices, their sums and differences with the window stay inside 32 bits
	if (n_q > kMaxIndex32 / 4 || n_k > kMaxIndex32 / 4 || window > kMaxIndex32 / 4) return ANYGPU_ERR_TOO_LARGE;
	return ANYGPU_OK;
}

int check_attention(const void* q, const void* k, const void* v, const void* y, int64_t batch_heads, int64_t q_per_kv,
                    int64_t n_q, int64_t n_k, int64_t head_dim, float alpha, float softcap, int64_t window)
{
	const int rc = check_attention_shape(batch_heads, q_per_kv, n_q, n_k, head_dim, window);
	if (rc != ANYGPU_OK) return rc;
	if (!(softcap >= 0.0f) || !std::isfinite(softcap) || !std::isfinite(alpha)) return ANYGPU_ERR_UNSUPPORTED;
	if (batch_heads == 0 || n_q == 0) return ANYGPU_OK;
	if (q == nullptr || y == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if (n_k > 0 && (k == nullptr || v == nullptr)) return ANYGPU_ERR_NULL_POINTER;
	const uintptr_t bits = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
	                       reinterpret_cast<uintptr_t>(y);
	if (bits % 16 != 0) return ANYGPU_ERR_UNSUPPORTED;
	return ANYGPU_OK;
}

// Device address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
std::atomic<void*> scratch_ptr[kMaxDevices];

hipError_t scratch_of_current_device(void** ptr)
{
	int device = 0;
	hipError_t e = hipGetDevice(&device);
	if (e != hipSuccess) return e;
	if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
	void* p = scratch_ptr[device].load(std::memory_order_acquire);
	if (p == nullptr)
	{
		e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
		if (e != hipSuccess) return e;
		if (p == nullptr) return hipErrorInvalidSymbol;
		scratch_ptr[device].store(p, std::memory_order_release);     // (two threads racing here store the same address)
	}
	*ptr = p;
	return hipSuccess;
}

template <typename T>
int conv_update_entry(const void* x, void* state, const void* w, const void* b, void* y,
                      int64_t batch, int64_t chan, int64_t width, void* stream)
{
	if (batch < 0 || chan < 0) return ANYGPU_ERR_BAD_SHAPE;
	if (width < 1 || width > 4) return ANYGPU_ERR_UNSUPPORTED;
	if (batch == 0 || chan == 0) return ANYGPU_OK;
	if (x == nullptr || w == nullptr || b == nullptr || y == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if (state == nullptr && width > 1) return ANYGPU_ERR_NULL_POINTER;
	if (chan > kMaxIndex32 || batch > (kMaxIndex32 * 256) / chan) return ANYGPU_ERR_TOO_LARGE;   // grid of rows / 256 blocks
	return (int)anygpu::launch_causal_conv1d_silu_update<T>(x, state, w, b, y, batch, chan, (int)width, as_stream(stream));
}

template <typename T>
int gated_rmsnorm_entry(const void* x, const void* z, const void* w, void* y, int64_t rows, int64_t cols,
                        float eps, int zero_centered, void* stream)
{
	if (rows < 0 || cols < 0) return ANYGPU_ERR_BAD_SHAPE;
	if (rows == 0 || cols == 0) return ANYGPU_OK;
	if (x == nullptr || w == nullptr || y == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if (!(eps >= 0.0f)) return ANYGPU_ERR_UNSUPPORTED;
	if (rows > kMaxIndex32 || cols > kMaxIndex32) return ANYGPU_ERR_TOO_LARGE;                 // one block per row
	return (int)anygpu::launch_gated_rmsnorm<T>(x, z, w, y, rows, cols, eps, zero_centered, as_stream(stream));
}

template <typename T>
int conv_entry(const void* x, const void* w, const void* b, void* y,
               int64_t batch, int64_t chan, int64_t seqlen, int64_t width, void* stream)
{
	const int rc = check_conv(x, w, b, y, batch, chan, seqlen, width);
	if (rc != ANYGPU_OK) return rc;
	return (int)anygpu::launch_causal_conv1d_silu<T>(x, w, b, y, batch, chan, seqlen, (int)width, as_stream(stream));
}

}  // namespace

extern "C" {

#define ANYGPU_EXPORT __attribute__((visibility("default")))

ANYGPU_EXPORT int anygpu_hip_abi_version(void) { return kAbiVersion; }

ANYGPU_EXPORT const char* anygpu_hip_target(void) { return "gfx950"; }

ANYGPU_EXPORT const char* anygpu_hip_error_string(int code)
{
	switch (code)
	{
	case ANYGPU_OK: return "success";
	case ANYGPU_ERR_NULL_POINTER: return "a required buffer pointer is NULL";
	case ANYGPU_ERR_BAD_SHAPE: return "negative or inconsistent sizes";
	case ANYGPU_ERR_BAD_STRIDE: return "a stride or leading dimension is smaller than the extent it spans";
	case ANYGPU_ERR_UNSUPPORTED: return "argument value outside what the kernels implement";
	case ANYGPU_ERR_TOO_LARGE: return "an extent exceeds what the launch geometry can index";
	case ANYGPU_ERR_SCRATCH_TOO_SMALL: return "the shape needs more scratch than the library's fixed device array holds";
	default: break;
	}
	if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
	return "unknown anygpu error code";
}

ANYGPU_EXPORT int anygpu_set_workspace(void* stream, void* workspace, int64_t bytes)
{
	if (bytes < 0) return ANYGPU_ERR_BAD_SHAPE;
	if (workspace == nullptr && bytes > 0) return ANYGPU_ERR_NULL_POINTER;
	if (reinterpret_cast<uintptr_t>(workspace) % 256 != 0) return ANYGPU_ERR_UNSUPPORTED;
	return anygpu::band::workspace_set(as_stream(stream), workspace, (size_t)bytes);
}

ANYGPU_EXPORT int anygpu_release_workspaces(void)
{
	return (int)anygpu::band::workspace_release_all();
}

ANYGPU_EXPORT int anygpu_gemm_f16_f32acc(const void* A, const void* B, void* C,
                                         int64_t M, int64_t N, int64_t K,
                                         int64_t lda, int64_t ldb, int64_t ldc,
                                         int b_layout, void* stream)
{
	const int rc = check_gemm(A, B, C, M, N, K, lda, ldb, ldc, ANYGPU_A_ROW_MAJOR, b_layout);
	if (rc != ANYGPU_OK) return rc;
	return (int)anygpu::launch_gemm_f16(A, B, C, M, N, K, lda, ldb, ldc, 0, 0, 0, 1, b_layout, as_stream(stream));
}

namespace {

int gemm_f16_epilogue_entry(const void* A, const void* B, const void* B2, const void* bias, void* C,
                            int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                            int b_layout, int epilogue, float ep_param, void* stream)
{
	const int rc = check_gemm(A, B, C, M, N, K, lda, ldb, ldc, ANYGPU_A_ROW_MAJOR, b_layout);
	if (rc != ANYGPU_OK) return rc;
	if (M == 0 || N == 0) return ANYGPU_OK;
	if (K == 0) return ANYGPU_ERR_UNSUPPORTED;            // (an empty sum with an epilogue: not a case any caller has)
	bool supported = true;
	const hipError_t err = anygpu::launch_gemm_f16_epilogue(A, B, B2, bias, C, M, N, K, lda, ldb, ldc, b_layout, epilogue, ep_param,
	                                                        as_stream(stream), &supported);
	if (!supported) return ANYGPU_ERR_UNSUPPORTED;
	return (int)err;
}

}  // namespace

ANYGPU_EXPORT int anygpu_gemm_f16_f32acc_bias(const void* A, const void* B, const void* bias, void* C,
                                              int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                              int b_layout, void* stream)
{
	if (bias == nullptr && M > 0 && N > 0) return ANYGPU_ERR_NULL_POINTER;
	return gemm_f16_epilogue_entry(A, B, nullptr, bias, C, M, N, K, lda, ldb, ldc, b_layout, anygpu::kEpiBias, 0.0f, stream);
}

ANYGPU_EXPORT int anygpu_gemm_f16_f32acc_softcap(const void* A, const void* B, void* C,
                                                 int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                                 int b_layout, float softcap, void* stream)
{
	if (!(softcap > 0.0f) || !std::isfinite(softcap)) return ANYGPU_ERR_UNSUPPORTED;
	return gemm_f16_epilogue_entry(A, B, nullptr, nullptr, C, M, N, K, lda, ldb, ldc, b_layout, anygpu::kEpiSoftcap, softcap, stream);
}

ANYGPU_EXPORT int anygpu_gemm_f16_f32acc_gelu_mul(const void* A, const void* B_gate, const void* B_up, void* C,
                                                  int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                                  int b_layout, void* stream)
{
	if (B_up == nullptr && M > 0 && N > 0 && K > 0) return ANYGPU_ERR_NULL_POINTER;
	return gemm_f16_epilogue_entry(A, B_gate, B_up, nullptr, C, M, N, K, lda, ldb, ldc, b_layout, anygpu::kEpiGeluMul, 0.0f, stream);
}

ANYGPU_EXPORT int anygpu_gemm_f16_f32acc_probe(const void* A, const void* B, void* C,
                                               int64_t M, int64_t N, int64_t K,
                                               int64_t lda, int64_t ldb, int64_t ldc,
                                               int b_layout, uint64_t* probe, void* stream)
{
	const int rc = check_gemm(A, B, C, M, N, K, lda, ldb, ldc, ANYGPU_A_ROW_MAJOR, b_layout);
	if (rc != ANYGPU_OK) return rc;
	if (probe == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if (!anygpu::gemm_f16_probe_applies(A, B, C, M, N, K, lda, ldb, ldc, b_layout)) return ANYGPU_ERR_UNSUPPORTED;
	return (int)anygpu::launch_gemm_f16_probe(A, B, C, M, N, K, lda, ldb, ldc, reinterpret_cast<unsigned long long*>(probe), as_stream(stream));
}

ANYGPU_EXPORT int anygpu_stream_probe(const void* src, void* dst, int64_t bytes, int block, int vectors_per_lane,
                                      int nt_load, int nt_store, int64_t grid_limit, void* stream)
{
	if (bytes < 0 || bytes % 16 != 0 || grid_limit < 0) return ANYGPU_ERR_BAD_SHAPE;
	if (block != 256 && block != 512 && block != 1024) return ANYGPU_ERR_UNSUPPORTED;
	if (vectors_per_lane != 1 && vectors_per_lane != 2 && vectors_per_lane != 4 && vectors_per_lane != 8) return ANYGPU_ERR_UNSUPPORTED;
	if (bytes == 0) return ANYGPU_OK;
	if (src == nullptr || dst == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) return ANYGPU_ERR_UNSUPPORTED;
	const int64_t nvec = bytes / 16;
	if (nvec / ((int64_t)block * vectors_per_lane) >= kMaxIndex32) return ANYGPU_ERR_TOO_LARGE;
	return (int)anygpu::launch_stream_probe(src, dst, nvec, block, vectors_per_lane, nt_load != 0, nt_store != 0, grid_limit,
	                                        as_stream(stream));
}

ANYGPU_EXPORT int anygpu_gemm_f16_f32acc_batched(const void* A, const void* B, void* C,
                                                 int64_t M, int64_t N, int64_t K,
                                                 int64_t lda, int64_t ldb, int64_t ldc,
                                                 int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                                                 int b_layout, void* stream)
{
	int rc = check_gemm(A, B, C, M, N, K, lda, ldb, ldc, ANYGPU_A_ROW_MAJOR, b_layout);
	if (rc == ANYGPU_OK) rc = check_batch(batch, stride_a, stride_b, stride_c, M, N, ldc);
	if (rc != ANYGPU_OK) return rc;
	return (int)anygpu::launch_gemm_f16(A, B, C, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, batch,
	                                    b_layout, as_stream(stream));
}

ANYGPU_EXPORT int anygpu_gemm_f32(const float* A, const float* B, const float* bias, float* C,
                                  int64_t M, int64_t N, int64_t K,
                                  int64_t lda, int64_t ldb, int64_t ldc,
                                  int a_layout, int b_layout, void* stream)
{
	const int rc = check_gemm(A, B, C, M, N, K, lda, ldb, ldc, a_layout, b_layout);
	if (rc != ANYGPU_OK) return rc;
	return (int)anygpu::launch_gemm_f32(A, B, bias, C, M, N, K, lda, ldb, ldc, 0, 0, 0, 1, a_layout, b_layout,
	                                    as_stream(stream));
}

ANYGPU_EXPORT int anygpu_gemm_f32_batched(const float* A, const float* B, float* C,
                                          int64_t M, int64_t N, int64_t K,
                                          int64_t lda, int64_t ldb, int64_t ldc,
                                          int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                                          int a_layout, int b_layout, void* stream)
{
	int rc = check_gemm(A, B, C, M, N, K, lda, ldb, ldc, a_layout, b_layout);
	if (rc == ANYGPU_OK) rc = check_batch(batch, stride_a, stride_b, stride_c, M, N, ldc);
	if (rc != ANYGPU_OK) return rc;
	return (int)anygpu::launch_gemm_f32(A, B, nullptr, C, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, batch,
	                                    a_layout, b_layout, as_stream(stream));
}

ANYGPU_EXPORT int anygpu_gemm_f32_softcap(const float* A, const float* B, float* C,
                                          int64_t M, int64_t N, int64_t K,
                                          int64_t lda, int64_t ldb, int64_t ldc,
                                          int b_layout, float softcap, void* stream)
{
	const int rc = check_gemm(A, B, C, M, N, K, lda, ldb, ldc, ANYGPU_A_ROW_MAJOR, b_layout);
	if (rc != ANYGPU_OK) return rc;
	if (!(softcap > 0.0f) || !std::isfinite(softcap)) return ANYGPU_ERR_UNSUPPORTED;
	return (int)anygpu::launch_gemm_f32_softcap(A, B, C, M, N, K, lda, ldb, ldc, b_layout, softcap, as_stream(stream));
}

ANYGPU_EXPORT int anygpu_gemm_f32_gelu_mul(const float* A, const float* B_gate, const float* B_up, float* C,
                                           int64_t M, int64_t N, int64_t K,
                                           int64_t lda, int64_t ldb, int64_t ldc,
                                           int b_layout, void* stream)
{
	const int rc = check_gemm(A, B_gate, C, M, N, K, lda, ldb, ldc, ANYGPU_A_ROW_MAJOR, b_layout);
	if (rc != ANYGPU_OK) return rc;
	if (B_up == nullptr && M > 0 && N > 0 && K > 0) return ANYGPU_ERR_NULL_POINTER;
	return (int)anygpu::launch_gemm_f32_gelu_mul(A, B_gate, B_up, C, M, N, K, lda, ldb, ldc, b_layout, as_stream(stream));
}

ANYGPU_EXPORT int anygpu_softmax_rows_f16(const void* x, void* y, int64_t rows, int64_t cols,
                                          int64_t x_row_stride, int64_t y_row_stride,
                                          int64_t q_len, int64_t diag,
                                          float alpha, float softcap, int causal, int64_t window, void* stream)
{
	return softmax_entry<anygpu::half_t>(x, y, rows, cols, x_row_stride, y_row_stride, q_len, diag, alpha, softcap,
	                                     causal, window, stream);
}

ANYGPU_EXPORT int anygpu_softmax_rows_f32(const float* x, float* y, int64_t rows, int64_t cols,
                                          int64_t x_row_stride, int64_t y_row_stride,
                                          int64_t q_len, int64_t diag,
                                          float alpha, float softcap, int causal, int64_t window, void* stream)
{
	return softmax_entry<float>(x, y, rows, cols, x_row_stride, y_row_stride, q_len, diag, alpha, softcap,
	                            causal, window, stream);
}

ANYGPU_EXPORT int anygpu_softmax_rows_masked_f16(const void* x, const void* mask, void* y, int64_t rows, int64_t cols,
                                                 int64_t x_row_stride, int64_t mask_row_stride, int64_t y_row_stride,
                                                 int64_t q_len, float alpha, float softcap, void* stream)
{
	return softmax_masked_entry<anygpu::half_t>(x, mask, y, rows, cols, x_row_stride, mask_row_stride, y_row_stride,
	                                            q_len, alpha, softcap, stream);
}

ANYGPU_EXPORT int anygpu_softmax_rows_masked_f32(const float* x, const float* mask, float* y, int64_t rows, int64_t cols,
                                                 int64_t x_row_stride, int64_t mask_row_stride, int64_t y_row_stride,
                                                 int64_t q_len, float alpha, float softcap, void* stream)
{
	return softmax_masked_entry<float>(x, mask, y, rows, cols, x_row_stride, mask_row_stride, y_row_stride,
	                                   q_len, alpha, softcap, stream);
}

ANYGPU_EXPORT int anygpu_sdp_attention_fwd_f16(const void* q, const void* k, const void* v, void* y,
                                               int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                               float alpha, float softcap, int causal, int64_t window, void* stream)
{
	const int rc = check_attention(q, k, v, y, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha, softcap, window);
	if (rc != ANYGPU_OK) return rc;
	if (batch_heads == 0 || n_q == 0) return ANYGPU_OK;
	return (int)anygpu::launch_sdp_attention_fwd_f16(q, k, v, y, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha, softcap,
	                                                 causal, window, as_stream(stream));
}

ANYGPU_EXPORT int anygpu_sdp_attention_fwd_masked_f16(const void* q, const void* k, const void* v, const void* mask, void* y,
                                                      int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                                      int64_t mask_stride, float alpha, float softcap, void* stream)
{
	const int rc = check_attention(q, k, v, y, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha, softcap, 0);
	if (rc != ANYGPU_OK) return rc;
	if (batch_heads == 0 || n_q == 0) return ANYGPU_OK;
	if (mask == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if (mask_stride < n_k) return ANYGPU_ERR_BAD_STRIDE;
	if (reinterpret_cast<uintptr_t>(mask) % 2 != 0) return ANYGPU_ERR_UNSUPPORTED;
	return (int)anygpu::launch_sdp_attention_fwd_f16(q, k, v, y, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha, softcap,
	                                                 0, 0, as_stream(stream), mask, mask_stride);
}

ANYGPU_EXPORT int anygpu_sdp_attention_fwd_f32(const float* q, const float* k, const float* v, float* y,
                                               int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                               float alpha, float softcap, int causal, int64_t window, void* stream)
{
	const int rc = check_attention(q, k, v, y, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha, softcap, window);
	if (rc != ANYGPU_OK) return rc;
	if (batch_heads == 0 || n_q == 0) return ANYGPU_OK;
	return (int)anygpu::launch_sdp_attention_fwd_f32(q, k, v, y, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha, softcap,
	                                                 causal, window, as_stream(stream));
}

ANYGPU_EXPORT int anygpu_sdp_attention_fwd_masked_f32(const float* q, const float* k, const float* v, const float* mask, float* y,
                                                      int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                                      int64_t mask_stride, float alpha, float softcap, void* stream)
{
	const int rc = check_attention(q, k, v, y, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha, softcap, 0);
	if (rc != ANYGPU_OK) return rc;
	if (batch_heads == 0 || n_q == 0) return ANYGPU_OK;
	if (mask == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if (mask_stride < n_k) return ANYGPU_ERR_BAD_STRIDE;
	return (int)anygpu::launch_sdp_attention_fwd_f32(q, k, v, y, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha, softcap,
	                                                 0, 0, as_stream(stream), mask, mask_stride);
}

ANYGPU_EXPORT int64_t anygpu_sdp_attention_decode_workspace_bytes(int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k,
                                                                  int64_t head_dim, int causal, int64_t window)
{
	const int rc = check_attention_shape(batch_heads, q_per_kv, n_q, n_k, head_dim, window);
	if (rc != ANYGPU_OK) return rc;
	if (batch_heads == 0 || n_q == 0) return 0;
	if (!anygpu::sdp_attention_decode_f16_supports(q_per_kv, n_q, head_dim)) return ANYGPU_ERR_UNSUPPORTED;
	return anygpu::sdp_attention_decode_workspace_bytes(batch_heads, q_per_kv, n_q, n_k, head_dim, causal, window);
}

ANYGPU_EXPORT int anygpu_sdp_attention_decode_f16(const void* q, const void* k, const void* v, void* y,
                                                  void* workspace, int64_t workspace_bytes,
                                                  int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                                  float alpha, float softcap, int causal, int64_t window, void* stream)
{
	const int rc = check_attention(q, k, v, y, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha, softcap, window);
	if (rc != ANYGPU_OK) return rc;
	if (batch_heads == 0 || n_q == 0) return ANYGPU_OK;
	if (!anygpu::sdp_attention_decode_f16_supports(q_per_kv, n_q, head_dim)) return ANYGPU_ERR_UNSUPPORTED;
	const int64_t need = anygpu::sdp_attention_decode_workspace_bytes(batch_heads, q_per_kv, n_q, n_k, head_dim, causal, window);
	if (workspace == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if (workspace_bytes < need) return ANYGPU_ERR_BAD_SHAPE;
	if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return ANYGPU_ERR_UNSUPPORTED;
	return (int)anygpu::launch_sdp_attention_decode_f16(q, k, v, y, workspace, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha,
	                                                    softcap, causal, window, as_stream(stream));
}

ANYGPU_EXPORT int anygpu_sdp_attention_decode_f16_static(const void* q, const void* k, const void* v, void* y,
                                                         int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                                         float alpha, float softcap, int causal, int64_t window, void* stream)
{
	const int rc = check_attention(q, k, v, y, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha, softcap, window);
	if (rc != ANYGPU_OK) return rc;
	// (looked up before the early return for empty problems, so that an empty call can serve as the set-up call)
	void* ws = nullptr;
	const hipError_t e = scratch_of_current_device(&ws);
	if (e != hipSuccess) return (int)e;
	if (batch_heads == 0 || n_q == 0) return ANYGPU_OK;
	if (!anygpu::sdp_attention_decode_f16_supports(q_per_kv, n_q, head_dim)) return ANYGPU_ERR_UNSUPPORTED;
	const int64_t need = anygpu::sdp_attention_decode_workspace_bytes(batch_heads, q_per_kv, n_q, n_k, head_dim, causal, window);
	if (need > (int64_t)ANYGPU_DECODE_STATIC_SCRATCH_BYTES) return ANYGPU_ERR_SCRATCH_TOO_SMALL;
	return (int)anygpu::launch_sdp_attention_decode_f16(q, k, v, y, ws, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha,
	                                                    softcap, causal, window, as_stream(stream));
}

ANYGPU_EXPORT int64_t anygpu_sdp_attention_decode_f32_workspace_bytes(int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k,
                                                                      int64_t head_dim, int causal, int64_t window)
{
	const int rc = check_attention_shape(batch_heads, q_per_kv, n_q, n_k, head_dim, window);
	if (rc != ANYGPU_OK) return rc;
	if (batch_heads == 0 || n_q == 0) return 0;
	if (!anygpu::sdp_attention_decode_f32_supports(q_per_kv, n_q, head_dim)) return ANYGPU_ERR_UNSUPPORTED;
	return anygpu::sdp_attention_decode_f32_workspace_bytes(batch_heads, q_per_kv, n_q, n_k, head_dim, causal, window);
}

ANYGPU_EXPORT int anygpu_sdp_attention_decode_f32(const float* q, const float* k, const float* v, float* y,
                                                  void* workspace, int64_t workspace_bytes,
                                                  int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                                  float alpha, float softcap, int causal, int64_t window, void* stream)
{
	const int rc = check_attention(q, k, v, y, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha, softcap, window);
	if (rc != ANYGPU_OK) return rc;
	if (batch_heads == 0 || n_q == 0) return ANYGPU_OK;
	if (!anygpu::sdp_attention_decode_f32_supports(q_per_kv, n_q, head_dim)) return ANYGPU_ERR_UNSUPPORTED;
	const int64_t need = anygpu::sdp_attention_decode_f32_workspace_bytes(batch_heads, q_per_kv, n_q, n_k, head_dim, causal, window);
	if (workspace == nullptr) return ANYGPU_ERR_NULL_POINTER;
	if (workspace_bytes < need) return ANYGPU_ERR_BAD_SHAPE;
	if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return ANYGPU_ERR_UNSUPPORTED;
	return (int)anygpu::launch_sdp_attention_decode_f32(q, k, v, y, workspace, batch_heads, q_per_kv, n_q, n_k, head_dim, alpha,
	                                                    softcap, causal, window, as_stream(stream));
}

ANYGPU_EXPORT int anygpu_causal_conv1d_silu_f16(const void* x, const void* w, const void* bias, void* y,
                                                int64_t batch, int64_t chan, int64_t seqlen, int64_t width,
                                                void* stream)
{
	return conv_entry<anygpu::half_t>(x, w, bias, y, batch, chan, seqlen, width, stream);
}

ANYGPU_EXPORT int anygpu_causal_conv1d_silu_f32(const float* x, const float* w, const float* bias, float* y,
                                                int64_t batch, int64_t chan, int64_t seqlen, int64_t width,
                                                void* stream)
{
	return conv_entry<float>(x, w, bias, y, batch, chan, seqlen, width, stream);
}


ANYGPU_EXPORT int anygpu_causal_conv1d_silu_update_f16(const void* x, void* state, const void* w, const void* bias, void* y,
                                                       int64_t batch, int64_t chan, int64_t width, void* stream)
{
	return conv_update_entry<anygpu::half_t>(x, state, w, bias, y, batch, chan, width, stream);
}

ANYGPU_EXPORT int anygpu_causal_conv1d_silu_update_f32(const float* x, float* state, const float* w, const float* bias, float* y,
                                                       int64_t batch, int64_t chan, int64_t width, void* stream)
{
	return conv_update_entry<float>(x, state, w, bias, y, batch, chan, width, stream);
}

ANYGPU_EXPORT int anygpu_gated_rmsnorm_f16(const void* x, const void* z, const void* w, void* y,
                                           int64_t rows, int64_t cols, float eps, int zero_centered, void* stream)
{
	return gated_rmsnorm_entry<anygpu::half_t>(x, z, w, y, rows, cols, eps, zero_centered, stream);
}

ANYGPU_EXPORT int anygpu_gated_rmsnorm_f32(const float* x, const float* z, const float* w, float* y,
                                           int64_t rows, int64_t cols, float eps, int zero_centered, void* stream)
{
	return gated_rmsnorm_entry<float>(x, z, w, y, rows, cols, eps, zero_centered, stream);
}

}  // extern "C"
