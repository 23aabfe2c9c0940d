// Host-side launch functions implemented by the kernel translation units and called by the
// C ABI layer.  Arguments are already validated when these are reached.
#pragma once

#include <hip/hip_runtime.h>
#include <atomic>
#include <cstdint>

namespace anygpu {

// The runtime keeps the last error of the calling thread until somebody reads it, whoever
// caused it.  Launchers call this before their own launch so that the code they return
// afterwards (hipGetLastError) belongs to that launch and to nothing earlier in the process.
inline void discard_stale_error() { (void)hipGetLastError(); }

// Compute units of the current device (256 on an MI355X), asked once per device; 256 if the runtime cannot tell.
inline int device_cu_count()
{
	// (launchers on several host threads may ask at once: the cache is written and read atomically, and two threads
	// that both find it empty store the same value)
	static std::atomic<int> cached[64] = {};
	int device = 0;
	if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
	int cus = cached[device].load(std::memory_order_relaxed);
	if (cus == 0)
	{
		if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) cus = 256;
		cached[device].store(cus, std::memory_order_relaxed);
	}
	return cus;
}

// mask (may be NULL): additive [q_len, cols] matrix of the element type, rows mask_stride apart
template <typename T>
hipError_t launch_softmax_rows(const void* x, void* y, int64_t rows, int64_t cols, int64_t xs, int64_t ys,
                               int64_t q_len, int64_t diag, float alpha, float softcap, int causal,
                               int64_t window, const void* mask, int64_t mask_stride, hipStream_t stream);

template <typename T>
hipError_t launch_causal_conv1d_silu(const void* x, const void* w, const void* bias, void* y,
                                     int64_t batch, int64_t chan, int64_t seqlen, int width,
                                     hipStream_t stream);

// one new sample per (batch, chan) row; state [batch, chan, width - 1] is shifted in place
template <typename T>
hipError_t launch_causal_conv1d_silu_update(const void* x, void* state, const void* w, const void* bias, void* y,
                                            int64_t batch, int64_t chan, int width, hipStream_t stream);

// y = rms_norm(x * silu(z)) * (w + zero_centered) over rows of `cols`; z == NULL: no gate
template <typename T>
hipError_t launch_gated_rmsnorm(const void* x, const void* z, const void* w, void* y, int64_t rows, int64_t cols,
                                float eps, int zero_centered, hipStream_t stream);

// What launch_gemm_f16 does to the sums where its plan has a place for it besides a tile kernel's own epilogue: the
// few-row kernels and the merge behind a cut along K.  epilogue: kEpiBias (fp16 bias) or kEpiSoftcap.  On return
// `handled` says whether the product was launched that way; if not, nothing was launched.
struct GemmF16Finish
{
	int epilogue;
	const void* bias;
	float ep_param;
	bool handled;
};

// `batch` independent products of one shape, operand b of product i at base + i * stride_b (elements).  `finish`
// (batch 1 only): see GemmF16Finish.
hipError_t launch_gemm_f16(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                           int64_t lda, int64_t ldb, int64_t ldc,
                           int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                           int b_layout, hipStream_t stream, GemmF16Finish* finish = nullptr);

// The fp16 product with an epilogue (gemm_epilogue.hpp: kEpiBias with an fp16 bias, kEpiSoftcap, kEpiGeluMul with B2);
// *supported = false and nothing launched for the few shapes no kernel with that epilogue takes.
hipError_t launch_gemm_f16_epilogue(const void* A, const void* B, const void* B2, const void* bias, void* C,
                                    int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                    int b_layout, int epilogue, float ep_param, hipStream_t stream, bool* supported);

// The fp16 product through the four-wave 256 x 256 tile kernel with its clock probe (see gemm_f16_ring.hpp); false /
// nothing launched when the product does not meet that kernel's conditions.
bool gemm_f16_probe_applies(const void* A, const void* B, const void* C, int64_t M, int64_t N, int64_t K,
                            int64_t lda, int64_t ldb, int64_t ldc, int b_layout);
hipError_t launch_gemm_f16_probe(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                                 int64_t lda, int64_t ldb, int64_t ldc, unsigned long long* probe, hipStream_t stream);

// Few rows (M <= 64) against n-contiguous fp16 weights with very many columns (gemm_band_kn_f16.hip); epilogue kEpiBias
// (nothing added) or kEpiSoftcap.
bool gemm_band_kn_f16_applies(const void* A, const void* B, const void* C, int64_t M, int64_t N, int64_t K,
                              int64_t lda, int64_t ldb, int64_t ldc);
hipError_t launch_gemm_band_kn_f16(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                                   int64_t lda, int64_t ldb, int64_t ldc, int epilogue, float ep_param, hipStream_t stream);

// Few rows (M <= max_rows <= 64) against k-contiguous weights ([N, K]) with the many columns of an output head, fp32 or
// fp16 (gemm_band_kc_wide.hip); epilogue kEpiBias (bias may be NULL) or kEpiSoftcap.
template <typename T>
bool gemm_band_kc_wide_applies(const T* A, const T* B, const T* C, int64_t M, int64_t N, int64_t K,
                               int64_t lda, int64_t ldb, int64_t ldc, int64_t max_rows);
// (fewer columns, with the cut along K that then fills the chip; planes in the stream's workspace)
template <typename T>
bool gemm_band_kc_wide_split_applies(const T* A, const T* B, const T* C, int64_t M, int64_t N, int64_t K,
                                     int64_t lda, int64_t ldb, int64_t ldc, int64_t max_rows, hipStream_t stream);
template <typename T>
hipError_t launch_gemm_band_kc_wide(const T* A, const T* B, const T* bias, T* C, int64_t M, int64_t N, int64_t K,
                                    int64_t lda, int64_t ldb, int64_t ldc, int epilogue, float ep_param, hipStream_t stream);

// dst[i] = src[i] over nvec 16-byte vectors in the stated launch geometry (stream_probe.hip)
hipError_t launch_stream_probe(const void* src, void* dst, int64_t nvec, int block, int vectors_per_lane, int nt_load,
                               int nt_store, int64_t grid_limit, hipStream_t stream);

// Aligned copies of operands the tile kernels cannot fetch as they lie (gemm_repack.hip): `rows` rows of `cols` elements
// at any alignment into rows of pitch ld_dst (a multiple of 64 elements, 16-byte aligned), zeros behind `cols` and in
// the rows from `rows` up to rows_dst; and the same from a [k_rows, n_cols] matrix read down its columns,
// dst[n][k] = src[k][n].  elem_bytes 2 or 4.
hipError_t launch_repack_rows(const void* src, int64_t ld_src, int64_t rows, int64_t cols, void* dst, int64_t ld_dst,
                              int elem_bytes, hipStream_t stream, int64_t rows_dst = 0);
hipError_t launch_repack_transposed(const void* src, int64_t ld_src, int64_t k_rows, int64_t n_cols, void* dst, int64_t ld_dst,
                                    int elem_bytes, hipStream_t stream);

hipError_t launch_gemm_f32(const float* A, const float* B, const float* bias, float* C,
                           int64_t M, int64_t N, int64_t K,
                           int64_t lda, int64_t ldb, int64_t ldc,
                           int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                           int a_layout, int b_layout, hipStream_t stream);

// C = softcap * tanh((A * B) / softcap)
hipError_t launch_gemm_f32_softcap(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K,
                                   int64_t lda, int64_t ldb, int64_t ldc, int b_layout, float softcap, hipStream_t stream);

// C = gelu_tanh(A * B_gate) * (A * B_up), elementwise; both right operands share layout and leading dimension
hipError_t launch_gemm_f32_gelu_mul(const float* A, const float* B_gate, const float* B_up, float* C,
                                    int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                    int b_layout, hipStream_t stream);

// Fused attention forward, fp16: q [batch_heads, n_q, head_dim], k and v [batch_heads / q_per_kv, n_k, head_dim],
// y like q; mask rules as in launch_softmax_rows with the diagonal at n_k - n_q.  mask: optional additive mask of halves
// [n_q, n_k] (rows mask_stride halves apart) shared by all heads, added behind scale and softcap; it replaces the index rules
// (causal and window are ignored with it).
bool sdp_attention_fwd_f16_supports(int64_t head_dim);
hipError_t launch_sdp_attention_fwd_f16(const void* q, const void* k, const void* v, void* y,
                                        int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                        float alpha, float softcap, int causal, int64_t window, hipStream_t stream,
                                        const void* mask = nullptr, int64_t mask_stride = 0);

// The same in float32 with the fp32 matrix instruction.  mask: optional additive mask [n_q, n_k] (rows mask_stride floats
// apart) shared by all heads, added behind scale and softcap, on top of the index rules.
bool sdp_attention_fwd_f32_supports(int64_t head_dim);
hipError_t launch_sdp_attention_fwd_f32(const float* q, const float* k, const float* v, float* y,
                                        int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                        float alpha, float softcap, int causal, int64_t window, hipStream_t stream,
                                        const float* mask = nullptr, int64_t mask_stride = 0);

// Decode form of the fused attention (q_per_kv * n_q <= 16 rows per key / value head): the key range is split over
// waves, partial results go through `workspace` (sdp_attention_decode_workspace_bytes of fp32 scratch, 16-byte aligned).
bool sdp_attention_decode_f16_supports(int64_t q_per_kv, int64_t n_q, int64_t head_dim);
int64_t sdp_attention_decode_workspace_bytes(int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                             int causal, int64_t window);
hipError_t launch_sdp_attention_decode_f16(const void* q, const void* k, const void* v, void* y, void* workspace,
                                           int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                           float alpha, float softcap, int causal, int64_t window, hipStream_t stream);

// Decode form in float32: keys in tiles of 16, both operands straight from global memory.
bool sdp_attention_decode_f32_supports(int64_t q_per_kv, int64_t n_q, int64_t head_dim);
int64_t sdp_attention_decode_f32_workspace_bytes(int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                                 int causal, int64_t window);
hipError_t launch_sdp_attention_decode_f32(const float* q, const float* k, const float* v, float* y, void* workspace,
                                           int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                           float alpha, float softcap, int causal, int64_t window, hipStream_t stream);

// Few-row products (M <= kSkinnyMaxRows, one product, row-major A): bandwidth-shaped kernels that
// stream B once.  `epilogue` is an Epilogue value; B2 only for kEpiGeluMul, bias only for kEpiBias
// (either may be NULL).  T is float or _Float16.  gemm_skinny_applies says whether shape, leading
// dimensions and alignment allow them; the launchers of the tile kernels ask it first.
constexpr int64_t kSkinnyMaxRows = 8;

template <typename T>
bool gemm_skinny_applies(const T* A, const T* B, const T* B2, int64_t M, int64_t N, int64_t K,
                         int64_t lda, int64_t ldb, int b_layout);

template <typename T>
hipError_t launch_gemm_skinny(const T* A, const T* B, const T* B2, const T* bias, T* C,
                              int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                              int b_layout, int epilogue, float ep_param, hipStream_t stream);

// Bands of few rows (kBandMinRows <= M <= kBandMaxRows, one product, row-major A, k-contiguous B): the
// weights stream through the MFMA operand registers once, K is split over blocks when the columns alone do
// not fill the chip.  Same arguments as the skinny launchers, which the launchers ask after these: from 5
// rows on the FMA loops of the skinny kernels fall behind (256000 x 2304 fp32 weights, 8 rows: 511 us
// against 398 us); in fp32 already from 3 rows (4 rows x 14336 -> 4096: 86 us with FMAs, 41 us as a band;
// 4096 -> 32768: 113 against 93; the fp16 skinny kernel with its packed dot products holds up to 4 rows).
constexpr int64_t kBandMinRows = 5;
constexpr int64_t kBandMinRowsF32 = 3;
constexpr int64_t kBandMaxRows = 64;

template <typename T>
bool gemm_band_applies(const T* A, const T* B, const T* B2, const T* C, int64_t M, int64_t N, int64_t K,
                       int64_t lda, int64_t ldb, int64_t ldc, int b_layout);

template <typename T>
hipError_t launch_gemm_band(const T* A, const T* B, const T* B2, const T* bias, T* C,
                            int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                            int epilogue, float ep_param, hipStream_t stream);

// The same for n-contiguous fp32 weights (row-major B) from one row on: there the band kernel is ahead of the
// skinny one at every row count (9216 x 2304 weights, 4 rows: 21 us against 50 us).  Any N from 4 on (the last vector of a row is moved back to end at N).
// `dual`: two weight matrices (kEpiGeluMul), which are limited to 32 rows.
bool gemm_band_ncontig_applies(const float* A, const float* B, const float* B2, const float* C, int64_t M, int64_t N, int64_t K,
                               int64_t lda, int64_t ldb, int64_t ldc, bool dual);

hipError_t launch_gemm_band_ncontig(const float* A, const float* B, const float* B2, const float* bias, float* C,
                                    int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                    int epilogue, float ep_param, hipStream_t stream);

}  // namespace anygpu
