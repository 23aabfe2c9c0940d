// Host-layer launchers -> C ABI of libanygpu_hip.so.  This is the only translation unit of
// the host layer that knows the ABI; it turns every non-zero return code into the fail-stop
// convention of the layer (message with the code and its text, exit(1)).
#include "mm_ops.cuh"
#include "fast_mm.cuh"
#include "softmax_ops.cuh"
#include "causal_conv1d.cuh"
#include "norm_ops.cuh"
#include "flash_sdpa_fwd.cuh"
#include "mlp_gemma2_fused_upproj.cuh"
#include "mlp_gemma2_dp_linear.cuh"
#include "sdpa_gemma2_linear.cuh"
#include "gemma_linsoftcap.cuh"

#include "anygpu_hip.h"

namespace {

void* const kNullStream = nullptr;

void check_abi(int code, const char* what, const char* file, int line)
{
	if (code == ANYGPU_OK) return;
	std::string msg = std::string(what) + ": " + anygpu_hip_error_string(code);
	fail_runtime(code, msg.c_str(), file, line);
}

#define ABI_CHECK(call) check_abi((call), #call, __FILE__, __LINE__)

// out[M, N] = lhs * rhs with rhs either [K, N] (row-major) or [N, K] (column-major storage of B)
template <typename T>
void mm_dispatch(const Tensor<T, CUDA>& lhs, const Tensor<T, CUDA>& rhs, const Tensor<T, CUDA>& out,
                 int a_layout, int b_layout, const float32* bias)
{
	const int64 m = (a_layout == ANYGPU_A_ROW_MAJOR) ? lhs.shape[0] : lhs.shape[1];
	const int64 k = (a_layout == ANYGPU_A_ROW_MAJOR) ? lhs.shape[1] : lhs.shape[0];
	const int64 n = (b_layout == ANYGPU_B_ROW_MAJOR) ? rhs.shape[1] : rhs.shape[0];
	// dense operands: the leading dimension is the extent of the innermost axis
	const int64 lda = std::max<int64>(lhs.shape[1], 1);
	const int64 ldb = std::max<int64>(rhs.shape[1], 1);
	const int64 ldc = std::max<int64>(n, 1);
	if constexpr (std::is_same_v<T, float32>)
	{
		ABI_CHECK(anygpu_gemm_f32(lhs.buffer(), rhs.buffer(), bias, out.buffer(), m, n, k, lda, ldb, ldc,
		                          a_layout, b_layout, kNullStream));
	}
	else
	{
		static_assert(std::is_same_v<T, float16>, "Unsupported data type");
		ABI_CHECK(anygpu_gemm_f16_f32acc(lhs.buffer(), rhs.buffer(), out.buffer(), m, n, k, lda, ldb, ldc,
		                                 b_layout, kNullStream));
	}
}

template <typename T>
void softmax_dispatch(const Tensor<T, CUDA>& x, const SoftmaxPrologue& p, Tensor<T, CUDA>& y)
{
	const int64 rows = x.shape[0], cols = x.shape[1];
	const int64 pitch = std::max<int64>(cols, 1);
	if constexpr (std::is_same_v<T, float32>)
	{
		ABI_CHECK(anygpu_softmax_rows_f32(x.buffer(), y.buffer(), rows, cols, pitch, pitch, p.q_len, p.diag,
		                                  p.alpha, p.softcap, p.causal ? 1 : 0, p.window, kNullStream));
	}
	else
	{
		static_assert(std::is_same_v<T, float16>, "Unsupported data type");
		ABI_CHECK(anygpu_softmax_rows_f16(x.buffer(), y.buffer(), rows, cols, pitch, pitch, p.q_len, p.diag,
		                                  p.alpha, p.softcap, p.causal ? 1 : 0, p.window, kNullStream));
	}
}

}  // namespace

void cu_tensor_mm_f32_opt0(const Tensor<float32, CUDA>& lhs, const Tensor<float32, CUDA>& rhs, const Tensor<float32, CUDA>& out)
{
	mm_dispatch(lhs, rhs, out, ANYGPU_A_ROW_MAJOR, ANYGPU_B_ROW_MAJOR, nullptr);
}

void cu_tensor_gemm_f32_opt0(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA>& wt,
                             const Tensor<float32, CUDA>& bt, const Tensor<float32, CUDA>& out)
{
	mm_dispatch(xt, wt, out, ANYGPU_A_ROW_MAJOR, ANYGPU_B_ROW_MAJOR, bt.buffer());
}

void opt1::cu_tensor_mm_f32(const Tensor<float32, CUDA>& lhs, const Tensor<float32, CUDA>& rhs, const Tensor<float32, CUDA>& out)
{
	mm_dispatch(lhs, rhs, out, ANYGPU_A_ROW_MAJOR, ANYGPU_B_ROW_MAJOR, nullptr);
}

void opt2::cu_tensor_mm_f16(const Tensor<float16, CUDA>& lhs, const Tensor<float16, CUDA>& rhs, const Tensor<float16, CUDA>& out)
{
	mm_dispatch(lhs, rhs, out, ANYGPU_A_ROW_MAJOR, ANYGPU_B_ROW_MAJOR, nullptr);
}

void hip_tensor_mm_nt_f16(const Tensor<float16, CUDA>& lhs, const Tensor<float16, CUDA>& rhs_nk, const Tensor<float16, CUDA>& out)
{
	mm_dispatch(lhs, rhs_nk, out, ANYGPU_A_ROW_MAJOR, ANYGPU_B_COL_MAJOR, nullptr);
}

void hip_tensor_mm_nt_f32(const Tensor<float32, CUDA>& lhs, const Tensor<float32, CUDA>& rhs_nk, const Tensor<float32, CUDA>& out)
{
	mm_dispatch(lhs, rhs_nk, out, ANYGPU_A_ROW_MAJOR, ANYGPU_B_COL_MAJOR, nullptr);
}

#define ANYGPU_DEFINE_FAST_MM(NAME, T, A_LAYOUT)                                              \
	void NAME(const Tensor<T, CUDA>& xt, const Tensor<T, CUDA>& wt, Tensor<T, CUDA>& yt)      \
	{                                                                                         \
		mm_dispatch(xt, wt, yt, A_LAYOUT, ANYGPU_B_ROW_MAJOR, nullptr);                       \
	}

ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f32_cb, float32, ANYGPU_A_ROW_MAJOR)
ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f32_v1, float32, ANYGPU_A_ROW_MAJOR)
ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f32_v2, float32, ANYGPU_A_ROW_MAJOR)
ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f32_v2_1, float32, ANYGPU_A_ROW_MAJOR)
ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f32_v3, float32, ANYGPU_A_ROW_MAJOR)
ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f32_v4, float32, ANYGPU_A_ROW_MAJOR)
ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f32_v4_1, float32, ANYGPU_A_ROW_MAJOR)
ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f32_v4_2, float32, ANYGPU_A_COL_MAJOR)
ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f16_v1, float16, ANYGPU_A_ROW_MAJOR)
ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f16_v2, float16, ANYGPU_A_ROW_MAJOR)
ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f16_v3, float16, ANYGPU_A_ROW_MAJOR)
ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f16_v3_1, float16, ANYGPU_A_ROW_MAJOR)
ANYGPU_DEFINE_FAST_MM(cu_fast_mm_f16_v3_2, float16, ANYGPU_A_ROW_MAJOR)

#undef ANYGPU_DEFINE_FAST_MM

void cu_tensor_softmax_f32(const Tensor<float32, CUDA>& x, Tensor<float32, CUDA>& y)
{
	softmax_dispatch(x, SoftmaxPrologue{}, y);
}

void hip_tensor_softmax_f16(const Tensor<float16, CUDA>& x, Tensor<float16, CUDA>& y)
{
	softmax_dispatch(x, SoftmaxPrologue{}, y);
}

void hip_tensor_softmax_fused_f32(const Tensor<float32, CUDA>& x, const SoftmaxPrologue& prologue, Tensor<float32, CUDA>& y)
{
	softmax_dispatch(x, prologue, y);
}

void hip_tensor_softmax_fused_f16(const Tensor<float16, CUDA>& x, const SoftmaxPrologue& prologue, Tensor<float16, CUDA>& y)
{
	softmax_dispatch(x, prologue, y);
}

template<typename dtype>
void hip_tensor_mm_batched(const Tensor<dtype, CUDA>& lhs, const Tensor<dtype, CUDA>& rhs, const Tensor<dtype, CUDA>& out,
                           const int64 batch, const int64 m, const int64 n, const int64 k, const bool rhs_is_nk)
{
	const int b_layout = rhs_is_nk ? ANYGPU_B_COL_MAJOR : ANYGPU_B_ROW_MAJOR;
	const int64 lda = std::max<int64>(k, 1), ldb = std::max<int64>(rhs_is_nk ? k : n, 1), ldc = std::max<int64>(n, 1);
	if constexpr (std::is_same_v<dtype, float32>)
	{
		ABI_CHECK(anygpu_gemm_f32_batched(lhs.buffer(), rhs.buffer(), out.buffer(), m, n, k, lda, ldb, ldc,
		                                  m * k, n * k, m * n, batch, ANYGPU_A_ROW_MAJOR, b_layout, kNullStream));
	}
	else
	{
		static_assert(std::is_same_v<dtype, float16>, "Unsupported data type");
		ABI_CHECK(anygpu_gemm_f16_f32acc_batched(lhs.buffer(), rhs.buffer(), out.buffer(), m, n, k, lda, ldb, ldc,
		                                         m * k, n * k, m * n, batch, b_layout, kNullStream));
	}
}

template void hip_tensor_mm_batched<float32>(const Tensor<float32, CUDA>&, const Tensor<float32, CUDA>&,
                                             const Tensor<float32, CUDA>&, int64, int64, int64, int64, bool);
template void hip_tensor_mm_batched<float16>(const Tensor<float16, CUDA>&, const Tensor<float16, CUDA>&,
                                             const Tensor<float16, CUDA>&, int64, int64, int64, int64, bool);

template<typename dtype>
void hip_tensor_softmax_masked(const Tensor<dtype, CUDA>& x, const Tensor<dtype, CUDA>& mask, const float32 alpha,
                               const int64 q_len, Tensor<dtype, CUDA>& y)
{
	const int64 rows = x.shape[0], cols = x.shape[1];
	const int64 pitch = std::max<int64>(cols, 1);
	if constexpr (std::is_same_v<dtype, float32>)
	{
		ABI_CHECK(anygpu_softmax_rows_masked_f32(x.buffer(), mask.buffer(), y.buffer(), rows, cols, pitch, pitch, pitch,
		                                         q_len, alpha, 0.f, kNullStream));
	}
	else
	{
		static_assert(std::is_same_v<dtype, float16>, "Unsupported data type");
		ABI_CHECK(anygpu_softmax_rows_masked_f16(x.buffer(), mask.buffer(), y.buffer(), rows, cols, pitch, pitch, pitch,
		                                         q_len, alpha, 0.f, kNullStream));
	}
}

template void hip_tensor_softmax_masked<float32>(const Tensor<float32, CUDA>&, const Tensor<float32, CUDA>&, float32,
                                                 int64, Tensor<float32, CUDA>&);
template void hip_tensor_softmax_masked<float16>(const Tensor<float16, CUDA>&, const Tensor<float16, CUDA>&, float32,
                                                 int64, Tensor<float16, CUDA>&);

void cu_tensor_causal_conv1d_f32(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA>& wt,
                                 const Tensor<float32, CUDA>& bt, Tensor<float32, CUDA>& yt)
{
	ABI_CHECK(anygpu_causal_conv1d_silu_f32(xt.buffer(), wt.buffer(), bt.buffer(), yt.buffer(),
	                                        xt.shape[0], xt.shape[1], xt.shape[2], wt.shape[1], kNullStream));
}

void hip_tensor_causal_conv1d_f16(const Tensor<float16, CUDA>& xt, const Tensor<float16, CUDA>& wt,
                                  const Tensor<float16, CUDA>& bt, Tensor<float16, CUDA>& yt)
{
	ABI_CHECK(anygpu_causal_conv1d_silu_f16(xt.buffer(), wt.buffer(), bt.buffer(), yt.buffer(),
	                                        xt.shape[0], xt.shape[1], xt.shape[2], wt.shape[1], kNullStream));
}

/* ---- GEMM epilogues of the Gemma2 callers ---- */

void cu_tensor_gemma_linear_softcap_f32(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA>& wt,
                                        const float32 final_softcapping, Tensor<float32, CUDA>& yt)
{
	const int64 n = xt.shape[0] * xt.shape[1];   // batch * seq_len rows
	const int64 hsize = wt.shape[1], vsize = wt.shape[0];
	ABI_CHECK(anygpu_gemm_f32_softcap(xt.buffer(), wt.buffer(), yt.buffer(), n, vsize, hsize,
	                                  std::max<int64>(hsize, 1), std::max<int64>(hsize, 1), std::max<int64>(vsize, 1),
	                                  ANYGPU_B_COL_MAJOR, final_softcapping, kNullStream));
}

namespace {

void fused_upproj(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA>& wt_gp,
                  const Tensor<float32, CUDA>& wt_up, Tensor<float32, CUDA>& yt)
{
	const int64 sl = xt.shape[0] * xt.shape[1];
	const int64 hsize = wt_gp.shape[0], isize = wt_gp.shape[1];
	ABI_CHECK(anygpu_gemm_f32_gelu_mul(xt.buffer(), wt_gp.buffer(), wt_up.buffer(), yt.buffer(), sl, isize, hsize,
	                                   std::max<int64>(hsize, 1), std::max<int64>(isize, 1), std::max<int64>(isize, 1),
	                                   ANYGPU_B_ROW_MAJOR, kNullStream));
}

}  // namespace

void cu_mlp_gemma2_fused_upproj_f32_v1(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA>& wt_gp,
                                       const Tensor<float32, CUDA>& wt_up, Tensor<float32, CUDA>& yt)
{
	fused_upproj(xt, wt_gp, wt_up, yt);
}

void cu_mlp_gemma2_fused_upproj_f32_v2(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA>& wt_gp,
                                       const Tensor<float32, CUDA>& wt_up, Tensor<float32, CUDA>& yt)
{
	fused_upproj(xt, wt_gp, wt_up, yt);
}

namespace {

// y (batch, seq_len, out) = x (batch, seq_len, in) * w (in, out): the leading axes fold into rows
void linear_over_tokens(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA>& wt, Tensor<float32, CUDA>& yt)
{
	const int64 sl = xt.shape[0] * xt.shape[1];
	const int64 in_features = wt.shape[0], out_features = wt.shape[1];
	ABI_CHECK(anygpu_gemm_f32(xt.buffer(), wt.buffer(), nullptr, yt.buffer(), sl, out_features, in_features,
	                          std::max<int64>(in_features, 1), std::max<int64>(out_features, 1), std::max<int64>(out_features, 1),
	                          ANYGPU_A_ROW_MAJOR, ANYGPU_B_ROW_MAJOR, kNullStream));
}

}  // namespace

void cu_mlp_gemma2_dp_linear_f32_v1(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA>& wt_dp, Tensor<float32, CUDA>& yt)
{
	linear_over_tokens(xt, wt_dp, yt);
}

void cu_mlp_gemma2_dp_linear_f32_v4(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA>& wt_dp, Tensor<float32, CUDA>& yt)
{
	linear_over_tokens(xt, wt_dp, yt);
}

void cu_sdpa_gemma2_linear_f32_v1(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA>& wt, Tensor<float32, CUDA>& yt)
{
	linear_over_tokens(xt, wt, yt);
}

/* ---- Mamba2 neighbours of the convolution ---- */

void hip_tensor_causal_conv1d_update_f32(const Tensor<float32, CUDA>& xt, Tensor<float32, CUDA>& state,
                                         const Tensor<float32, CUDA>& wt, const Tensor<float32, CUDA>& bt,
                                         Tensor<float32, CUDA>& yt)
{
	ABI_CHECK(anygpu_causal_conv1d_silu_update_f32(xt.buffer(), wt.shape[1] > 1 ? state.buffer() : nullptr, wt.buffer(),
	                                               bt.buffer(), yt.buffer(), xt.shape[0], xt.shape[1], wt.shape[1], kNullStream));
}

void hip_tensor_causal_conv1d_update_f16(const Tensor<float16, CUDA>& xt, Tensor<float16, CUDA>& state,
                                         const Tensor<float16, CUDA>& wt, const Tensor<float16, CUDA>& bt,
                                         Tensor<float16, CUDA>& yt)
{
	ABI_CHECK(anygpu_causal_conv1d_silu_update_f16(xt.buffer(), wt.shape[1] > 1 ? state.buffer() : nullptr, wt.buffer(),
	                                               bt.buffer(), yt.buffer(), xt.shape[0], xt.shape[1], wt.shape[1], kNullStream));
}

namespace {

// rows of wt.numel() contiguous elements; a default-constructed zt (no axes, no buffer) means "no gate"
template <typename T>
void rms_norm_dispatch(const Tensor<T, CUDA>& xt, const Tensor<T, CUDA>& zt, const Tensor<T, CUDA>& wt,
                       float32 eps, bool zero_centered, Tensor<T, CUDA>& yt)
{
	const int64 cols = wt.numel();
	const int64 rows = cols > 0 ? xt.numel() / cols : 0;
	const T* gate = zt.dim > 0 ? zt.buffer() : nullptr;
	if constexpr (std::is_same_v<T, float32>)
		ABI_CHECK(anygpu_gated_rmsnorm_f32(xt.buffer(), gate, wt.buffer(), yt.buffer(), rows, cols, eps, zero_centered ? 1 : 0, kNullStream));
	else
		ABI_CHECK(anygpu_gated_rmsnorm_f16(xt.buffer(), gate, wt.buffer(), yt.buffer(), rows, cols, eps, zero_centered ? 1 : 0, kNullStream));
}

}  // namespace

void cu_tensor_rms_norm_f32(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA> wt, const float32 eps,
                            const bool zero_centered, Tensor<float32, CUDA>& yt)
{
	rms_norm_dispatch(xt, Tensor<float32, CUDA>(), wt, eps, zero_centered, yt);
}

void cu_tensor_rms_norm_f32_v1(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA> wt, const float32 eps,
                               const bool zero_centered, Tensor<float32, CUDA>& yt)
{
	rms_norm_dispatch(xt, Tensor<float32, CUDA>(), wt, eps, zero_centered, yt);
}

void hip_tensor_gated_rms_norm_f32(const Tensor<float32, CUDA>& xt, const Tensor<float32, CUDA>& zt, const Tensor<float32, CUDA>& wt,
                                   const float32 eps, const bool zero_centered, Tensor<float32, CUDA>& yt)
{
	rms_norm_dispatch(xt, zt, wt, eps, zero_centered, yt);
}

void hip_tensor_gated_rms_norm_f16(const Tensor<float16, CUDA>& xt, const Tensor<float16, CUDA>& zt, const Tensor<float16, CUDA>& wt,
                                   const float32 eps, const bool zero_centered, Tensor<float16, CUDA>& yt)
{
	rms_norm_dispatch(xt, zt, wt, eps, zero_centered, yt);
}

/* ---- fused attention ---- */

void hip_flash_sdpa_fwd_f16(const SoftmaxPrologue& prologue, const Tensor<float16, CUDA>& qt, const Tensor<float16, CUDA>& kt,
                            const Tensor<float16, CUDA>& vt, Tensor<float16, CUDA>& yt)
{
	const int64 dim = qt.dim;
	const int64 n_q = qt.shape[dim - 2], d = qt.shape[dim - 1], n_k = kt.shape[dim - 2];
	const int64 heads = dim >= 3 ? qt.shape[dim - 3] : 1, kv_heads = dim >= 3 ? kt.shape[dim - 3] : 1;
	const int64 batch_heads = (n_q * d) > 0 ? qt.numel() / (n_q * d) : 0;
	ABI_CHECK(anygpu_sdp_attention_fwd_f16(qt.buffer(), kt.buffer(), vt.buffer(), yt.buffer(), batch_heads,
	                                       kv_heads > 0 ? heads / kv_heads : 1, n_q, n_k, d, prologue.alpha, prologue.softcap,
	                                       prologue.causal ? 1 : 0, prologue.window, kNullStream));
}

void hip_flash_sdpa_fwd_f32(const SoftmaxPrologue& prologue, const Tensor<float32, CUDA>& qt, const Tensor<float32, CUDA>& kt,
                            const Tensor<float32, CUDA>& vt, Tensor<float32, CUDA>& yt)
{
	const int64 dim = qt.dim;
	const int64 n_q = qt.shape[dim - 2], d = qt.shape[dim - 1], n_k = kt.shape[dim - 2];
	const int64 heads = dim >= 3 ? qt.shape[dim - 3] : 1, kv_heads = dim >= 3 ? kt.shape[dim - 3] : 1;
	const int64 batch_heads = (n_q * d) > 0 ? qt.numel() / (n_q * d) : 0;
	ABI_CHECK(anygpu_sdp_attention_fwd_f32(qt.buffer(), kt.buffer(), vt.buffer(), yt.buffer(), batch_heads,
	                                       kv_heads > 0 ? heads / kv_heads : 1, n_q, n_k, d, prologue.alpha, prologue.softcap,
	                                       prologue.causal ? 1 : 0, prologue.window, kNullStream));
}

void hip_flash_sdpa_fwd_masked_f32(const float32 alpha, const Tensor<float32, CUDA>& qt, const Tensor<float32, CUDA>& kt,
                                   const Tensor<float32, CUDA>& vt, const Tensor<float32, CUDA>& mask, Tensor<float32, CUDA>& yt)
{
	const int64 dim = qt.dim;
	const int64 n_q = qt.shape[dim - 2], d = qt.shape[dim - 1], n_k = kt.shape[dim - 2];
	const int64 batch_heads = (n_q * d) > 0 ? qt.numel() / (n_q * d) : 0;
	ABI_CHECK(anygpu_sdp_attention_fwd_masked_f32(qt.buffer(), kt.buffer(), vt.buffer(), mask.buffer(), yt.buffer(), batch_heads, 1,
	                                              n_q, n_k, d, n_k, alpha, 0.0f, kNullStream));
}

void hip_flash_sdpa_fwd_masked_f16(const float32 alpha, const Tensor<float16, CUDA>& qt, const Tensor<float16, CUDA>& kt,
                                   const Tensor<float16, CUDA>& vt, const Tensor<float16, CUDA>& mask, Tensor<float16, CUDA>& yt)
{
	const int64 dim = qt.dim;
	const int64 n_q = qt.shape[dim - 2], d = qt.shape[dim - 1], n_k = kt.shape[dim - 2];
	const int64 batch_heads = (n_q * d) > 0 ? qt.numel() / (n_q * d) : 0;
	ABI_CHECK(anygpu_sdp_attention_fwd_masked_f16(qt.buffer(), kt.buffer(), vt.buffer(), mask.buffer(), yt.buffer(), batch_heads, 1,
	                                              n_q, n_k, d, n_k, alpha, 0.0f, kNullStream));
}

void cu_flash_sdpa_fwd_d256_v1(const float32 alpha, const Tensor<float32, CUDA>& qt, const Tensor<float32, CUDA>& kt,
                               const Tensor<float32, CUDA>& vt, Tensor<float32, CUDA>& yt)
{
	SoftmaxPrologue p;
	p.alpha = alpha;
	hip_flash_sdpa_fwd_f32(p, qt, kt, vt, yt);
}

namespace {

struct AttentionShape
{
	int64 batch_heads, q_per_kv, n_q, n_k, d;
};

template <typename T>
AttentionShape attention_shape(const Tensor<T, CUDA>& qt, const Tensor<T, CUDA>& kt)
{
	const int64 dim = qt.dim;
	AttentionShape s;
	s.n_q = qt.shape[dim - 2];
	s.d = qt.shape[dim - 1];
	s.n_k = kt.shape[dim - 2];
	const int64 heads = dim >= 3 ? qt.shape[dim - 3] : 1, kv_heads = dim >= 3 ? kt.shape[dim - 3] : 1;
	s.q_per_kv = kv_heads > 0 ? heads / kv_heads : 1;
	s.batch_heads = (s.n_q * s.d) > 0 ? qt.numel() / (s.n_q * s.d) : 0;
	return s;
}

}  // namespace

bool hip_flash_sdpa_decode_applies(const Tensor<float16, CUDA>& qt, const Tensor<float16, CUDA>& kt)
{
	const AttentionShape s = attention_shape(qt, kt);
	// few rows per key / value head and enough keys for the split to pay; up to 128 rows of up to 16 queries per head
	// where the fused form (a block per head and 128 queries) would leave half of the chip idle
	const int64 rows = s.q_per_kv * s.n_q;
	if (rows < 1 || s.n_k < 256) return false;
	return rows <= 16 || (rows <= 128 && s.n_q <= 16 && s.batch_heads <= 128);
}

int64 hip_flash_sdpa_decode_workspace_floats(const SoftmaxPrologue& prologue, const Tensor<float16, CUDA>& qt,
                                             const Tensor<float16, CUDA>& kt)
{
	const AttentionShape s = attention_shape(qt, kt);
	const int64 bytes = anygpu_sdp_attention_decode_workspace_bytes(s.batch_heads, s.q_per_kv, s.n_q, s.n_k, s.d,
	                                                                prologue.causal ? 1 : 0, prologue.window);
	if (bytes < 0) check_abi(static_cast<int>(bytes), "anygpu_sdp_attention_decode_workspace_bytes", __FILE__, __LINE__);
	return (bytes + 3) / 4;
}

void hip_flash_sdpa_decode_f16(const SoftmaxPrologue& prologue, const Tensor<float16, CUDA>& qt, const Tensor<float16, CUDA>& kt,
                               const Tensor<float16, CUDA>& vt, Tensor<float32, CUDA>& workspace, Tensor<float16, CUDA>& yt)
{
	const AttentionShape s = attention_shape(qt, kt);
	ABI_CHECK(anygpu_sdp_attention_decode_f16(qt.buffer(), kt.buffer(), vt.buffer(), yt.buffer(), workspace.buffer(),
	                                          workspace.numel() * static_cast<int64>(sizeof(float32)), s.batch_heads, s.q_per_kv,
	                                          s.n_q, s.n_k, s.d, prologue.alpha, prologue.softcap, prologue.causal ? 1 : 0,
	                                          prologue.window, kNullStream));
}

bool hip_flash_sdpa_decode_applies(const Tensor<float32, CUDA>& qt, const Tensor<float32, CUDA>& kt)
{
	const AttentionShape s = attention_shape(qt, kt);
	const int64 rows = s.q_per_kv * s.n_q;
	if (rows < 1 || s.n_k < 256) return false;
	return rows <= 16 || (rows <= 128 && s.n_q <= 16 && s.batch_heads <= 128);
}

int64 hip_flash_sdpa_decode_workspace_floats(const SoftmaxPrologue& prologue, const Tensor<float32, CUDA>& qt,
                                             const Tensor<float32, CUDA>& kt)
{
	const AttentionShape s = attention_shape(qt, kt);
	const int64 bytes = anygpu_sdp_attention_decode_f32_workspace_bytes(s.batch_heads, s.q_per_kv, s.n_q, s.n_k, s.d,
	                                                                    prologue.causal ? 1 : 0, prologue.window);
	if (bytes < 0) check_abi(static_cast<int>(bytes), "anygpu_sdp_attention_decode_f32_workspace_bytes", __FILE__, __LINE__);
	return (bytes + 3) / 4;
}

void hip_flash_sdpa_decode_f32(const SoftmaxPrologue& prologue, const Tensor<float32, CUDA>& qt, const Tensor<float32, CUDA>& kt,
                               const Tensor<float32, CUDA>& vt, Tensor<float32, CUDA>& workspace, Tensor<float32, CUDA>& yt)
{
	const AttentionShape s = attention_shape(qt, kt);
	ABI_CHECK(anygpu_sdp_attention_decode_f32(qt.buffer(), kt.buffer(), vt.buffer(), yt.buffer(), workspace.buffer(),
	                                          workspace.numel() * static_cast<int64>(sizeof(float32)), s.batch_heads, s.q_per_kv,
	                                          s.n_q, s.n_k, s.d, prologue.alpha, prologue.softcap, prologue.causal ? 1 : 0,
	                                          prologue.window, kNullStream));
}
