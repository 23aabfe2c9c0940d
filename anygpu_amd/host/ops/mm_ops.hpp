// Matrix multiplication operators: tensor_mm, tensor_gemm (+bias), tensor_linear.
// Overloaded on the device tag: Tensor<T, CPU> runs the plain host loops, Tensor<T, CUDA> runs the
// gfx950 MFMA kernels.  A GPU tensor never takes the host path and the other way round.
// Reference interface: srcs/ops/mm_ops.hpp:11-232.
#ifndef __MM_OPS__
#define __MM_OPS__

#include "mm_ops.cuh"
#include "shape_ops.hpp"

#include "tensor.hpp"
#include "core_concepts.hpp"

namespace mm_detail {

/*
  res[r, c] = bias[c] + sum over l (ascending) of lhs[r, l] * rhs[l, c], every operand addressed
  through its own strides.  The product is formed in dtype; the running sum is float32
  whatever dtype is, and the bias (when present) is added to the finished sum.
*/
template<typename dtype>
inline void strided_matmul(const Tensor<dtype, CPU>& lhs, const Tensor<dtype, CPU>& rhs, const dtype* bias,
                           Tensor<dtype, CPU>& res)
{
	const int64 m = lhs.shape[0], k = lhs.shape[1], n = rhs.shape[1];
	const dtype* a = lhs.buffer();
	const dtype* b = rhs.buffer();
	dtype* out = res.buffer();
	for (int64 r = 0; r < m; ++r)
	{
		const dtype* a_row = a + r * lhs.stride[0];
		for (int64 c = 0; c < n; ++c)
		{
			const dtype* b_col = b + c * rhs.stride[1];
			float32 acc = 0.f;
			for (int64 l = 0; l < k; ++l)
			{
				acc += a_row[l * lhs.stride[1]] * b_col[l * rhs.stride[0]];
			}
			dtype value = static_cast<dtype>(acc);
			if (bias != nullptr) value = static_cast<dtype>(acc + bias[c]);
			out[r * res.stride[0] + c * res.stride[1]] = value;
		}
	}
}

template<typename dtype, Device device>
inline Tensor<dtype, device> result_like(const int64 m, const int64 n)
{
	return Tensor<dtype, device>(std::vector<int64>({ m, n }));
}

}  // namespace mm_detail


/* ---- tensor_mm: res = lhs * rhs ---- */

template<NotHalfFloatType dtype>
inline void tensor_mm(const Tensor<dtype, CPU>& lhs, const Tensor<dtype, CPU>& rhs, Tensor<dtype, CPU>& res)
{
	ACASSERT(matmul_compatible(lhs, rhs) == true, "matrix multiplication requires compatible matrices");
	ACASSERT(lhs.shape[0] == res.shape[0] && rhs.shape[1] == res.shape[1], "result mtx shape is wrong");
	mm_detail::strided_matmul<dtype>(lhs, rhs, nullptr, res);
}

template<typename dtype>
inline void tensor_mm(const Tensor<dtype, CUDA>& lhs, const Tensor<dtype, CUDA>& rhs, Tensor<dtype, CUDA>& res)
{
	ACASSERT(matmul_compatible(lhs, rhs) == true, "matrix multiplication requires compatible matrices");
	ACASSERT(lhs.shape[0] == res.shape[0] && rhs.shape[1] == res.shape[1], "result mtx shape is wrong");

	if constexpr (std::is_same_v<dtype, float32>)
	{
		cu_tensor_mm_f32_opt0(lhs, rhs, res);
	}
	else if constexpr (std::is_same_v<dtype, float16>)
	{
		opt2::cu_tensor_mm_f16(lhs, rhs, res);
	}
	else
	{
		static_assert(std::is_same_v<dtype, float32>, "Unsupported data type");
	}
}

template<NotHalfFloatType dtype>
inline Tensor<dtype, CPU> tensor_mm(const Tensor<dtype, CPU>& lhs, const Tensor<dtype, CPU>& rhs)
{
	auto res = mm_detail::result_like<dtype, CPU>(lhs.shape[0], rhs.shape[1]);
	tensor_mm(lhs, rhs, res);
	return res;
}

template<typename dtype>
inline Tensor<dtype, CUDA> tensor_mm(const Tensor<dtype, CUDA>& lhs, const Tensor<dtype, CUDA>& rhs)
{
	auto res = mm_detail::result_like<dtype, CUDA>(lhs.shape[0], rhs.shape[1]);
	tensor_mm(lhs, rhs, res);
	return res;
}

/*
  Addition without a counterpart in the reference: right operand given as its [N, K] storage
  (column-major B; the [out, in] layout of a weight matrix), so no transpose pass is needed:
  res[M, N] = lhs[M, K] * rhs_nk^T.  GPU only; on the host the same product is
  tensor_mm(lhs, view of rhs_nk with swapped strides).
*/
template<typename dtype>
inline Tensor<dtype, CUDA> tensor_mm_nt(const Tensor<dtype, CUDA>& lhs, const Tensor<dtype, CUDA>& rhs_nk)
{
	ACASSERT(lhs.dim == 2 && rhs_nk.dim == 2 && lhs.shape[1] == rhs_nk.shape[1],
		"matrix multiplication requires compatible matrices");
	auto res = mm_detail::result_like<dtype, CUDA>(lhs.shape[0], rhs_nk.shape[0]);
	if constexpr (std::is_same_v<dtype, float16>) hip_tensor_mm_nt_f16(lhs, rhs_nk, res);
	else
	{
		static_assert(std::is_same_v<dtype, float32>, "Unsupported data type");
		hip_tensor_mm_nt_f32(lhs, rhs_nk, res);
	}
	return res;
}


/* ---- tensor_gemm: xt * wt + bt, bias per output column ---- */

template<NotHalfFloatType dtype>
inline Tensor<dtype, CPU> tensor_gemm(
	const Tensor<dtype, CPU>& xt,
	const Tensor<dtype, CPU>& wt,
	const Tensor<dtype, CPU>& bt)
{
	ACASSERT(matmul_compatible(xt, wt) == true, "matrix multiplication requires compatible matrices");
	ACASSERT(wt.shape[1] == bt.shape[0], "incorrect bias shape");
	auto res = mm_detail::result_like<dtype, CPU>(xt.shape[0], wt.shape[1]);
	mm_detail::strided_matmul<dtype>(xt, wt, bt.buffer(), res);
	return res;
}

template<typename dtype>
inline Tensor<dtype, CUDA> tensor_gemm(
	const Tensor<dtype, CUDA>& xt,
	const Tensor<dtype, CUDA>& wt,
	const Tensor<dtype, CUDA>& bt)
{
	ACASSERT(matmul_compatible(xt, wt) == true, "matrix multiplication requires compatible matrices");
	ACASSERT(wt.shape[1] == bt.shape[0], "incorrect bias shape");
	static_assert(std::is_same_v<dtype, float32>, "Unsupported data type");
	auto res = mm_detail::result_like<dtype, CUDA>(xt.shape[0], wt.shape[1]);
	cu_tensor_gemm_f32_opt0(xt, wt, bt, res);
	return res;
}


/* ---- tensor_linear: (*, in_features) x (in_features, out_features) [+ (out_features)] ---- */

namespace mm_detail {

template<typename dtype, Device device, typename Product>
inline Tensor<dtype, device> linear_over_rows(const Tensor<dtype, device>& xt, Product&& product)
{
	// fold every leading axis into rows, multiply, unfold again
	const int64 d = xt.dim;
	const int64 cols = xt.shape[d - 1];
	const int64 rows = xt.numel() / cols;
	Tensor<dtype, device> xw = product(tensor_view(xt, { rows, cols }));
	std::vector<int64> y_shape = cvt_array2vector(d, xt.shape);
	y_shape[d - 1] = xw.shape[1];
	return tensor_view(xw, y_shape);
}

}  // namespace mm_detail

template<FloatingPointType dtype, Device device>
inline Tensor<dtype, device> tensor_linear(
	const Tensor<dtype, device>& xt,  // (*, in_features)
	const Tensor<dtype, device>& wt,  // (in_features, out_features)
	const Tensor<dtype, device>& bt)  // (out_features)
{
	return mm_detail::linear_over_rows(xt, [&](const Tensor<dtype, device>& x2d) { return tensor_gemm(x2d, wt, bt); });
}

template<FloatingPointType dtype, Device device>
inline Tensor<dtype, device> tensor_linear(
	const Tensor<dtype, device>& xt,  // (*, in_features)
	const Tensor<dtype, device>& wt)  // (in_features, out_features)
{
	return mm_detail::linear_over_rows(xt, [&](const Tensor<dtype, device>& x2d) { return tensor_mm(x2d, wt); });
}

#endif  // __MM_OPS__
