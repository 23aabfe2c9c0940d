// Row softmax over the last axis of a 2-D tensor (reference interface: srcs/ops/softmax_ops.hpp:15-106).
// Tensor<T, CPU> runs the host loops; Tensor<T, CUDA> runs the gfx950 kernel, optionally with the
// attention prologue (scale, softcap, causal / sliding-window mask) fused in.
#ifndef __SOFTMAX_OPS__
#define __SOFTMAX_OPS__

#include "softmax_ops.cuh"

#include "tensor.hpp"
#include "core_concepts.hpp"

/*
  Host softmax.  Per row: running maximum; e = (dtype)exp((double)(x - max)) stored to y while
  the sum grows left to right in dtype; then every e is multiplied by (dtype)1 / sum.
  Honours the strides of x.
*/
template<PreciseFloatType dtype>
inline Tensor<dtype, CPU> tensor_softmax(const Tensor<dtype, CPU>& x)
{
	ACASSERT(x.dim == 2, "softmax expects 2 dimensional tensors");

	const int64 m = x.shape[0];
	const int64 n = x.shape[1];
	Tensor<dtype, CPU> y(std::vector<int64>({ m, n }));

	const dtype* x_data = x.buffer();
	dtype* y_data = y.buffer();
	const int64 xs_r = x.stride[0], xs_c = x.stride[1];
	const int64 ys_r = y.stride[0], ys_c = y.stride[1];

	for (int64 r = 0; r < m; ++r)
	{
		const dtype* xr = x_data + r * xs_r;
		dtype* yr = y_data + r * ys_r;

		dtype row_max = xr[0];
		for (int64 c = 1; c < n; ++c)
		{
			const dtype v = xr[c * xs_c];
			if (v > row_max) row_max = v;
		}

		dtype total = 0;
		for (int64 c = 0; c < n; ++c)
		{
			const dtype shifted = xr[c * xs_c] - row_max;
			const dtype e = static_cast<dtype>(std::exp(static_cast<double>(shifted)));
			yr[c * ys_c] = e;
			total = (c == 0) ? e : total + e;
		}

		const dtype inv_total = static_cast<dtype>(1.0) / total;
		for (int64 c = 0; c < n; ++c)
		{
			yr[c * ys_c] = yr[c * ys_c] * inv_total;
		}
	}

	return y;
}

/* GPU softmax; float32 as in the reference, float16 in addition (float32 internals). */
template<typename dtype>
inline Tensor<dtype, CUDA> tensor_softmax(const Tensor<dtype, CUDA>& x)
{
	ACASSERT(x.dim == 2, "softmax expects 2 dimensional tensors");
	Tensor<dtype, CUDA> y(std::vector<int64>({ x.shape[0], x.shape[1] }));

	if constexpr (std::is_same_v<dtype, float32>)
	{
		cu_tensor_softmax_f32(x, y);
	}
	else if constexpr (std::is_same_v<dtype, float16>)
	{
		hip_tensor_softmax_f16(x, y);
	}
	else
	{
		static_assert(std::is_same_v<dtype, float32>, "Unsupported data type");
	}
	return y;
}

/*
  Addition without a counterpart in the reference: softmax of the scaled, optionally capped and
  masked scores in one kernel; equivalent to tensor_softmax(tensor_add(tensor_mul(x, alpha), mask))
  with the mask the prologue describes (and the softcap between the two when it is on).
*/
template<typename dtype>
inline Tensor<dtype, CUDA> tensor_softmax(const Tensor<dtype, CUDA>& x, const SoftmaxPrologue& prologue)
{
	ACASSERT(x.dim == 2, "softmax expects 2 dimensional tensors");
	ACASSERT(prologue.window >= 0, "sliding window can not be negative");
	Tensor<dtype, CUDA> y(std::vector<int64>({ x.shape[0], x.shape[1] }));

	if constexpr (std::is_same_v<dtype, float32>)
	{
		hip_tensor_softmax_fused_f32(x, prologue, y);
	}
	else
	{
		static_assert(std::is_same_v<dtype, float16>, "Unsupported data type");
		hip_tensor_softmax_fused_f16(x, prologue, y);
	}
	return y;
}

#endif  // __SOFTMAX_OPS__
