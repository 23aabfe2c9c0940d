// RMS normalisation.  Reference interface: srcs/ops/norm_ops.hpp:129-225 (tensor_rms_norm).
#ifndef __NORM_OPS__
#define __NORM_OPS__

#include "norm_ops.cuh"

#include "tensor.hpp"
#include "core_concepts.hpp"

#include <cmath>

namespace norm_detail {

// number of elements the weight spans, after checking that it matches the trailing axes from `axis` on
template<typename dtype, Device device>
inline int64 region_size(const Tensor<dtype, device>& xt, const int32 axis, const Tensor<dtype, device>& wt)
{
	const int32 dim = xt.dim;
	ACASSERT((-dim <= axis && axis < dim), "axis is out of range");
	const int32 paxis = (dim + axis) % dim;
	int64 size = 1;
	for (int32 k = paxis; k < dim; ++k)
	{
		ACASSERT(xt.shape[k] == wt.shape[k - paxis], "wt shape is incorrect");
		size *= xt.shape[k];
	}
	return size;
}

}  // namespace norm_detail

/*
  Host loops over contiguous memory: per region the squares are summed left to right in dtype, then
  y = (x / sqrt(mean + eps)) * (w + delta), delta = 1 for zero-centred weights.
*/
template<PreciseFloatType dtype>
inline Tensor<dtype, CPU> tensor_rms_norm(
	const Tensor<dtype, CPU>& xt,
	const int32 axis,
	const Tensor<dtype, CPU> wt,
	const dtype eps,
	const bool zero_centered = false)
{
	const int64 size = norm_detail::region_size(xt, axis, wt);
	Tensor<dtype, CPU> yt(xt.dim, xt.shape);
	const dtype* x_data = xt.buffer();
	const dtype* w_data = wt.buffer();
	dtype* y_data = yt.buffer();
	const dtype delta = zero_centered ? static_cast<dtype>(1.0) : static_cast<dtype>(0.0);
	const int64 regions = size > 0 ? yt.size() / size : 0;
	for (int64 r = 0; r < regions; ++r)
	{
		const dtype* xr = x_data + r * size;
		dtype* yr = y_data + r * size;
		dtype squares = static_cast<dtype>(0);
		for (int64 ix = 0; ix < size; ++ix) squares += xr[ix] * xr[ix];
		const dtype mean = squares / static_cast<dtype>(size);
		for (int64 ix = 0; ix < size; ++ix) yr[ix] = (xr[ix] / std::sqrt(mean + eps)) * (w_data[ix] + delta);
	}
	return yt;
}

/* GPU path; float32 as in the reference, float16 in addition. */
template<FloatingPointType dtype>
inline Tensor<dtype, CUDA> tensor_rms_norm(
	const Tensor<dtype, CUDA>& xt,
	const int32 axis,
	const Tensor<dtype, CUDA> wt,
	const dtype eps,
	const bool zero_centered = false)
{
	norm_detail::region_size(xt, axis, wt);
	Tensor<dtype, CUDA> yt(xt.dim, xt.shape);
	if constexpr (std::is_same_v<dtype, float32>)
	{
		cu_tensor_rms_norm_f32_v1(xt, wt, eps, zero_centered, yt);
	}
	else
	{
		static_assert(std::is_same_v<dtype, float16>, "Unsupported data types");
		hip_tensor_gated_rms_norm_f16(xt, Tensor<float16, CUDA>(), wt, static_cast<float32>(eps), zero_centered, yt);
	}
	return yt;
}

#endif  // __NORM_OPS__
