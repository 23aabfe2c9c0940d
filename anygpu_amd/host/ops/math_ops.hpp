// Elementwise activation on host tensors.  On the GPU the one caller on this path (the Gemma2 MLP)
// has the activation folded into the epilogue of its projection kernel, so only the host form
// exists here.  Reference: srcs/ops/math_ops.hpp:16-35 (tensor_silu), :55-93 (tensor_gelu, exact and tanh form).
#ifndef __MATH_OPS__
#define __MATH_OPS__

#include "tensor.hpp"
#include "core_concepts.hpp"

#include <cmath>

/* silu(x) = x / (1 + exp(-x)), evaluated in dtype. */
template<PreciseFloatType dtype>
inline Tensor<dtype, CPU> tensor_silu(const Tensor<dtype, CPU>& xt)
{
	Tensor<dtype, CPU> yt(xt.dim, xt.shape);
	const dtype* x_data = xt.buffer();
	dtype* y_data = yt.buffer();
	const int64 length = xt.size();
	for (int64 k = 0; k < length; ++k) y_data[k] = x_data[k] / (static_cast<dtype>(1.0) + std::exp(-x_data[k]));
	return yt;
}

/*
  gelu(x) = x / 2 * (1 + erf(x / sqrt(2)));  with approx: x / 2 * (1 + tanh(sqrt(2 / pi) * (x + 0.044715 x^3))).
  Everything is evaluated in dtype (constants cast to it first).
*/
template<PreciseFloatType dtype>
inline Tensor<dtype, CPU> tensor_gelu(const Tensor<dtype, CPU>& xt, const bool approx = false)
{
	Tensor<dtype, CPU> yt(xt.dim, xt.shape);
	const dtype* x_data = xt.buffer();
	dtype* y_data = yt.buffer();
	const int64 length = xt.size();
	const dtype half = static_cast<dtype>(0.5), one = static_cast<dtype>(1.0);
	const dtype inv_sqrt2 = one / std::sqrt(static_cast<dtype>(2.0));
	const dtype slope = static_cast<dtype>(std::sqrt(2.0 / 3.14159265358979323846));
	const dtype cubic = static_cast<dtype>(0.044715);
	for (int64 k = 0; k < length; ++k)
	{
		const dtype x = x_data[k];
		const dtype gate = approx ? std::tanh(slope * (x + cubic * x * x * x)) : std::erf(x * inv_sqrt2);
		y_data[k] = x * half * (one + gate);
	}
	return yt;
}

#endif  // __MATH_OPS__
