// Elementwise scale and add on host tensors.  On the GPU these two steps sit between the score
// matmul and the softmax of an attention block; there they are folded into the softmax kernel
// (SoftmaxPrologue) instead of running as kernels of their own, so only the host forms exist
// here.  Reference: srcs/ops/binary_ops.hpp:11-29 (add), :61-76 (mul by scalar), :103-121 (mul, elementwise).
#ifndef __BINARY_OPS__
#define __BINARY_OPS__

#include "tensor.hpp"
#include "core_concepts.hpp"

template<NotHalfFloatType dtype>
inline Tensor<dtype, CPU> tensor_add(const Tensor<dtype, CPU>& lhs, const Tensor<dtype, CPU>& rhs)
{
	ACASSERT(elementwise_compatible(lhs, rhs) == true, "tensors are not elementwise compatible");
	Tensor<dtype, CPU> res(lhs.dim, lhs.shape, lhs.stride);
	const int64 length = lhs.size();
	const dtype* a = lhs.buffer();
	const dtype* b = rhs.buffer();
	dtype* r = res.buffer();
	for (int64 ix = 0; ix < length; ++ix) r[ix] = a[ix] + b[ix];
	return res;
}

template<NotHalfFloatType dtype>
inline Tensor<dtype, CPU> tensor_mul(const Tensor<dtype, CPU>& lhs, const dtype rhs)
{
	Tensor<dtype, CPU> res(lhs.dim, lhs.shape, lhs.stride);
	const int64 length = lhs.size();
	const dtype* a = lhs.buffer();
	dtype* r = res.buffer();
	for (int64 ix = 0; ix < length; ++ix) r[ix] = a[ix] * rhs;
	return res;
}

template<NotHalfFloatType dtype>
inline Tensor<dtype, CPU> tensor_mul(const Tensor<dtype, CPU>& lhs, const Tensor<dtype, CPU>& rhs)
{
	ACASSERT(elementwise_compatible(lhs, rhs) == true, "tensors are not elementwise compatible");
	Tensor<dtype, CPU> res(lhs.dim, lhs.shape, lhs.stride);
	const int64 length = lhs.size();
	const dtype* a = lhs.buffer();
	const dtype* b = rhs.buffer();
	dtype* r = res.buffer();
	for (int64 ix = 0; ix < length; ++ix) r[ix] = a[ix] * b[ix];
	return res;
}

#endif  // __BINARY_OPS__
