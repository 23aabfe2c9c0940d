// GPU matmul launchers of the host layer.  Names and signatures are those of the reference's
// srcs/kernels/cuda/mm_ops.cuh:10-64; each forwards to the gfx950 MFMA kernels through the C ABI
// (include/anygpu_hip.h).  Launchers take sizes from shape[] and pointers from buffer() and
// expect densely packed row-major operands, as the reference's do; they return after queueing
// the work on the null stream and stop the process on any error.
#ifndef __MM_OPS_CUH__
#define __MM_OPS_CUH__

#include "tensor.hpp"

/* C = lhs * rhs, float32, any shape. */
void cu_tensor_mm_f32_opt0(
	const Tensor<float32, CUDA>& lhs,
	const Tensor<float32, CUDA>& rhs,
	const Tensor<float32, CUDA>& out);

/* out = xt * wt + bt (bias per output column), float32, any shape. */
void cu_tensor_gemm_f32_opt0(
	const Tensor<float32, CUDA>& xt,
	const Tensor<float32, CUDA>& wt,
	const Tensor<float32, CUDA>& bt,
	const Tensor<float32, CUDA>& out);

namespace opt1
{
	/* float32 matmul; the reference variant required multiples of 64, this one takes any shape. */
	void cu_tensor_mm_f32(
		const Tensor<float32, CUDA>& lhs,
		const Tensor<float32, CUDA>& rhs,
		const Tensor<float32, CUDA>& out);
}

namespace opt2
{
	/* float16 matmul with float32 accumulation on the matrix cores; any shape. */
	void cu_tensor_mm_f16(
		const Tensor<float16, CUDA>& lhs,
		const Tensor<float16, CUDA>& rhs,
		const Tensor<float16, CUDA>& out);
}

/*
  Additions without a counterpart in the reference: the right operand stored [N, K]
  ("column-major B", the [out, in] layout weights arrive in).  out[M, N] = lhs[M, K] * rhs_nk^T.
*/
void hip_tensor_mm_nt_f16(
	const Tensor<float16, CUDA>& lhs,
	const Tensor<float16, CUDA>& rhs_nk,
	const Tensor<float16, CUDA>& out);

void hip_tensor_mm_nt_f32(
	const Tensor<float32, CUDA>& lhs,
	const Tensor<float32, CUDA>& rhs_nk,
	const Tensor<float32, CUDA>& out);

/*
  `batch` products of one shape in one launch over densely packed operands:
  out[i] (m x n) = lhs[i] (m x k) * rhs[i], rhs[i] stored [k, n] or, with rhs_is_nk, [n, k].
  The tensors may have any number of leading axes; only their buffers are used.
*/
template<typename dtype>
void hip_tensor_mm_batched(
	const Tensor<dtype, CUDA>& lhs,
	const Tensor<dtype, CUDA>& rhs,
	const Tensor<dtype, CUDA>& out,
	const int64 batch, const int64 m, const int64 n, const int64 k,
	const bool rhs_is_nk);

#endif  // __MM_OPS_CUH__
