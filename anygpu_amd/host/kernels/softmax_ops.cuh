// GPU softmax launchers of the host layer (reference: srcs/kernels/cuda/softmax_ops.cuh:6-8).
#ifndef __SOFTMAX_OPS_CUH__
#define __SOFTMAX_OPS_CUH__

#include "tensor.hpp"

/*
  What the attention caller does to a score matrix before softmax, folded into the softmax
  kernel: multiply by alpha, optional logit softcap cap * tanh(s / cap), causal mask (key j
  visible to query i iff j <= i + diag) and sliding window (key j visible iff j > i + diag - window).
  Row r of the matrix belongs to query i = r % q_len (q_len == 0: i = r).
  The default-constructed value is the plain softmax.
*/
struct SoftmaxPrologue
{
	float32 alpha = 1.f;
	float32 softcap = 0.f;   // 0 switches the cap off
	bool causal = false;
	int64 window = 0;        // 0 switches the window off
	int64 q_len = 0;
	int64 diag = 0;
};

void cu_tensor_softmax_f32(
	const Tensor<float32, CUDA>& x,
	Tensor<float32, CUDA>& y);

/* Additions without a counterpart in the reference: half precision and the fused prologue. */
void hip_tensor_softmax_f16(
	const Tensor<float16, CUDA>& x,
	Tensor<float16, CUDA>& y);

void hip_tensor_softmax_fused_f32(
	const Tensor<float32, CUDA>& x,
	const SoftmaxPrologue& prologue,
	Tensor<float32, CUDA>& y);

void hip_tensor_softmax_fused_f16(
	const Tensor<float16, CUDA>& x,
	const SoftmaxPrologue& prologue,
	Tensor<float16, CUDA>& y);

/*
  y[r, :] = softmax(alpha * x[r, :] + mask[r % q_len, :]); mask is a dense [q_len, cols] additive
  matrix (any leading axes of extent 1), x and y dense [rows, cols].
*/
template<typename dtype>
void hip_tensor_softmax_masked(
	const Tensor<dtype, CUDA>& x,
	const Tensor<dtype, CUDA>& mask,
	const float32 alpha,
	const int64 q_len,
	Tensor<dtype, CUDA>& y);

#endif  // __SOFTMAX_OPS_CUH__
