// Launcher of the q / k / v / o projections of the Gemma2 attention block
// (reference: srcs/kernels/cuda/sdpa_gemma2_linear.cuh:6-11).
#ifndef __SDPA_GEMMA2_LINEAR_CUH__
#define __SDPA_GEMMA2_LINEAR_CUH__

#include "tensor.hpp"

/* yt = xt * wt: xt (batch, seq_len, in_features), wt (in_features, out_features), yt (batch, seq_len, out_features). */
void cu_sdpa_gemma2_linear_f32_v1(
	const Tensor<float32, CUDA>& xt,
	const Tensor<float32, CUDA>& wt,
	Tensor<float32, CUDA>& yt);

#endif  // __SDPA_GEMMA2_LINEAR_CUH__
