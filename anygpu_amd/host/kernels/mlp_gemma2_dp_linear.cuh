// Launchers of the Gemma2 MLP's down projection
// (reference: srcs/kernels/cuda/mlp_gemma2_dp_linear.cuh:6-20).
#ifndef __MLP_GEMMA2_DP_LINEAR_CUH__
#define __MLP_GEMMA2_DP_LINEAR_CUH__

#include "tensor.hpp"

/*
  yt = xt * wt_dp: xt (batch, seq_len, intermediate), wt_dp (intermediate, hidden), yt (batch, seq_len, hidden).
  The reference fixes 9216 and 2304 in its kernels; here the sizes come from the weight's shape.  Both names
  (two generations of the reference's tiling) run the fp32 MFMA GEMM.
*/
void cu_mlp_gemma2_dp_linear_f32_v1(
	const Tensor<float32, CUDA>& xt,
	const Tensor<float32, CUDA>& wt_dp,
	Tensor<float32, CUDA>& yt);

void cu_mlp_gemma2_dp_linear_f32_v4(
	const Tensor<float32, CUDA>& xt,
	const Tensor<float32, CUDA>& wt_dp,
	Tensor<float32, CUDA>& yt);

#endif  // __MLP_GEMMA2_DP_LINEAR_CUH__
