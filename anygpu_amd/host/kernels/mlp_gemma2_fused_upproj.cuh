// Launchers of the Gemma2 MLP's fused gate / up projection
// (reference: srcs/kernels/cuda/mlp_gemma2_fused_upproj.cuh:6-19).
#ifndef __MLP_GEMMA2_FUSED_UPPROJ_CUH__
#define __MLP_GEMMA2_FUSED_UPPROJ_CUH__

#include "tensor.hpp"

/*
  yt = gelu_tanh(xt * wt_gp) (*) (xt * wt_up), (*) elementwise.
  xt (batch, seq_len, hidden), wt_gp and wt_up (hidden, intermediate), yt (batch, seq_len, intermediate).
  The reference fixes hidden = 2304 and intermediate = 9216 in its kernels; here they come from the
  weight's shape.  Both names run the same kernel: one MFMA tile kernel that reads xt once and keeps
  two accumulator sets, with the activation and the product in its epilogue.
*/
void cu_mlp_gemma2_fused_upproj_f32_v1(
	const Tensor<float32, CUDA>& xt,
	const Tensor<float32, CUDA>& wt_gp,
	const Tensor<float32, CUDA>& wt_up,
	Tensor<float32, CUDA>& yt);

void cu_mlp_gemma2_fused_upproj_f32_v2(
	const Tensor<float32, CUDA>& xt,
	const Tensor<float32, CUDA>& wt_gp,
	const Tensor<float32, CUDA>& wt_up,
	Tensor<float32, CUDA>& yt);

#endif  // __MLP_GEMMA2_FUSED_UPPROJ_CUH__
