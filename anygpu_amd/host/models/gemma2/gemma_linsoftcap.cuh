// Launcher of the Gemma2 output head with logit soft-capping
// (reference: srcs/models/gemma2/gemma_linsoftcap.cuh:6-10).
#ifndef __GEMMA_LIN_SOFTCAP_CUH__
#define __GEMMA_LIN_SOFTCAP_CUH__

#include "tensor.hpp"

/* yt[b, s, v] = cap * tanh((sum_h xt[b, s, h] * wt[v, h]) / cap); wt is (vocab, hidden). */
void cu_tensor_gemma_linear_softcap_f32(
	const Tensor<float32, CUDA>& xt,
	const Tensor<float32, CUDA>& wt,
	const float32 final_softcapping,
	Tensor<float32, CUDA>& yt);

#endif  // __GEMMA_LIN_SOFTCAP_CUH__
