// Gemma2 output head: logits against the (tied) embedding table, squashed into (-cap, cap).
// Reference interface: srcs/models/gemma2/gemma_linsoftcap.hpp:12-41 (GPU only there as well).
#ifndef __GEMMA_LIN_SOFTCAP__
#define __GEMMA_LIN_SOFTCAP__

#include "gemma_linsoftcap.cuh"

#include "tensor.hpp"
#include "core_concepts.hpp"

template<FloatingPointType dtype>
inline Tensor<dtype, CUDA> tensor_gemma_linear_softcap(
	const Tensor<dtype, CUDA>& xt,  // (batch, seq_len, hidden)
	const Tensor<dtype, CUDA>& wt,  // (vocab, hidden)
	const dtype final_softcapping)
{
	static_assert(std::is_same_v<dtype, float32>, "Unsupported data types");
	ACASSERT(xt.dim == 3, "xt should be 3 dim");
	ACASSERT(wt.dim == 2 && xt.shape[2] == wt.shape[1], "hidden size should match for xt and wt");

	Tensor<dtype, CUDA> yt(std::vector<int64>{ xt.shape[0], xt.shape[1], wt.shape[0] });
	cu_tensor_gemma_linear_softcap_f32(xt, wt, final_softcapping, yt);
	return yt;
}

#endif  // __GEMMA_LIN_SOFTCAP__
