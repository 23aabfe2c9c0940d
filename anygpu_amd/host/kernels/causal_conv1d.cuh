// GPU causal conv1d + SiLU launchers of the host layer
// (reference: srcs/kernels/cuda/causal_conv1d.cuh:6-10).
#ifndef __CAUSAL_CONV1D_CUH__
#define __CAUSAL_CONV1D_CUH__

#include "tensor.hpp"

void cu_tensor_causal_conv1d_f32(
	const Tensor<float32, CUDA>& xt,
	const Tensor<float32, CUDA>& wt,
	const Tensor<float32, CUDA>& bt,
	Tensor<float32, CUDA>& yt);

/* Addition without a counterpart in the reference: half precision tensors (float32 internals). */
void hip_tensor_causal_conv1d_f16(
	const Tensor<float16, CUDA>& xt,
	const Tensor<float16, CUDA>& wt,
	const Tensor<float16, CUDA>& bt,
	Tensor<float16, CUDA>& yt);

#endif  // __CAUSAL_CONV1D_CUH__
