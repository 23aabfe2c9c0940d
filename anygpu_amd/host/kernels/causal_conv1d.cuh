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

/* Decode step: xt (batch, dims) is the newest sample of every row, state (batch, dims, width - 1) the
   samples in front of it, oldest first; the state is shifted by one and takes xt.  No counterpart in
   the reference, which has the whole-sequence form only. */
void hip_tensor_causal_conv1d_update_f32(
	const Tensor<float32, CUDA>& xt,
	Tensor<float32, CUDA>& state,
	const Tensor<float32, CUDA>& wt,
	const Tensor<float32, CUDA>& bt,
	Tensor<float32, CUDA>& yt);

void hip_tensor_causal_conv1d_update_f16(
	const Tensor<float16, CUDA>& xt,
	Tensor<float16, CUDA>& state,
	const Tensor<float16, CUDA>& wt,
	const Tensor<float16, CUDA>& bt,
	Tensor<float16, CUDA>& yt);

#endif  // __CAUSAL_CONV1D_CUH__
