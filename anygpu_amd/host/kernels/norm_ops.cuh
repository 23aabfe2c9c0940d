// GPU RMS-norm launchers of the host layer (reference: srcs/kernels/cuda/norm_ops.cuh:14-37).
#ifndef __NORM_OPS_CUH__
#define __NORM_OPS_CUH__

#include "tensor.hpp"

/* y = x / sqrt(mean(x^2) + eps) * (w + (zero_centered ? 1 : 0)) over regions of wt.numel() contiguous elements. */
void cu_tensor_rms_norm_f32(
	const Tensor<float32, CUDA>& xt,
	const Tensor<float32, CUDA> wt,
	const float32 eps,
	const bool zero_centered,
	Tensor<float32, CUDA>& yt);

/* The reference keeps a second, tuned kernel under this name; both names run the same kernel here. */
void cu_tensor_rms_norm_f32_v1(
	const Tensor<float32, CUDA>& xt,
	const Tensor<float32, CUDA> wt,
	const float32 eps,
	const bool zero_centered,
	Tensor<float32, CUDA>& yt);

/* Additions without a counterpart in the reference: the gate x * silu(z) applied inside the norm kernel
   (zt may be a default-constructed tensor: no gate), and half precision tensors (float32 internals). */
void hip_tensor_gated_rms_norm_f32(
	const Tensor<float32, CUDA>& xt,
	const Tensor<float32, CUDA>& zt,
	const Tensor<float32, CUDA>& wt,
	const float32 eps,
	const bool zero_centered,
	Tensor<float32, CUDA>& yt);

void hip_tensor_gated_rms_norm_f16(
	const Tensor<float16, CUDA>& xt,
	const Tensor<float16, CUDA>& zt,
	const Tensor<float16, CUDA>& wt,
	const float32 eps,
	const bool zero_centered,
	Tensor<float16, CUDA>& yt);

#endif  // __NORM_OPS_CUH__
