// Gated RMS norm of the Zamba2 Mamba2 mixer: rms_norm(x * silu(z)) * w over the last axis.
// Reference interface: srcs/models/zamba2/zamba_gated_rmsnorm.hpp:9-23.
#ifndef __ZAMBA_GATED_RMSNORM__
#define __ZAMBA_GATED_RMSNORM__

#include "tensor.hpp"
#include "core_concepts.hpp"
#include "ops.hpp"

/*
  As in the reference one group spans the row; gsize is accepted and not used.  A host tensor takes the
  three operator calls, a GPU tensor one kernel that applies the gate while it reads the row.
*/
template<FloatingPointType dtype, Device device>
inline Tensor<dtype, device> tensor_zamba_gated_rmsnorm(
	const Tensor<dtype, device>& xt,
	const Tensor<dtype, device>& zt,
	const Tensor<dtype, device>& wt,
	const int gsize,
	const dtype eps)
{
	(void)gsize;
	ACASSERT(elementwise_compatible(xt, zt) == true, "tensors are not elementwise compatible");
	if constexpr (device == CUDA)
	{
		ACASSERT(wt.dim == 1 && xt.shape[xt.dim - 1] == wt.shape[0], "wt shape is incorrect");
		Tensor<dtype, CUDA> yt(xt.dim, xt.shape);
		if constexpr (std::is_same_v<dtype, float32>)
			hip_tensor_gated_rms_norm_f32(xt, zt, wt, eps, false, yt);
		else
		{
			static_assert(std::is_same_v<dtype, float16>, "Unsupported data types");
			hip_tensor_gated_rms_norm_f16(xt, zt, wt, static_cast<float32>(eps), false, yt);
		}
		return yt;
	}
	else
	{
		auto silu_zt = tensor_silu(zt);
		auto gated = tensor_mul(xt, silu_zt);
		return tensor_rms_norm(gated, -1, wt, eps);
	}
}

#endif  // __ZAMBA_GATED_RMSNORM__
