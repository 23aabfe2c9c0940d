// Gemma2 MLP: down(act(x Wgate) (*) (x Wup)) with the tanh form of GELU.
// Reference interface: srcs/models/gemma2/gemma_mlp.hpp:12-141 (weights, tensor_gemma_mlp_fused_uprpoj,
// tensor_gemma_mlp_dp_linear, tensor_gemma_mlp).
#ifndef __GEMMA_MLP__
#define __GEMMA_MLP__

#include "mlp_gemma2_fused_upproj.cuh"
#include "mlp_gemma2_dp_linear.cuh"

#include "tensor.hpp"
#include "core_concepts.hpp"
#include "ops.hpp"
#include "dat_file.hpp"

template<FloatingPointType dtype, Device device>
struct GemmaMLPweights
{
	Tensor<dtype, device> gate_proj_weight;  // (hidden, intermediate)
	Tensor<dtype, device> up_proj_weight;    // (hidden, intermediate)
	Tensor<dtype, device> down_proj_weight;  // (intermediate, hidden)

	/* Reads the three matrices from .dat files.  Checkpoints keep them as (out_features, in_features);
	   with transpose they are turned into the (in_features, out_features) form the products take. */
	void load_weights(
		const std::string& path_gate_proj_weight,
		const std::string& path_up_proj_weight,
		const std::string& path_down_proj_weight,
		const bool transpose = true)
	{
		auto fetch = [&](const std::string& path) {
			auto t = load_tensor<dtype>(path);
			return copy_to_device<dtype, CPU, device>(transpose ? tensor_transp(t) : t);
		};
		gate_proj_weight = fetch(path_gate_proj_weight);
		up_proj_weight = fetch(path_up_proj_weight);
		down_proj_weight = fetch(path_down_proj_weight);
	}
};

/*
  variant 0: three operator calls (the path a host tensor takes): linear, gelu, linear, mul.
  variant 1, 2: the fused kernel (GPU tensors only); the two numbers are the reference's names for two
  generations of its fused kernel and select the same kernel here.
*/
template<FloatingPointType dtype, Device device, int variant>
inline Tensor<dtype, device> tensor_gemma_mlp_fused_uprpoj(
	const GemmaMLPweights<dtype, device>& mlp_weights,
	const Tensor<dtype, device>& x)
{
	if constexpr (device == CUDA)
	{
		static_assert(std::is_same_v<dtype, float32>, "Unsupported data types");
		static_assert(variant == 1 || variant == 2, "a GPU tensor takes the fused kernel");
		ACASSERT(x.dim == 3, "x should be 3 dim");
		ACASSERT(elementwise_compatible(mlp_weights.gate_proj_weight, mlp_weights.up_proj_weight),
		         "gate and up weights must have one shape");
		ACASSERT(x.shape[2] == mlp_weights.gate_proj_weight.shape[0], "hidden size should match for x and the weights");
		Tensor<dtype, device> out(std::vector<int64>{ x.shape[0], x.shape[1], mlp_weights.gate_proj_weight.shape[1] });
		if constexpr (variant == 1)
			cu_mlp_gemma2_fused_upproj_f32_v1(x, mlp_weights.gate_proj_weight, mlp_weights.up_proj_weight, out);
		else
			cu_mlp_gemma2_fused_upproj_f32_v2(x, mlp_weights.gate_proj_weight, mlp_weights.up_proj_weight, out);
		return out;
	}
	else
	{
		auto gated_x = tensor_linear(x, mlp_weights.gate_proj_weight);
		auto act_gated_x = tensor_gelu(gated_x, true);
		auto up_x = tensor_linear(x, mlp_weights.up_proj_weight);
		return tensor_mul(act_gated_x, up_x);
	}
}

/*
  Down projection.  variant 0: tensor_linear (any device); variant 1, 4: the reference's names for two
  generations of its specialised kernel, the fp32 MFMA GEMM here (GPU tensors only).
*/
template<FloatingPointType dtype, Device device, int variant>
inline Tensor<dtype, device> tensor_gemma_mlp_dp_linear(
	const GemmaMLPweights<dtype, device>& mlp_weights,
	const Tensor<dtype, device>& x)
{
	if constexpr (device == CUDA && (variant == 1 || variant == 4))
	{
		static_assert(std::is_same_v<dtype, float32>, "Unsupported data types");
		ACASSERT(x.dim == 3, "x should be 3 dim");
		ACASSERT(x.shape[2] == mlp_weights.down_proj_weight.shape[0], "intermediate size should match for x and the weight");
		Tensor<dtype, device> out(std::vector<int64>{ x.shape[0], x.shape[1], mlp_weights.down_proj_weight.shape[1] });
		if constexpr (variant == 1)
			cu_mlp_gemma2_dp_linear_f32_v1(x, mlp_weights.down_proj_weight, out);
		else
			cu_mlp_gemma2_dp_linear_f32_v4(x, mlp_weights.down_proj_weight, out);
		return out;
	}
	else
	{
		return tensor_linear(x, mlp_weights.down_proj_weight);
	}
}

/* The whole block: fused gate / up projection and down projection on the GPU, operator calls on the host. */
template<FloatingPointType dtype, Device device>
inline Tensor<dtype, device> tensor_gemma_mlp(
	const GemmaMLPweights<dtype, device>& mlp_weights,
	const Tensor<dtype, device>& x)
{
	if constexpr (device == CUDA)
	{
		auto mid = tensor_gemma_mlp_fused_uprpoj<dtype, device, 2>(mlp_weights, x);
		return tensor_gemma_mlp_dp_linear<dtype, device, 4>(mlp_weights, mid);
	}
	else
	{
		auto mid = tensor_gemma_mlp_fused_uprpoj<dtype, device, 0>(mlp_weights, x);
		return tensor_gemma_mlp_dp_linear<dtype, device, 0>(mlp_weights, mid);
	}
}

#endif  // __GEMMA_MLP__
