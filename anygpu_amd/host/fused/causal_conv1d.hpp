// Depthwise causal conv1d fused with bias and SiLU (the convolution in front of a Mamba2 mixer).
//   x (batch, dims, seq_len), weights (dims, width), bias (dims) -> y (batch, dims, seq_len)
//   y = silu(conv1d(x, weights.unsqueeze(1), bias, stride=1, padding=width-1, groups=dims))[..., :seq_len]
// Reference interface: srcs/fused/causal_conv1d.hpp:24-117.
#ifndef __CAUSAL_CONV1D__
#define __CAUSAL_CONV1D__

#include "causal_conv1d.cuh"

#include "tensor.hpp"
#include "core_concepts.hpp"

/*
  Host loops.  For every (batch, channel) row and position s: taps k = 0..width-1 ascending,
  tap k reads x[s + k - (width - 1)], negative positions are skipped (zero padding on the left);
  then the bias is added and the value passes through v / (1 + exp(-v)).  Sums in dtype.
*/
template<PreciseFloatType dtype>
inline Tensor<dtype, CPU> tensor_causal_conv1d(
	const Tensor<dtype, CPU>& xt,
	const Tensor<dtype, CPU>& wt,
	const Tensor<dtype, CPU>& bt)
{
	ACASSERT(xt.dim == 3, "xt needs to be 3 dimensional");
	ACASSERT(xt.shape[1] == wt.shape[0], "xt and wt need to have the same dims");
	ACASSERT(wt.shape[0] == bt.shape[0], "wt and bt need to have the same dims");

	Tensor<dtype, CPU> yt(xt.dim, xt.shape);
	const int64 batch = xt.shape[0], dims = xt.shape[1], seq_len = xt.shape[2];
	const int64 width = wt.shape[1];

	const dtype* x_data = xt.buffer();
	const dtype* w_data = wt.buffer();
	const dtype* b_data = bt.buffer();
	dtype* y_data = yt.buffer();

	for (int64 bix = 0; bix < batch; ++bix)
	{
		for (int64 dix = 0; dix < dims; ++dix)
		{
			const dtype* x_row = x_data + bix * xt.stride[0] + dix * xt.stride[1];
			dtype* y_row = y_data + bix * yt.stride[0] + dix * yt.stride[1];
			const dtype* taps = w_data + dix * wt.stride[0];

			for (int64 six = 0; six < seq_len; ++six)
			{
				dtype out = 0;
				for (int64 k = 0; k < width; ++k)
				{
					const int64 src = six + k - (width - 1);
					if (src >= 0) out += taps[k] * x_row[src];
				}
				out += b_data[dix];
				y_row[six] = out / (static_cast<dtype>(1.0) + std::exp(-out));
			}
		}
	}

	return yt;
}

/* GPU path; float32 as in the reference, float16 in addition.  Kernel width up to 4. */
template<FloatingPointType dtype>
inline Tensor<dtype, CUDA> tensor_causal_conv1d(
	const Tensor<dtype, CUDA>& xt,
	const Tensor<dtype, CUDA>& wt,
	const Tensor<dtype, CUDA>& bt)
{
	ACASSERT(xt.dim == 3, "xt needs to be 3 dimensional");
	ACASSERT(xt.shape[1] == wt.shape[0], "xt and wt need to have the same dims");
	ACASSERT(wt.shape[0] == bt.shape[0], "wt and bt need to have the same dims");
	ACASSERT(wt.shape[1] <= 4, "kernel width needs to be under 4");

	Tensor<dtype, CUDA> yt(xt.dim, xt.shape);

	if constexpr (std::is_same_v<dtype, float32>)
	{
		cu_tensor_causal_conv1d_f32(xt, wt, bt, yt);
	}
	else
	{
		static_assert(std::is_same_v<dtype, float16>, "Unsupported data types");
		hip_tensor_causal_conv1d_f16(xt, wt, bt, yt);
	}

	return yt;
}

/*
  Decode step of the same convolution.  xt (batch, dims) holds the newest sample of every row, state
  (batch, dims, width - 1) the samples in front of it, oldest first; the result is the convolution's
  output at that position and the state moves on by one sample (in place).  Starting from a zero state,
  seq_len steps give the columns of tensor_causal_conv1d.
*/
template<PreciseFloatType dtype>
inline Tensor<dtype, CPU> tensor_causal_conv1d_update(
	const Tensor<dtype, CPU>& xt,
	Tensor<dtype, CPU>& state,
	const Tensor<dtype, CPU>& wt,
	const Tensor<dtype, CPU>& bt)
{
	ACASSERT(xt.dim == 2 && state.dim == 3, "xt needs to be 2 and state 3 dimensional");
	ACASSERT(xt.shape[1] == wt.shape[0], "xt and wt need to have the same dims");
	ACASSERT(wt.shape[0] == bt.shape[0], "wt and bt need to have the same dims");
	ACASSERT(state.shape[0] == xt.shape[0] && state.shape[1] == xt.shape[1] && state.shape[2] == wt.shape[1] - 1,
	         "state needs to be (batch, dims, width - 1)");

	Tensor<dtype, CPU> yt(xt.dim, xt.shape);
	const int64 rows = xt.shape[0] * xt.shape[1], dims = xt.shape[1], width = wt.shape[1];
	const dtype* x_data = xt.buffer();
	const dtype* w_data = wt.buffer();
	const dtype* b_data = bt.buffer();
	dtype* s_data = state.buffer();
	dtype* y_data = yt.buffer();

	for (int64 row = 0; row < rows; ++row)
	{
		const int64 dix = row % dims;
		dtype* hist = s_data + row * (width - 1);
		dtype out = 0;
		for (int64 k = 0; k < width; ++k) out += w_data[dix * width + k] * (k < width - 1 ? hist[k] : x_data[row]);
		out += b_data[dix];
		y_data[row] = out / (static_cast<dtype>(1.0) + std::exp(-out));
		for (int64 k = 0; k + 2 < width; ++k) hist[k] = hist[k + 1];
		if (width > 1) hist[width - 2] = x_data[row];
	}
	return yt;
}

template<FloatingPointType dtype>
inline Tensor<dtype, CUDA> tensor_causal_conv1d_update(
	const Tensor<dtype, CUDA>& xt,
	Tensor<dtype, CUDA>& state,
	const Tensor<dtype, CUDA>& wt,
	const Tensor<dtype, CUDA>& bt)
{
	ACASSERT(xt.dim == 2 && state.dim == 3, "xt needs to be 2 and state 3 dimensional");
	ACASSERT(xt.shape[1] == wt.shape[0], "xt and wt need to have the same dims");
	ACASSERT(wt.shape[0] == bt.shape[0], "wt and bt need to have the same dims");
	ACASSERT(wt.shape[1] <= 4, "kernel width needs to be under 4");
	ACASSERT(state.shape[0] == xt.shape[0] && state.shape[1] == xt.shape[1] && state.shape[2] == wt.shape[1] - 1,
	         "state needs to be (batch, dims, width - 1)");

	Tensor<dtype, CUDA> yt(xt.dim, xt.shape);
	if constexpr (std::is_same_v<dtype, float32>)
	{
		hip_tensor_causal_conv1d_update_f32(xt, state, wt, bt, yt);
	}
	else
	{
		static_assert(std::is_same_v<dtype, float16>, "Unsupported data types");
		hip_tensor_causal_conv1d_update_f16(xt, state, wt, bt, yt);
	}
	return yt;
}

#endif  // __CAUSAL_CONV1D__
