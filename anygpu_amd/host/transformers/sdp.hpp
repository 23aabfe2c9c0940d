// Scaled dot-product attention with an additive mask over tensors of shape [..., n, d]
// (reference interface: srcs/transformers/sdp.hpp:207-274).
//
// Host tensors: per matrix, qk = q k^T, scaled, mask added, softmax, times v -- the reference's
// per-matrix chain with the transpose taken as a strided view.
// GPU tensors: three launches for ALL matrices instead of six per matrix: one batched GEMM
// q k^T with k in its [n, d] storage (no transpose pass), one softmax with scale and mask fused,
// one batched GEMM p v with v in its [n, d] storage.
#ifndef __SDP__
#define __SDP__

#include "ops.hpp"
#include "attention_tools.hpp"
#include "flash_sdpa_fwd.cuh"

namespace sdp_detail {

template<typename dtype, Device device>
inline int64 leading_matrices(const Tensor<dtype, device>& t)
{
	int64 n = 1;
	for (int64 ix = 0; ix < t.dim - 2; ++ix) n *= t.shape[ix];
	return n;
}

}  // namespace sdp_detail

template<FloatingPointType dtype, Device device>
inline Tensor<dtype, device> sdp_attention_masked_scaled_fwd(
	const Tensor<dtype, device>& qw,
	const Tensor<dtype, device>& kw,
	const Tensor<dtype, device>& vw,
	const Tensor<dtype, device>& mask,
	const dtype alpha)
{
	if constexpr (device == CPU)
	{
		static_assert(PreciseFloatType<dtype>, "for cpu only precise float is supported");
	}

	ACASSERT(qw.dim == kw.dim && vw.dim == kw.dim, "dimension missmatch");
	ACASSERT(mask.dim == qw.dim, "mask dimension is inappropriate");
	ACASSERT(qw.dim >= 2, "attention needs at least 2 dimensional tensors");

	const int64 dim = qw.dim;
	for (int64 ix = 0; ix < dim - 2; ++ix)
	{
		ACASSERT(qw.shape[ix] == kw.shape[ix] && kw.shape[ix] == vw.shape[ix],
			"qw, kw, vw needs to have the same number of 2d matrices");
		ACASSERT(mask.shape[ix] == 1, "mask needs to have 1s in the first dims except the last two");
	}
	const int64 num_mtcs = sdp_detail::leading_matrices(qw);
	const int64 n_q = qw.shape[dim - 2], d = qw.shape[dim - 1];
	const int64 n_k = kw.shape[dim - 2], d_v = vw.shape[dim - 1];
	ACASSERT(kw.shape[dim - 1] == d && vw.shape[dim - 2] == n_k, "qw, kw, vw shapes do not fit each other");
	ACASSERT(mask.shape[dim - 2] == n_q && mask.shape[dim - 1] == n_k, "mask shape does not fit the scores");

	// output: the shape of q with the feature size of v
	Shape y_shape = qw.shape;
	y_shape[dim - 1] = d_v;
	Tensor<dtype, device> y(dim, y_shape);

	if constexpr (device == CPU)
	{
		auto maskn = tensor_view(mask, { n_q, n_k });
		auto q_mtcs = tensor_split(tensor_view(qw, { num_mtcs, n_q, d }), num_mtcs);
		auto k_mtcs = tensor_split(tensor_view(kw, { num_mtcs, n_k, d }), num_mtcs);
		auto v_mtcs = tensor_split(tensor_view(vw, { num_mtcs, n_k, d_v }), num_mtcs);
		auto y_mtcs = tensor_split(tensor_view(y, { num_mtcs, n_q, d_v }), num_mtcs);
		for (int64 ix = 0; ix < num_mtcs; ++ix)
		{
			auto q_mtx = tensor_view(q_mtcs[ix], { n_q, d });
			auto v_mtx = tensor_view(v_mtcs[ix], { n_k, d_v });
			auto y_mtx = tensor_view(y_mtcs[ix], { n_q, d_v });
			// k^T as a view: shape [d, n_k], strides (1, d)
			auto k_tr = tensor_view(k_mtcs[ix], { n_k, d });
			k_tr.shape = { d, n_k };
			k_tr.stride = { 1, d };

			auto qk = tensor_mm(q_mtx, k_tr);
			auto nqk = tensor_mul(qk, alpha);
			auto nqk_masked = tensor_add(nqk, maskn);
			auto score = tensor_softmax(nqk_masked);
			tensor_mm(score, v_mtx, y_mtx);
		}
	}
	else
	{
		static_assert(std::is_same_v<dtype, float32> || std::is_same_v<dtype, float16>, "Unsupported data type");
		// a head dimension the fused kernels have: one kernel that reads the mask as data, no score matrix
		if (d == d_v && (d == 64 || d == 128 || d == 256) && num_mtcs > 0 && n_q > 0 && n_k > 0)
		{
			if constexpr (std::is_same_v<dtype, float32>)
				hip_flash_sdpa_fwd_masked_f32(static_cast<float32>(alpha), qw, kw, vw, mask, y);
			else
				hip_flash_sdpa_fwd_masked_f16(static_cast<float32>(alpha), qw, kw, vw, mask, y);
			return y;
		}
		Tensor<dtype, CUDA> scores(std::vector<int64>({ num_mtcs * n_q, n_k }));
		Tensor<dtype, CUDA> probs(std::vector<int64>({ num_mtcs * n_q, n_k }));
		hip_tensor_mm_batched(qw, kw, scores, num_mtcs, n_q, n_k, d, /*rhs stored [n, k]*/ true);
		hip_tensor_softmax_masked(scores, mask, static_cast<float32>(alpha), n_q, probs);
		hip_tensor_mm_batched(probs, vw, y, num_mtcs, n_q, d_v, n_k, /*rhs stored [n, k]*/ false);
	}

	return y;
}

/* Single-matrix attention without mask: softmax(q k^T / sqrt(d)) v (reference: sdp.hpp:14-46). */
template<FloatingPointType dtype, Device device>
inline Tensor<dtype, device> single_head_attention_fwd(
	const Tensor<dtype, device>& qw,
	const Tensor<dtype, device>& kw,
	const Tensor<dtype, device>& vw)
{
	const int64 d = qw.shape[1], n_k = kw.shape[0];
	const dtype alpha = calculate_alpha<dtype>(static_cast<int>(d));
	if constexpr (device == CPU)
	{
		static_assert(PreciseFloatType<dtype>, "for cpu only precise float is supported");
		auto k_tr = kw;
		k_tr.shape = { d, n_k };
		k_tr.stride = { 1, d };
		auto score = tensor_softmax(tensor_mul(tensor_mm(qw, k_tr), alpha));
		return tensor_mm(score, vw);
	}
	else
	{
		auto qk = tensor_mm_nt(qw, kw);
		SoftmaxPrologue p;
		p.alpha = static_cast<float32>(alpha);
		return tensor_mm(tensor_softmax(qk, p), vw);
	}
}

/*
  Single-matrix attention through the fused kernels (reference: sdp_attention_fwd_cuda_flash, sdp.hpp:48-73, float32,
  d = 256 only).  Both precisions run the one-kernel form for d = 64, 128 or 256; float32 with another d runs
  q k^T, softmax with the scale folded in and p v.
*/
template<FloatingPointType dtype>
inline Tensor<dtype, CUDA> sdp_attention_fwd_cuda_flash(
	const Tensor<dtype, CUDA>& qw,
	const Tensor<dtype, CUDA>& kw,
	const Tensor<dtype, CUDA>& vw)
{
	const int64 N = qw.shape[0], d = qw.shape[1];   // (N, d)
	ACASSERT(kw.shape[0] == N, "qw and kw differs in sequence length");
	ACASSERT(vw.shape[0] == N, "qw and vw differs in sequence length");
	ACASSERT(kw.shape[1] == d && vw.shape[1] == d, "hidden dimensions differ");
	if constexpr (std::is_same_v<dtype, float16>)
	{
		ACASSERT(d == 64 || d == 128 || d == 256, "hidden dimension must be 64, 128 or 256");
		Tensor<dtype, CUDA> y(qw.dim, qw.shape);
		SoftmaxPrologue p;
		p.alpha = static_cast<float32>(calculate_alpha<float32>(static_cast<int>(d)));
		hip_flash_sdpa_fwd_f16(p, qw, kw, vw, y);
		return y;
	}
	else
	{
		if (d != 64 && d != 128 && d != 256) return single_head_attention_fwd(qw, kw, vw);
		Tensor<dtype, CUDA> y(qw.dim, qw.shape);
		const float32 alpha = static_cast<float32>(calculate_alpha<float32>(static_cast<int>(d)));
		if (d == 256)
		{
			cu_flash_sdpa_fwd_d256_v1(alpha, qw, kw, vw, y);
		}
		else
		{
			SoftmaxPrologue p;
			p.alpha = alpha;
			hip_flash_sdpa_fwd_f32(p, qw, kw, vw, y);
		}
		return y;
	}
}

/*
  Attention over (..., heads, n, d) tensors with the mask given by rules instead of a tensor: scale, optional
  softcap, causal rule with the diagonal at n_k - n_q, optional sliding window (the fields of SoftmaxPrologue).
  GPU tensors with d = 64, 128 or 256 take the fused kernels (k and v may have fewer heads than q); host tensors and
  float32 with another d take sdp_attention_masked_scaled_fwd with the mask the rules describe.
*/
template<FloatingPointType dtype, Device device>
inline Tensor<dtype, device> sdp_attention_rules_fwd(
	const Tensor<dtype, device>& qw,
	const Tensor<dtype, device>& kw,
	const Tensor<dtype, device>& vw,
	const SoftmaxPrologue& rules)
{
	const int64 dim = qw.dim;
	ACASSERT(dim >= 2 && kw.dim == dim && vw.dim == dim, "dimension missmatch");
	const int64 n_q = qw.shape[dim - 2], n_k = kw.shape[dim - 2], d = qw.shape[dim - 1];
	ACASSERT(kw.shape[dim - 1] == d && vw.shape[dim - 1] == d && vw.shape[dim - 2] == n_k, "q, k and v need one head dimension");
	if constexpr (device == CUDA && std::is_same_v<dtype, float16>)
	{
		ACASSERT(d == 64 || d == 128 || d == 256, "hidden dimension must be 64, 128 or 256");
		ACASSERT(rules.softcap >= 0.f && rules.window >= 0, "softcap and window must not be negative");
		Tensor<dtype, CUDA> y(qw.dim, qw.shape);
		if (hip_flash_sdpa_decode_applies(qw, kw))
		{
			// generation step: the split-key form; its scratch lives for this call only
			Tensor<float32, CUDA> workspace(std::vector<int64>{ std::max<int64>(hip_flash_sdpa_decode_workspace_floats(rules, qw, kw), 4) });
			hip_flash_sdpa_decode_f16(rules, qw, kw, vw, workspace, y);
		}
		else
		{
			hip_flash_sdpa_fwd_f16(rules, qw, kw, vw, y);
		}
		return y;
	}
	else if constexpr (device == CUDA && std::is_same_v<dtype, float32>)
	{
		if (d == 64 || d == 128 || d == 256)
		{
			ACASSERT(rules.softcap >= 0.f && rules.window >= 0, "softcap and window must not be negative");
			Tensor<dtype, CUDA> y(qw.dim, qw.shape);
			if (hip_flash_sdpa_decode_applies(qw, kw))
			{
				Tensor<float32, CUDA> workspace(std::vector<int64>{ std::max<int64>(hip_flash_sdpa_decode_workspace_floats(rules, qw, kw), 4) });
				hip_flash_sdpa_decode_f32(rules, qw, kw, vw, workspace, y);
			}
			else
			{
				hip_flash_sdpa_fwd_f32(rules, qw, kw, vw, y);
			}
			return y;
		}
		ACASSERT(rules.softcap == 0.f, "the softcap needs the fused kernel");
		auto hmask = crt_rule_mask<float32>(n_q, n_k, rules.causal, rules.window, n_k - n_q);
		std::vector<int64> mshape(static_cast<size_t>(dim), 1);
		mshape[dim - 2] = n_q;
		mshape[dim - 1] = n_k;
		auto mview = tensor_view(hmask, mshape);
		return sdp_attention_masked_scaled_fwd(qw, kw, vw, mview.copy_to_cuda(), static_cast<dtype>(rules.alpha));
	}
	else
	{
		ACASSERT(rules.softcap == 0.f, "the softcap needs the fused kernel");
		auto hmask = crt_rule_mask<float32>(n_q, n_k, rules.causal, rules.window, n_k - n_q);
		Tensor<dtype, CPU> hm = cvt_tensor_from_float32<dtype>(hmask);
		std::vector<int64> mshape(static_cast<size_t>(dim), 1);
		mshape[dim - 2] = n_q;
		mshape[dim - 1] = n_k;
		auto mview = tensor_view(hm, mshape);
		if constexpr (device == CUDA)
			return sdp_attention_masked_scaled_fwd(qw, kw, vw, mview.copy_to_cuda(), static_cast<dtype>(rules.alpha));
		else
			return sdp_attention_masked_scaled_fwd(qw, kw, vw, mview, static_cast<dtype>(rules.alpha));
	}
}

#endif  // __SDP__
