// Helpers of the attention callers: the scale factor 1 / sqrt(d), rounded to the element type
// (reference: srcs/transformers/attention_tools.hpp:7-40), and the additive mask that the causal and
// sliding-window rules describe (reference: scripts/sdp_test_cases.py:164-168 for the causal part,
// srcs/models/gemma2/gemma_slide_mask.cu:17-29 for the window).
#ifndef __ATTENTION_TOOLS__
#define __ATTENTION_TOOLS__

#include "tensor.hpp"
#include "core_concepts.hpp"

#include <cmath>
#include <limits>
#include <vector>

template<FloatingPointType T>
inline T calculate_alpha(const int d)
{
	return static_cast<T>(1.f / sqrtf(static_cast<float32>(d)));
}

/*
  Additive (q_len, k_len) mask on the host: -inf where key j lies above the shifted diagonal (j > i + diag, causal
  rule), float lowest where it has slid out of the window (window > 0 and j <= i + diag - window), 0 elsewhere.
*/
template<PreciseFloatType T>
inline Tensor<T, CPU> crt_rule_mask(const int64 q_len, const int64 k_len, const bool causal, const int64 window, const int64 diag)
{
	Tensor<T, CPU> mask(std::vector<int64>({ q_len, k_len }));
	T* data = mask.buffer();
	for (int64 i = 0; i < q_len; ++i)
		for (int64 j = 0; j < k_len; ++j)
		{
			T v = static_cast<T>(0);
			if (causal && j > i + diag) v = -std::numeric_limits<T>::infinity();
			if (window > 0 && (i + diag) >= window && j <= i + diag - window) v = std::numeric_limits<T>::lowest();
			data[i * k_len + j] = v;
		}
	return mask;
}

#endif  // __ATTENTION_TOOLS__
