// Scale factor of dot-product attention: 1 / sqrt(d), rounded to the element type
// (reference: srcs/transformers/attention_tools.hpp:7-40).
#ifndef __ATTENTION_TOOLS__
#define __ATTENTION_TOOLS__

#include "tensor.hpp"
#include "core_concepts.hpp"

template<FloatingPointType T>
inline T calculate_alpha(const int d)
{
	return static_cast<T>(1.f / sqrtf(static_cast<float32>(d)));
}

#endif  // __ATTENTION_TOOLS__
