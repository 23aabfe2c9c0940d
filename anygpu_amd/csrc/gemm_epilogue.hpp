// What the GEMM kernels do to a finished sum before it is stored.
#pragma once

#include "device_utils.hpp"

namespace anygpu {

enum Epilogue
{
	kEpiBias = 0,      // + bias[n] when bias != NULL, else nothing
	kEpiSoftcap = 1,   // cap * tanh(sum / cap)
	kEpiGeluMul = 2    // gelu_tanh(A * B) * (A * B2): two products that share A, combined elementwise
};

// gelu(z) with the tanh approximation: z / 2 * (1 + tanh(sqrt(2 / pi) * (z + 0.044715 z^3))).  HALF_OUT: the result is
// rounded to fp16 (the cheaper tanh; here it is added to 1, so its absolute error is what counts either way).
template <bool HALF_OUT = false>
__device__ __forceinline__ float gelu_tanh_f32(float z)
{
	const float inner = 0.7978845608028654f * (z + 0.044715f * z * z * z);
	return z * 0.5f * (1.0f + (HALF_OUT ? tanh_for_half(inner) : tanh_f32(inner)));
}

// `sum2` is the second product (kEpiGeluMul only), `bias_n` the bias of this column or 0,
// `param` the cap of kEpiSoftcap.
template <int EPI, bool HALF_OUT = false>
__device__ __forceinline__ float finish_sum(float sum, float sum2, float bias_n, float param)
{
	// (times the reciprocal, which the compiler keeps out of the loops over a patch: a division per sum was half the
	// arithmetic of this epilogue, and a patch of 128 x 128 sums has nothing to hide it behind)
	if constexpr (EPI == kEpiSoftcap) return param * (HALF_OUT ? tanh_for_half(sum * (1.0f / param)) : tanh_f32(sum * (1.0f / param)));
	else if constexpr (EPI == kEpiGeluMul) return gelu_tanh_f32<HALF_OUT>(sum) * sum2;
	else return sum + bias_n;
}

}  // namespace anygpu
