// The reference keeps a ladder of experimental matmul kernels (srcs/kernels/cuda/fast_mm.cuh:7-98),
// each with its own entry point.  On gfx950 one MFMA kernel family serves all of them; the entry
// points are kept so that callers and tests naming a particular rung still link.  All take
// yt preallocated with shape [xt rows, wt cols] and any sizes (the "multiple of 128" demand of
// the originals is gone).
#ifndef __FAST_MM_CUH__
#define __FAST_MM_CUH__

#include "tensor.hpp"

#define ANYGPU_DECLARE_FAST_MM(NAME, T) \
	void NAME(const Tensor<T, CUDA>& xt, const Tensor<T, CUDA>& wt, Tensor<T, CUDA>& yt)

/* float32: xt [M, K], wt [K, N] */
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f32_cb, float32);
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f32_v1, float32);
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f32_v2, float32);
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f32_v2_1, float32);
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f32_v3, float32);
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f32_v4, float32);
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f32_v4_1, float32);
/* this rung alone takes the left operand pre-transposed: xt [K, M] */
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f32_v4_2, float32);

/* float16 inputs and output, float32 accumulation: xt [M, K], wt [K, N] */
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f16_v1, float16);
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f16_v2, float16);
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f16_v3, float16);
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f16_v3_1, float16);
ANYGPU_DECLARE_FAST_MM(cu_fast_mm_f16_v3_2, float16);

#undef ANYGPU_DECLARE_FAST_MM

#endif  // __FAST_MM_CUH__
