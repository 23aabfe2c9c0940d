// Small device-side helpers shared by the gfx950 kernels: 16-byte vector types, wave64
// reductions built on DPP, and fp32 transcendental wrappers.
#pragma once

#include <hip/hip_runtime.h>

namespace anygpu {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kWaveSize = 64;
constexpr float kLog2e = 1.4426950408889634f;

// One DPP move: lane l receives `v` from the lane selected by CTRL inside its row of 16
// lanes; with bound_ctrl set, lanes without a source read 0 (never the case for the
// permutations and rotations used here).
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v)
{
	return __builtin_bit_cast(float,
		__builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Value of `v` in lane `lane` as a wave-uniform scalar (the builtin moves 32 raw bits).
__device__ __forceinline__ float read_lane(float v, int lane)
{
	return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

struct MaxOp { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };
struct SumOp { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };

// All-reduce over the 64 lanes of a wave.  Within each row of 16 lanes: two quad
// permutations (xor 1, xor 2), then row rotations by 4 and 8.  The four row results are
// then read out as scalars and combined, which leaves the same value in every lane.
template <typename Op>
__device__ __forceinline__ float wave_allreduce(float v, Op op)
{
	v = op(v, dpp_move<0xB1>(v));    // quad_perm [1,0,3,2]
	v = op(v, dpp_move<0x4E>(v));    // quad_perm [2,3,0,1]
	v = op(v, dpp_move<0x124>(v));   // row_ror:4
	v = op(v, dpp_move<0x128>(v));   // row_ror:8
	const float r0 = read_lane(v, 0);
	const float r1 = read_lane(v, 16);
	const float r2 = read_lane(v, 32);
	const float r3 = read_lane(v, 48);
	return op(op(r0, r1), op(r2, r3));
}

// All-reduce over each row of 16 lanes of a wave (the first four steps of the above): every lane ends up with the
// result of its own row.
template <typename Op>
__device__ __forceinline__ float row_allreduce(float v, Op op)
{
	v = op(v, dpp_move<0xB1>(v));    // quad_perm [1,0,3,2]
	v = op(v, dpp_move<0x4E>(v));    // quad_perm [2,3,0,1]
	v = op(v, dpp_move<0x124>(v));   // row_ror:4
	v = op(v, dpp_move<0x128>(v));   // row_ror:8
	return v;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// Maximum over the four 16-lane rows of a wave, for every lane % 16, left in all four rows.  gfx950's row swaps do in
// the VALU what two cross-lane shuffles (each a trip through the LDS crossbar) do: v_permlane16_swap exchanges the
// odd rows of its first operand with the even rows of its second, v_permlane32_swap the upper half of the first with
// the lower half of the second; fed two copies of x they return {row 0, 0, 2, 2} and {1, 1, 3, 3}, then {lower, lower}
// and {upper, upper}.  (Written as assembly: the builtins of this compiler release fold the pair of results of a swap
// of two equal operands into one value.)
__device__ __forceinline__ float max_over_lane_rows(float x)
{
	float a = x, b = x;
	asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
	const float m = fmaxf(a, b);
	a = m;
	b = m;
	asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
	return fmaxf(a, b);
}

// tanh(x) = 1 - 2 / (1 + e^{2x}); saturates cleanly to +-1 for large |x| (e^{2x} -> inf or 0).
// Near zero that form cancels, so |x| < 1/16 uses the odd Taylor polynomial up to x^7
// (truncation error below 1e-11 relative at the switch point).
__device__ __forceinline__ float tanh_f32(float x)
{
	float e = fast_exp2(x * (2.0f * kLog2e));
	float big = 1.0f - 2.0f * fast_rcp(1.0f + e);
	float x2 = x * x;
	float small = x * (1.0f + x2 * (-1.0f / 3.0f + x2 * (2.0f / 15.0f + x2 * (-17.0f / 315.0f))));
	return fabsf(x) < 0.0625f ? small : big;
}

// tanh for results that are rounded to fp16 (half an ulp: 5e-4 relative): the closed form, whose absolute error of about
// 1.5e-7 is 4e-5 relative at |x| = 2^-8, and below that x itself (tanh(x) = x to 5e-6 relative there).  Two
// transcendentals and five other instructions instead of eleven others.
__device__ __forceinline__ float tanh_for_half(float x)
{
	const float e = fast_exp2(x * (2.0f * kLog2e));
	const float big = fmaf(fast_rcp(1.0f + e), -2.0f, 1.0f);
	return fabsf(x) < 0.00390625f ? x : big;
}

}  // namespace anygpu
