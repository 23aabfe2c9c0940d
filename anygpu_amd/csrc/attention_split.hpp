// Split-key plan and merge kernel of the decode forms of the attention (fp16 and fp32).
//
// With at most 16 query rows per key / value head there are too few (head, query block) pairs to fill the chip, so
// the visible keys of a head are cut into SPLITS, one wave each.  A wave leaves, per row, its unnormalised
// accumulators o_i (head_dim floats), its running maximum m_i (in the exponent's base-2 units) and its sum l_i in
// the workspace, [kv_heads][splits][rows][head_dim + 2] floats, and the merge kernel combines the splits of a row:
// M = max m_i,  y = sum o_i 2^(m_i - M) / sum l_i 2^(m_i - M).
#pragma once

#include <cstdint>

#include <hip/hip_runtime.h>

#include "device_utils.hpp"

namespace anygpu {

constexpr int kDecodeMaxRows = 16;
// One split per thread of the merge block.  64 splits of 8 tiles left 64 q heads / 8 kv heads x 32768 keys x 128
// at 33.8 us for the two launches, 128 splits of 4 tiles take 28.0 us; the old merge (one thread per column walking
// all splits) would have eaten that gain, since its time grew with the number of splits.
constexpr int kDecodeMaxSplits = 256;
constexpr int kDecodeTargetWaves = 1024;          // one wave per SIMD; two per SIMD measured 5 - 20 % slower

// a workspace row is head_dim + 2 floats long: its 16-byte accesses are aligned to 8 bytes only
typedef float4_t WsFloat4 __attribute__((aligned(8)));

struct DecodePlan
{
	int t_first, t_last, splits, tiles_per_split;
};

inline DecodePlan plan_decode(int64_t kv_heads, int64_t n_q, int64_t n_k, int causal, int64_t window, int keys_per_tile)
{
	// visible key tiles of a group: its first query decides the low end, its last the high end
	const int64_t diag = n_k - n_q;
	int64_t key_hi = n_k - 1;
	if (causal && (n_q - 1) + diag < key_hi) key_hi = (n_q - 1) + diag;
	int64_t key_lo = 0;
	if (window > 0 && diag - window + 1 > 0) key_lo = diag - window + 1;
	DecodePlan p;
	p.t_first = (int)(key_lo / keys_per_tile);
	p.t_last = key_hi >= 0 ? (int)(key_hi / keys_per_tile) : p.t_first - 1;
	const int64_t tiles = p.t_last - p.t_first + 1;
	if (tiles <= 0)
	{
		p.splits = 1;
		p.tiles_per_split = 0;
		return p;
	}
	int64_t want = (kDecodeTargetWaves + kv_heads - 1) / kv_heads;
	if (want > kDecodeMaxSplits) want = kDecodeMaxSplits;
	if (want > tiles) want = tiles;
	if (want < 1) want = 1;
	p.tiles_per_split = (int)((tiles + want - 1) / want);
	p.splits = (int)((tiles + p.tiles_per_split - 1) / p.tiles_per_split);
	return p;
}

__device__ __forceinline__ void store_merged(float* dst, const float4_t& v) { *reinterpret_cast<float4_t*>(dst) = v; }
__device__ __forceinline__ void store_merged(half_t* dst, const float4_t& v)
{
	half4_t out;
#pragma unroll
	for (int r = 0; r < 4; ++r) out[r] = (half_t)v[r];
	*reinterpret_cast<half4_t*>(dst) = out;
}

// One block of 256 threads per (key / value head, row).  Every thread fetches the maximum and the sum of one split
// and the block leaves the weights 2^(m_i - M) in LDS; then a thread owns four output columns and every
// (256 / (D / 4))-th split, so the loads of the partial rows are wide and independent, and the threads of a column
// quad add up through LDS.
template <int D, typename OutT>
__global__ __launch_bounds__(256) void sdp_decode_merge_kernel(const float* __restrict__ ws, OutT* __restrict__ y, int rows, int splits)
{
	constexpr int kQuads = D / 4;
	constexpr int kLanes = 256 / kQuads;
	static_assert(kDecodeMaxSplits <= 256, "one split per thread");
	__shared__ float weight[256];
	__shared__ float red[2][4];
	__shared__ float4_t part[256];
	const int row = blockIdx.x, kvh = blockIdx.y, t = threadIdx.x;
	const int lane = t & 63, wave = t >> 6;
	const float* base = ws + (((int64_t)kvh * splits) * rows + row) * (D + 2);
	const int64_t step = (int64_t)rows * (D + 2);
	const float m = t < splits ? base[t * step + D] : -INFINITY;
	const float l = t < splits ? base[t * step + D + 1] : 0.0f;
	float big = wave_allreduce(m, MaxOp());
	if (lane == 0) red[0][wave] = big;
	__syncthreads();
	big = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
	const float w = fast_exp2(m - (big == -INFINITY ? 0.0f : big));
	float sum = wave_allreduce(l * w, SumOp());
	weight[t] = w;
	if (lane == 0) red[1][wave] = sum;
	__syncthreads();
	sum = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);

	const int first = t / kQuads;
	float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 4
	for (int i = first; i < splits; i += kLanes)
	{
		const float4_t v = *reinterpret_cast<const WsFloat4*>(base + i * step + 4 * (t % kQuads));
		acc += v * weight[i];
	}
	part[t] = acc;
	__syncthreads();
	if (t < kQuads)
	{
#pragma unroll
		for (int i = 1; i < kLanes; ++i) acc += part[i * kQuads + t];
		const float4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
		store_merged(y + ((int64_t)kvh * rows + row) * D + 4 * t, sum > 0.0f ? acc / sum : zero);
	}
}

}  // namespace anygpu
