// Split-key plan and merge kernel of the decode forms of the attention (fp16 and fp32).
//
// With few query rows per key / value head there are too few (head, query block) pairs to fill the chip, so
// the visible keys of a head are cut into SPLITS, one wave each per group of 16 rows (the rows of a head beyond 16 go to
// further waves, which read the same keys out of the caches).  A wave leaves, per row, its unnormalised
// accumulators o_i (head_dim floats), its running maximum m_i (in the exponent's base-2 units) and its sum l_i in
// the workspace, [kv_heads][splits][rows][head_dim + 2] floats, and the merge kernel combines the splits of a row:
// M = max m_i,  y = sum o_i 2^(m_i - M) / sum l_i 2^(m_i - M).
#pragma once

#include <algorithm>
#include <cstdint>

#include <hip/hip_runtime.h>

#include "device_utils.hpp"
#include "launch.hpp"

namespace anygpu {

constexpr int kDecodeRowsPerWave = 16;
constexpr int kDecodeMaxRows = 128;               // eight groups of sixteen
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

// `units`: (key / value head, group of 16 rows) pairs, each of which walks the keys
inline DecodePlan plan_decode(int64_t units, int64_t n_q, int64_t n_k, int causal, int64_t window, int keys_per_tile)
{
	const int64_t kv_heads = units;
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

// Which split and which group of 16 rows a block of the partial kernels works on.  The groups of one split read the
// same keys, so they should run at the same time on the same XCD: consecutive blocks go to the eight XCDs in turn, so
// block 8 t + x takes split 8 (t / groups) + x of group t % groups.  False: a block past the last split.
__device__ __forceinline__ bool decode_locate(int groups, int splits, int& split, int& group)
{
	const unsigned x = blockIdx.x % 8u, t = blockIdx.x / 8u;
	group = (int)(t % (unsigned)groups);
	split = (int)(t / (unsigned)groups) * 8 + (int)x;
	return split < splits;
}
inline unsigned decode_blocks(int groups, int splits) { return (unsigned)((splits + 7) / 8 * 8 * groups); }

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

// ---------------------------------------------------------------------------------------------
// Key-split query blocks of the fused kernels (see AttnWalk): two blocks walk one half each of a query block's key tiles
// and leave [query][head_dim accumulators, maximum, sum] in the workspace, [head][split slot][half][query][head_dim + 2].
// ---------------------------------------------------------------------------------------------

// y rows of the key-split blocks from the `parts` partial results of each: one thread per four columns of a row.
template <int D, typename OutT>
__global__ __launch_bounds__(256) void sdp_attention_merge_halves_kernel(const float* __restrict__ partials, OutT* __restrict__ y,
                                                                         int n_q, int q_blocks, int n_split, int queries_per_block,
                                                                         int parts)
{
	constexpr int kQuads = D / 4;
	const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
	const int quad = (int)(item % kQuads);
	const int64_t row_item = item / kQuads;
	const int r = (int)(row_item % queries_per_block);
	const int64_t slot_item = row_item / queries_per_block;            // head * n_split + split slot
	const int split_slot = (int)(slot_item % n_split);
	const int64_t bh = slot_item / n_split;
	const int q_row = (q_blocks - 1 - split_slot) * queries_per_block + r;
	if (q_row >= n_q) return;
	const float* p0 = partials + ((slot_item * parts) * queries_per_block + r) * (D + 2);
	const int64_t step = (int64_t)queries_per_block * (D + 2);
	float big = -INFINITY;
	for (int i = 0; i < parts; ++i) big = fmaxf(big, p0[i * step + D]);
	const float safe = big == -INFINITY ? 0.0f : big;
	float sum = 0.0f;
	float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
	for (int i = 0; i < parts; ++i)
	{
		const float w = fast_exp2(p0[i * step + D] - safe);
		sum += p0[i * step + D + 1] * w;
		acc += *reinterpret_cast<const WsFloat4*>(p0 + i * step + 4 * quad) * w;
	}
	const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
	store_merged(y + (bh * n_q + q_row) * D + 4 * quad, acc * inv);
}

// How many of a head's latest query blocks to dispatch in two key halves (and how many unsplit ones go out before the
// halves).  Worth it when whole blocks cannot be packed evenly: at least a block per CU, and the longest block a large
// share of what a CU gets of the whole launch.  Bounded by the workspace of the stream (the K-split workspace of the
// GEMMs: a caller's, or the library's own for eager launches; none under capture without a caller's: then no split).
struct AttnSplitPlan { int64_t n_split, n_big; };

inline AttnSplitPlan plan_attention_split(int n_q, int n_k, int causal, int diag, int window, int64_t batch_heads,
                                          int queries_per_block, int keys_per_tile, int head_dim, size_t capacity)
{
	AttnSplitPlan plan{0, 0};
	const int64_t q_blocks = (n_q + queries_per_block - 1) / queries_per_block;
	const int cus = device_cu_count();
	if (q_blocks * batch_heads < cus || q_blocks > 65536 || capacity == 0) return plan;
	const auto tiles_of = [&](int64_t b) {
		const int64_t q0 = b * queries_per_block;
		const int64_t q_last = std::min<int64_t>(q0 + queries_per_block - 1, n_q - 1);
		int64_t key_hi = n_k - 1;
		if (causal && q_last + diag < key_hi) key_hi = q_last + diag;
		int64_t key_lo = 0;
		if (window > 0 && q0 + diag - window + 1 > 0) key_lo = q0 + diag - window + 1;
		return key_hi >= 0 && key_hi >= key_lo ? key_hi / keys_per_tile - key_lo / keys_per_tile + 1 : (int64_t)0;
	};
	int64_t total = 0, longest = 0;
	for (int64_t b = 0; b < q_blocks; ++b)
	{
		total += tiles_of(b);
		longest = std::max(longest, tiles_of(b));
	}
	const double per_cu = (double)total * (double)batch_heads / (double)cus;
	if (longest < 16 || (double)longest <= 0.6 * per_cu) return plan;
	const int64_t split_min = std::max<int64_t>(16, (int64_t)(0.6 * per_cu));
	// the latest blocks that are long enough, as far as the workspace holds their partial results
	const int64_t room = (int64_t)(capacity / ((size_t)batch_heads * 2 * queries_per_block * (head_dim + 2) * sizeof(float)));
	int64_t n_split = 0;
	while (n_split < q_blocks && n_split < room && tiles_of(q_blocks - 1 - n_split) >= split_min) ++n_split;
	if (n_split == 0) return plan;
	int64_t n_big = 0;
	while (n_split + n_big < q_blocks && 2 * tiles_of(q_blocks - 1 - n_split - n_big) > longest) ++n_big;
	plan.n_split = n_split;
	plan.n_big = n_big;
	return plan;
}

// Launches with so few query blocks that most CUs would idle while each block walks a long key range alone (a chunk of a
// long prompt against its cache; fewer blocks than CUs): every query block goes out as `parts` blocks, one per part of
// its key tiles.  Twice as many blocks as CUs are aimed at, every part at least 4 tiles, the partial results within
// `capacity` bytes.
// 1: no split.
inline int64_t plan_attention_parts(int n_q, int n_k, int causal, int diag, int64_t batch_heads, int queries_per_block,
                                    int keys_per_tile, int head_dim, size_t capacity)
{
	const int64_t q_blocks = (n_q + queries_per_block - 1) / queries_per_block;
	const int64_t blocks = q_blocks * batch_heads;
	const int cus = device_cu_count();
	if (blocks <= 0 || capacity == 0) return 1;
	if (blocks >= cus)
	{
		// the blocks fill the chip, but the last round of them only in part (320 blocks on 256 CUs): parts of at least 16
		// tiles where they fill the rounds 15 % better (fp32 32 / 8 heads x 1280 x 8192 x 128: 1575 -> 1343 us)
		if (blocks >= 4 * (int64_t)cus) return 1;
		int64_t key_hi0 = n_k - 1;
		if (causal && (int64_t)(n_q - 1) + diag < key_hi0) key_hi0 = (int64_t)(n_q - 1) + diag;
		const int64_t tiles0 = key_hi0 >= 0 ? key_hi0 / keys_per_tile + 1 : 0;
		const auto eff = [&](int64_t s) { return (double)(blocks * s) / (double)((blocks * s + cus - 1) / cus * cus); };
		int64_t best = 1;
		for (int64_t s = 2; s <= 8 && tiles0 / s >= 16; ++s)
			if (eff(s) > eff(best) * 1.02) best = s;
		const int64_t room0 = (int64_t)(capacity / ((size_t)blocks * queries_per_block * (head_dim + 2) * sizeof(float)));
		if (best > room0) best = room0;
		return best >= 2 && eff(best) > 1.15 * eff(1) ? best : 1;
	}
	// the key tiles of the last (longest) query block, from key 0 on or from the window's start: the window only shortens it
	int64_t key_hi = n_k - 1;
	if (causal && (int64_t)(n_q - 1) + diag < key_hi) key_hi = (int64_t)(n_q - 1) + diag;
	const int64_t tiles = key_hi >= 0 ? key_hi / keys_per_tile + 1 : 0;
	int64_t parts = (2 * cus + blocks - 1) / blocks;
	// (with more blocks than half the CUs only long ranges, 16 tiles a part: 8 heads x 3000 x 3000 x 128 causal 63 -> 46 us, but
	// 32 heads x 640 x 640 20 -> 27 in parts of 3 tiles)
	const int64_t part_tiles = blocks * 2 > cus ? 16 : 4;
	if (parts > tiles / part_tiles) parts = tiles / part_tiles;
	if (parts > 64) parts = 64;
	const int64_t room = (int64_t)(capacity / ((size_t)blocks * queries_per_block * (head_dim + 2) * sizeof(float)));
	if (parts > room) parts = room;
	return parts >= 2 ? parts : 1;
}

}  // namespace anygpu
