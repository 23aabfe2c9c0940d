// Visible-tile map of an attention mask tensor.
//
// The fused attention kernels that take the mask as data walk the key range of a query block tile by tile.  Which
// tiles the mask hides from the whole block is not known from the shapes, as it is for the index rules; a pass over
// the mask finds out: bit (t % 64) of word [query block][t / 64] is set when some query of the block sees some key of
// tile t.  The attention kernel then loads and multiplies the set tiles only (under a causal mask tensor half of
// them, under a sliding window fewer).  The mask is shared by all heads, so the pass reads it once where the
// attention kernel reads it once per head.
#pragma once

#include "device_utils.hpp"

#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdlib>

namespace anygpu {

// A mask value hides its key when its log2-domain form is -inf: -inf itself and, in float32, values so low that the
// multiplication by log2(e) overflows (the float lowest of the reference's mask builders).  The kernels apply the same test.
template <typename T>
__device__ __forceinline__ bool mask_value_visible(T value)
{
	return (float)value * 1.4426950408889634f > -INFINITY;
}

// One block of 16 waves per (query block, group of 16 tiles), a wave per tile: lane = key of the tile, 32 loads in
// flight per step.  The block leaves the 16 bits of its group; four groups are a word of the map.
template <typename T>
__global__ __launch_bounds__(1024) void attention_mask_tile_map_kernel(const T* __restrict__ mask, int64_t mask_stride, int n_q, int n_k,
                                                                       int queries_per_block, int keys_per_tile, int groups,
                                                                       unsigned short* __restrict__ map)
{
	__shared__ unsigned int bits;
	const int q_block = blockIdx.x / groups, group = blockIdx.x % groups;
	const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
	if (threadIdx.x == 0) bits = 0;
	__syncthreads();
	const int tiles = (n_k + keys_per_tile - 1) / keys_per_tile;
	const int r0 = q_block * queries_per_block;
	const int r1 = r0 + queries_per_block < n_q ? r0 + queries_per_block : n_q;
	const int t = 16 * group + wave;
	if (t < tiles)
	{
		// a step is 32 loads in flight, each a row (two rows with tiles of 32 keys); rows past the block's last and keys
		// past the end repeat the last one, so that no load sits behind a branch
		const int rows_per_load = 64 / keys_per_tile;                 // (tiles are 32 or 64 keys)
		const int key_raw = t * keys_per_tile + lane % keys_per_tile;
		const int key = key_raw < n_k ? key_raw : n_k - 1;
		const T* column = mask + key;
		bool seen = false;
		for (int r = r0 + lane / keys_per_tile; r < r1; r += 32 * rows_per_load)
		{
			T value[32];
#pragma unroll
			for (int j = 0; j < 32; ++j)
			{
				const int row = r + j * rows_per_load < r1 ? r + j * rows_per_load : r1 - 1;
				value[j] = column[(int64_t)row * mask_stride];
			}
#pragma unroll
			for (int j = 0; j < 32; ++j) seen |= mask_value_visible(value[j]);
		}
		if (__builtin_amdgcn_ballot_w64(seen) != 0 && lane == 0) atomicOr(&bits, 1u << wave);
	}
	__syncthreads();
	if (threadIdx.x == 0) map[(int64_t)q_block * groups + group] = (unsigned short)bits;
}

// Whether the map is made for a mask of n_q x n_k values.  Its pass costs a launch and a few memory latencies (8 - 12 us for
// small masks, 5.6 TB/s for large ones), which short key ranges do not earn back: from 4 M mask values on, or from 16384 keys
// on whatever the queries (a sliding window over a long cache hides most of them from a few queries as well).  The
// environment variable ANYGPU_ATTN_MASK_MAP_FROM, read at every launch, replaces the rule by "from that many mask values
// on" (0: always, a huge value: never).
inline bool attention_mask_map_wanted(int64_t n_q, int64_t n_k)
{
	const char* text = std::getenv("ANYGPU_ATTN_MASK_MAP_FROM");
	if (text != nullptr && *text != 0) return n_q * n_k >= std::atoll(text);
	return n_q * n_k >= (4ll << 20) || n_k >= 16384;
}

// 64-bit words of the map per query block
inline int64_t attention_tile_map_words(int64_t n_k, int keys_per_tile)
{
	return ((n_k + keys_per_tile - 1) / keys_per_tile + 63) / 64;
}

template <typename T>
inline hipError_t launch_attention_mask_tile_map(const T* mask, int64_t mask_stride, int64_t n_q, int64_t n_k, int queries_per_block,
                                                 int keys_per_tile, unsigned long long* map, hipStream_t stream)
{
	const int64_t q_blocks = (n_q + queries_per_block - 1) / queries_per_block;
	const int64_t groups = 4 * attention_tile_map_words(n_k, keys_per_tile);      // (those past the last tile write zeros)
	if (q_blocks * groups == 0) return hipSuccess;
	if (q_blocks * groups > 0x7FFFFFFFLL) return hipErrorInvalidValue;
	attention_mask_tile_map_kernel<T><<<dim3((unsigned)(q_blocks * groups)), dim3(1024), 0, stream>>>(
		mask, mask_stride, (int)n_q, (int)n_k, queries_per_block, keys_per_tile, (int)groups, reinterpret_cast<unsigned short*>(map));
	return hipGetLastError();
}

// The first set tile at or after t, up to t_last; t_last + 1 when there is none.  map_row: the words of the query block
// (nullptr: every tile counts as set).  Block-uniform arguments, scalar loads.
__device__ __forceinline__ int attention_next_visible_tile(const unsigned long long* __restrict__ map_row, int t, int t_last)
{
	if (map_row == nullptr) return t;
	while (t <= t_last)
	{
		const unsigned long long bits = map_row[t >> 6] >> (t & 63);
		if (bits != 0)
		{
			const int found = t + __builtin_ctzll(bits);
			return found <= t_last ? found : t_last + 1;
		}
		t = (t | 63) + 1;
	}
	return t_last + 1;
}

// The share of part `part` of `parts` among the set tiles of [t_first, t_last]: narrows the range to the set tiles number
// part * per .. (part + 1) * per - 1, per = ceil(set tiles / parts), so that the parts of a query block's key range carry
// equal numbers of visible tiles wherever the mask hides the others (a sliding window over a long cache leaves most
// equal parts of the RANGE empty).  An empty share comes back as t_first > t_last.  Block-uniform, scalar work.
__device__ __forceinline__ void attention_visible_share(const unsigned long long* __restrict__ map_row, int part, int parts,
                                                        int& t_first, int& t_last)
{
	if (t_first > t_last) return;
	const int w_first = t_first >> 6, w_last = t_last >> 6;
	auto word_in_range = [&](int w) {
		unsigned long long bits = map_row[w];
		if (w == w_first) bits &= ~0ull << (t_first & 63);
		if (w == w_last && (t_last & 63) != 63) bits &= (1ull << ((t_last & 63) + 1)) - 1;
		return bits;
	};
	int total = 0;
	for (int w = w_first; w <= w_last; ++w) total += __builtin_popcountll(word_in_range(w));
	const int per = (total + parts - 1) / parts;
	const int lo = part * per;
	const int hi = lo + per < total ? lo + per : total;           // set tiles lo .. hi - 1
	if (per == 0 || lo >= hi)
	{
		t_first = t_last + 1;
		return;
	}
	// tile index of the set bit number `nth` (counted from 0) of the range
	auto locate = [&](int nth) {
		for (int w = w_first; w <= w_last; ++w)
		{
			unsigned long long bits = word_in_range(w);
			const int here = __builtin_popcountll(bits);
			if (nth >= here)
			{
				nth -= here;
				continue;
			}
			for (; nth > 0; --nth) bits &= bits - 1;
			return 64 * w + __builtin_ctzll(bits);
		}
		return t_last;                                            // (not reached: nth < total)
	};
	const int first = locate(lo), last = locate(hi - 1);
	t_first = first;
	t_last = last;
}

}  // namespace anygpu
