// Which (head, query block) a block of a fused attention launch works on.
//
// Blocks are dispatched to the 8 XCDs in turn (block id % 8), each XCD has its own L2, and a query block of one head
// reads the same K / V tiles as its neighbours (their windows overlap) and as the other query heads of its key / value
// group (exactly the same tiles).  The natural (query block, head) grid hands neighbours to different XCDs, so every
// L2 fetches every tile again, and it runs through the query blocks of one head, heavy to light, before it starts
// the next head, so that under a causal mask light blocks of one head are dispatched before heavy blocks of the next
// and the launch ends on a few long blocks.  Here the work is cut into UNITS of `chunk` adjacent query blocks times
// the q_per_kv heads of one group; units are dealt to the XCDs in turn, heaviest (latest query blocks) first over
// ALL heads, and the blocks of a unit follow each other on their XCD.  The even spread of the heavy blocks is what
// pays (8 heads x 8192 x 256 causal, fp16: 580 -> 391 us; 16 x 4096 x 128 causal, fp32: 1116 -> 660 us).
#pragma once

#include <cstdint>

#include <hip/hip_runtime.h>

namespace anygpu {

constexpr int kAttnXcds = 8;
// Blocks per unit.  Measured over 1 .. 64 on causal and windowed launches of all three head dimensions: 1 to 4 are
// alike and best, from 16 on the heavy blocks spread less evenly (32 heads x 2048 x 64 causal, fp16: 42 us against
// 56 us); the heads of a group always stay together.
constexpr int kAttnUnitBlocks = 4;

// Key splits.  Under a sliding window many query blocks walk the same, maximal number of key tiles, and when that number
// is a large share of what one CU gets of the whole launch, whole blocks cannot be packed evenly onto the CUs (8 heads x
// 8192 queries, window 4096: 256 blocks of 66 tiles and 256 of 2 .. 64 on 256 CUs last 66 + 64 tile times where the
// work averages 99).  The `n_split` latest query blocks of every head are therefore dispatched as two blocks, one per
// half of the key range, that leave unnormalised partial results for a merge kernel.  Dispatch order, heaviest first:
// the `n_big` unsplit blocks below the split range that still walk more tiles than a half, then the halves, then the rest.
struct AttnWalk
{
	int q_blocks;        // dispatched ("virtual") query blocks per head: the real ones + n_split
	int groups;          // key / value groups (batch x kv heads)
	int q_per_kv;        // query heads per group
	int chunk;           // adjacent query blocks per unit
	int chunks;          // units per group
	int units;           // chunks * groups
	int units_per_xcd;
	int real_q_blocks;   // query blocks per head
	int n_split;         // the latest n_split query blocks of a head are dispatched in two halves of their key range
	int n_big;           // unsplit blocks dispatched before the halves
	int parts_all;       // > 1: every query block is dispatched as that many blocks, one per part of its key range
};

// parts_all > 1 (launches with too few query blocks for the chip, long key ranges): n_split and n_big do not apply, the
// partial results are laid out as if every query block were a split one (slot = blocks from the last).
inline AttnWalk make_attn_walk(int64_t q_blocks, int64_t batch_heads, int64_t q_per_kv, int64_t n_split = 0, int64_t n_big = 0,
                               int64_t parts_all = 1)
{
	AttnWalk w;
	w.real_q_blocks = (int)q_blocks;
	w.parts_all = (int)parts_all;
	if (parts_all > 1)
	{
		n_split = q_blocks;
		n_big = 0;
	}
	w.n_split = (int)n_split;
	w.n_big = (int)n_big;
	w.q_blocks = parts_all > 1 ? (int)(q_blocks * parts_all) : (int)(q_blocks + n_split);
	w.q_per_kv = (int)q_per_kv;
	w.groups = (int)(batch_heads / q_per_kv);
	w.chunk = q_per_kv >= kAttnUnitBlocks ? 1 : (int)(kAttnUnitBlocks / q_per_kv);
	if (w.chunk > w.q_blocks) w.chunk = w.q_blocks;
	w.chunks = (w.q_blocks + w.chunk - 1) / w.chunk;
	w.units = w.chunks * w.groups;
	w.units_per_xcd = (w.units + kAttnXcds - 1) / kAttnXcds;
	return w;
}

inline int64_t attn_walk_blocks(const AttnWalk& w)
{
	return (int64_t)kAttnXcds * w.units_per_xcd * w.chunk * w.q_per_kv;
}

// false: a padding block (the last round of units or the last chunk of a head is not full).  part / parts: which half
// of the key range the block walks (parts = 1: all of it); split_slot numbers the split blocks of a head from the last.
__device__ __forceinline__ bool attn_walk_locate_part(const AttnWalk& w, unsigned block, int& head, int& q_block,
                                                      int& part, int& parts, int& split_slot);

__device__ __forceinline__ bool attn_walk_locate(const AttnWalk& w, unsigned block, int& head, int& q_block)
{
	int part, parts, slot;
	return attn_walk_locate_part(w, block, head, q_block, part, parts, slot);
}

__device__ __forceinline__ bool attn_walk_locate_part(const AttnWalk& w, unsigned block, int& head, int& q_block,
                                                      int& part, int& parts, int& split_slot)
{
	const int xcd = (int)(block % kAttnXcds);
	const int slot = (int)(block / kAttnXcds);
	const int per_unit = w.chunk * w.q_per_kv;
	const int unit = (slot / per_unit) * kAttnXcds + xcd;
	const int member = slot % per_unit;
	if (unit >= w.units) return false;
	const int chunk_index = w.chunks - 1 - unit / w.groups;       // late query blocks walk the most keys: first
	const int group = unit % w.groups;
	const int v_block = chunk_index * w.chunk + (w.chunk - 1 - member / w.q_per_kv);
	head = group * w.q_per_kv + member % w.q_per_kv;
	part = 0;
	parts = 1;
	split_slot = 0;
	q_block = v_block;
	if (v_block >= w.q_blocks) return false;
	if (w.parts_all > 1)
	{
		q_block = v_block / w.parts_all;
		part = v_block % w.parts_all;
		parts = w.parts_all;
		split_slot = w.real_q_blocks - 1 - q_block;
		return true;
	}
	if (w.n_split > 0)
	{
		const int rank = w.q_blocks - 1 - v_block;               // 0: dispatched first
		const int first_split = w.real_q_blocks - w.n_split;     // first split query block
		if (rank < w.n_big) q_block = first_split - 1 - rank;
		else if (rank < w.n_big + 2 * w.n_split)
		{
			split_slot = (rank - w.n_big) >> 1;
			part = (rank - w.n_big) & 1;
			parts = 2;
			q_block = w.real_q_blocks - 1 - split_slot;
		}
		else q_block = first_split - w.n_big - 1 - (rank - w.n_big - 2 * w.n_split);
	}
	return true;
}

}  // namespace anygpu
