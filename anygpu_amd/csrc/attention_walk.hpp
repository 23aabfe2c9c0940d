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

struct AttnWalk
{
	int q_blocks;        // query blocks per head
	int groups;          // key / value groups (batch x kv heads)
	int q_per_kv;        // query heads per group
	int chunk;           // adjacent query blocks per unit
	int chunks;          // units per group
	int units;           // chunks * groups
	int units_per_xcd;
};

inline AttnWalk make_attn_walk(int64_t q_blocks, int64_t batch_heads, int64_t q_per_kv)
{
	AttnWalk w;
	w.q_blocks = (int)q_blocks;
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

// false: a padding block (the last round of units or the last chunk of a head is not full)
__device__ __forceinline__ bool attn_walk_locate(const AttnWalk& w, unsigned block, int& head, int& q_block)
{
	const int xcd = (int)(block % kAttnXcds);
	const int slot = (int)(block / kAttnXcds);
	const int per_unit = w.chunk * w.q_per_kv;
	const int unit = (slot / per_unit) * kAttnXcds + xcd;
	const int member = slot % per_unit;
	if (unit >= w.units) return false;
	const int chunk_index = w.chunks - 1 - unit / w.groups;       // late query blocks walk the most keys: first
	const int group = unit % w.groups;
	q_block = chunk_index * w.chunk + (w.chunk - 1 - member / w.q_per_kv);
	head = group * w.q_per_kv + member % w.q_per_kv;
	return q_block < w.q_blocks;
}

}  // namespace anygpu
