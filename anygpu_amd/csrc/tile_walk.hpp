// Which tile of C a block of a tiled GEMM launch works on.
#pragma once

#include <hip/hip_runtime.h>

namespace anygpu {

constexpr int kNumXcd = 8;

// Tile -> block mapping.  Workgroups are dealt round-robin to the 8 XCDs (each with its own
// L2), so block b runs on XCD b % 8.  Blocks of one XCD get a contiguous range of tile
// numbers, and tile numbers walk the tile grid in column strips of kGroupM rows, so an XCD
// works on a compact patch of C and re-uses A and B slabs out of its own L2.
template <int kGroupM>
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn)
{
	// XCD x runs the blocks x, x + 8, ...: they get a contiguous range of tile ids (the first total % 8 XCDs one more)
	const int total = tiles_m * tiles_n;
	const int xcd = bid % kNumXcd, share = total / kNumXcd, extra = total % kNumXcd;
	const int id = xcd * share + (xcd < extra ? xcd : extra) + bid / kNumXcd;
	const int per_group = kGroupM * tiles_n;
	const int g = id / per_group;
	const int first_m = g * kGroupM;
	const int rows = min(kGroupM, tiles_m - first_m);
	const int in_group = id - g * per_group;
	tm = first_m + in_group % rows;
	tn = in_group / rows;
}

}  // namespace anygpu
