// Pieces shared by the band kernels (few left-operand rows against a weight matrix that is streamed once):
// constants, the MFMA wrappers, the K-split plan and the partial-sum workspace.
#pragma once

#include "device_utils.hpp"
#include "gemm_epilogue.hpp"
#include "launch.hpp"

namespace anygpu {
namespace band {

constexpr int kBandThreads = 256;
constexpr int kBandMaxSplits = 32;
constexpr int64_t kBandEnoughBlocks = 256;        // tiles from which K is not split
constexpr int64_t kBandWantedBlocks = 512;
// Workspace of a (device, stream) pair.  The cut along K of the tile kernels prices the traffic of its fp32 planes and
// uses all of it (2048 x 14336 . 14336 x 4096 fp16: two planes of 32 MB, 244 -> 184 us); the band kernels keep their
// partial sums within the first kBandPlanBytes: their plan does not price that traffic, and more splits than fit
// there lost (64 x 4096 . 4096 x 14336 fp32: 83 us with 2 splits, 95 us with 5).
constexpr size_t kBandPartialBytes = (size_t)64 << 20;
constexpr size_t kBandPlanBytes = (size_t)16 << 20;

typedef float4_t Vec;      // 16 raw bytes of either element type

template <typename T, int MR> struct BandMma;

template <> struct BandMma<float, 16>
{
	typedef float4_t Acc;
	static constexpr int kRegs = 4;
	__device__ static void mma(const Vec& w, const Vec& a, Acc& acc)
	{
#pragma unroll
		for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w[e], a[e], acc, 0, 0, 0);
	}
};

template <> struct BandMma<float, 32>
{
	typedef float16_t Acc;
	static constexpr int kRegs = 16;
	__device__ static void mma(const Vec& w, const Vec& a, Acc& acc)
	{
#pragma unroll
		for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(w[e], a[e], acc, 0, 0, 0);
	}
};

template <> struct BandMma<half_t, 16>
{
	typedef float4_t Acc;
	static constexpr int kRegs = 4;
	__device__ static void mma(const Vec& w, const Vec& a, Acc& acc)
	{
		acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, w), __builtin_bit_cast(half8_t, a), acc, 0, 0, 0);
	}
};

template <> struct BandMma<half_t, 32>
{
	typedef float16_t Acc;
	static constexpr int kRegs = 16;
	__device__ static void mma(const Vec& w, const Vec& a, Acc& acc)
	{
		acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, w), __builtin_bit_cast(half8_t, a), acc, 0, 0, 0);
	}
};

// Partial-sum workspace of one (device, stream) pair: kBandPartialBytes, allocated on first use and kept
// for the life of the process; NULL when there is none and none can be made now (stream under capture).
float* band_workspace(hipStream_t stream);

inline bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

// How K is cut over blockIdx.y when the column tiles alone do not fill the chip.
struct SplitPlan
{
	int64_t splits;
	int64_t chunks_per_split;
	float* partial;        // workspace for splits > 1
};

// `chunk`: K elements per LDS chunk of the band (splits are whole chunks), `rows`: band rows (padded),
// `elem_bytes`: weight element size, `acc_floats`: partial sums per thread and split.
inline SplitPlan plan_band_splits(int64_t tiles, int64_t K, int64_t chunk, int64_t rows, int elem_bytes, int acc_floats,
                                  hipStream_t stream)
{
	const int64_t kchunks = (K + chunk - 1) / chunk;
	int64_t splits = 1;
	if (tiles < kBandEnoughBlocks)
	{
		splits = (kBandWantedBlocks + tiles - 1) / tiles;
		if (splits > kBandMaxSplits) splits = kBandMaxSplits;
		// a split writes and reads back 8 bytes per sum where it streams depth * elem_bytes bytes of weights per
		// column: splits stay deep enough for the partial sums to be at most a quarter of the traffic
		const int64_t min_depth = 32 * rows / elem_bytes;
		const int64_t min_chunks = (min_depth + chunk - 1) / chunk;
		if (splits > kchunks / min_chunks) splits = kchunks / min_chunks;
		const int64_t room = (int64_t)(kBandPlanBytes / ((size_t)tiles * kBandThreads * acc_floats * sizeof(float)));
		if (splits > room) splits = room;
		if (splits < 1) splits = 1;
	}
	SplitPlan plan;
	plan.chunks_per_split = (kchunks + splits - 1) / splits;
	plan.splits = (kchunks + plan.chunks_per_split - 1) / plan.chunks_per_split;
	plan.partial = nullptr;
	if (plan.splits > 1)
	{
		plan.partial = band_workspace(stream);
		if (!plan.partial)
		{
			plan.splits = 1;
			plan.chunks_per_split = kchunks;
		}
	}
	return plan;
}

}  // namespace band
}  // namespace anygpu
