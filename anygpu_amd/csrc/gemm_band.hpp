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
constexpr int64_t kBandEnoughBlocks = 256;        // column tiles that fill the chip by themselves
// Workspace of a (device, stream) pair.  The cut along K of the tile kernels prices the traffic of its fp32 planes and
// uses all of it (2048 x 14336 . 14336 x 4096 fp16: two planes of 32 MB, 244 -> 184 us); the band kernels keep their
// partial sums within the first kBandPlanBytes: their plan does not price that traffic, and more splits than fit
// there lost (64 x 4096 . 4096 x 14336 fp32: 83 us with 2 splits, 95 us with 5).
constexpr size_t kBandPartialBytes = (size_t)64 << 20;
// Aligned copies of GEMM operands that the tile kernels cannot fetch as they lie may need more (4095^3 fp32: two copies
// of 64 MiB): for those the library's own buffer of a stream grows on demand, in steps of kBandPartialBytes, up to this.
constexpr size_t kBandCopyBytes = (size_t)1 << 30;
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

// Partial-sum workspace of a (device, stream) pair.  Either the caller has handed one in for the stream
// (anygpu_set_workspace: any size, the library then allocates nothing for that stream), or the library owns one of
// kBandPartialBytes, allocated the first time an eager launch on the stream cuts a product and kept until
// anygpu_release_workspaces or the end of the process.  A stream that is being captured into a graph uses a caller's
// workspace or none: a graph never records the library's own buffer, and what a captured launch computes does not depend
// on what ran on the stream before.
// workspace_capacity: bytes a launch on `stream` may plan partial sums for right now (0: run uncut), without allocating.
// workspace_acquire: the buffer of at least that size; allocates the library's own on first use and returns the error if
// that fails.
// workspace_copy_capacity: the same for operand copies, which may make the library's own buffer grow (up to
// kBandCopyBytes); workspace_acquire with `at_least` > 0 returns a buffer of at least that many bytes, reallocating the
// library's own if it is smaller (hipFree waits for the device, so nothing still uses the old one).
size_t workspace_capacity(hipStream_t stream);
size_t workspace_copy_capacity(hipStream_t stream);
hipError_t workspace_acquire(hipStream_t stream, float** base, size_t at_least = 0);
// While one of these lives, the calling thread's view of every workspace starts `bytes` (rounded up to 256) further on:
// a launcher that has parked operand copies at the front of the stream's workspace calls the ordinary launchers
// underneath it, whose partial sums then go behind the copies.  The launcher holds pointers into the buffer, so while a
// reservation lives the library's own buffer does not grow: both capacities report what is left of it as it is.
class WorkspaceReserve
{
public:
	explicit WorkspaceReserve(size_t bytes);
	~WorkspaceReserve();
	WorkspaceReserve(const WorkspaceReserve&) = delete;
	WorkspaceReserve& operator=(const WorkspaceReserve&) = delete;

private:
	size_t previous_;
};
// the C ABI's anygpu_set_workspace / anygpu_release_workspaces
int workspace_set(hipStream_t stream, void* base, size_t bytes);
hipError_t workspace_release_all();

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
inline hipError_t plan_band_splits(int64_t tiles, int64_t K, int64_t chunk, int64_t rows, int elem_bytes, int acc_floats,
                                   hipStream_t stream, SplitPlan* out)
{
	const int64_t kchunks = (K + chunk - 1) / chunk;
	int64_t splits = 1;
	const int64_t cus = device_cu_count();
	// Every count of ranges is priced: the blocks of a launch run side by side, a CU's share of the memory bandwidth is
	// what its blocks divide, so the launch lasts as long as the CU with the most blocks needs for them (one block alone
	// does not keep enough loads in flight: priced like two); a cut adds the merge launch and the planes' traffic.
	// (Before: as many ranges as bring the blocks to 512.  32 x 36864 -> 4608 fp32: 141 -> 130 us, [K, N] 139 -> 123; 24 x 5120 ->
	// 65536 [K, N]: 233 -> 221; 16 x 4608 -> 36864, 288 tiles, now in two ranges: 167 -> 141; a few small products lose a
	// microsecond.)
	const size_t capacity = tiles < 2 * kBandEnoughBlocks ? workspace_capacity(stream) : 0;
	if (capacity > 0 && cus > 0)
	{
		const int64_t min_depth = 32 * rows / elem_bytes;
		const int64_t min_chunks = (min_depth + chunk - 1) / chunk;
		const size_t plan_bytes = capacity < kBandPlanBytes ? capacity : kBandPlanBytes;
		const double tile_sums = (double)kBandThreads * (double)acc_floats;
		const int64_t room = (int64_t)((double)plan_bytes / ((double)tiles * tile_sums * sizeof(float)));
		int64_t most = kchunks / min_chunks;
		if (most > kBandMaxSplits) most = kBandMaxSplits;
		if (most > room) most = room;
		const double chunk_us = (double)chunk * tile_sums / (double)rows * (double)elem_bytes * (double)cus / 6.4e6;
		double best = 0.0;
		for (int64_t s = 1; s <= most || s == 1; ++s)
		{
			const int64_t per = (kchunks + s - 1) / s;
			const int64_t ranges = (kchunks + per - 1) / per;
			if (ranges != s) continue;
			const int64_t most_per_cu = (tiles * ranges + cus - 1) / cus;
			double us = (double)(most_per_cu < 2 ? 2 : most_per_cu) * (double)per * chunk_us;
			if (ranges > 1) us += 4.6 + 8.0 * tile_sums * (double)tiles * (double)ranges / 5.0e6;
			if (s == 1 || us < 0.97 * best)
			{
				best = us;
				splits = ranges;
			}
		}
	}
	SplitPlan plan;
	plan.chunks_per_split = (kchunks + splits - 1) / splits;
	plan.splits = (kchunks + plan.chunks_per_split - 1) / plan.chunks_per_split;
	plan.partial = nullptr;
	if (plan.splits > 1)
	{
		const hipError_t err = workspace_acquire(stream, &plan.partial);
		if (err != hipSuccess) return err;
	}
	*out = plan;
	return hipSuccess;
}

}  // namespace band
}  // namespace anygpu
