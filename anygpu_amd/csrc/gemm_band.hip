// Products with a band of few left-operand rows (M <= 64: a short prompt, a small decode batch) against
// k-contiguous weights (column-major B, [N, K]).  The weight matrix dominates the traffic and has to be
// streamed from HBM once at full rate; a square MFMA tile of 64 or 128 rows would spend most of its matrix
// cycles on padding and leave the loads waiting behind them.
//
// Here the band of A rows is one MFMA operand of 16 or 32 rows (two of 32 for 33 .. 64 rows, which share every
// weight register) and the weights never pass through LDS:
// every lane loads 16-byte vectors of "its" weight row straight into the MFMA operand registers.  The
// k index inside an MFMA is a dummy index, so the lanes are free to take any k they like as long as both
// operands agree: with G lane groups (4 in the 16-row form, 2 in the 32-row form) load i of lane group g
// takes the 16 bytes (i * G + g) * 16 .. of each k step, so that one load instruction reads 64 or 32
// contiguous bytes of every weight row, four of them a contiguous run of 256 or 128 bytes, and the matching
// A values are read from an LDS copy of the band with the same addressing.  A block of 4 waves covers 128 output columns
// (32 per wave) and shares the band chunk in LDS; the loads of the next k step are in flight while the
// current one is multiplied.
//
// Weight matrices with few rows do not have 128-column tiles for every CU, so K is split over blockIdx.y:
// each split writes its partial sums (in register layout) to a workspace and a second small kernel adds
// them in split order, applies the epilogue and stores.  (Finishing in the last block to arrive, behind a
// ticket counter, needs a device-scope fence per block; with one L2 per XCD that fence writes the L2 back
// and cost more than the whole product: 60 - 90 us against 20.)  The workspace belongs to the
// (device, stream) pair, is allocated on first use and kept for the life of the process, like the
// workspace of a BLAS handle; a stream that is being captured and has none yet runs without the split.
#include "gemm_band.hpp"
#include "anygpu_hip.h"

#include <map>
#include <mutex>
#include <type_traits>
#include <utility>

namespace anygpu {

using namespace band;

namespace {

constexpr int kBandCols = 128;                    // output columns per block, 32 per wave

template <typename T, int MR, int MB>
struct BandShape
{
	static constexpr int kEV = 16 / (int)sizeof(T);      // elements per vector
	static constexpr int kGroups = kWaveSize / MR;        // lane groups along k
	static constexpr int kStepVecs = 4 * kGroups;         // vectors of one row per k step
	static constexpr int kStep = kStepVecs * kEV;         // elements per k step
	static constexpr int kRows = MR * MB;                 // band rows: MB MFMA row blocks of MR
	static constexpr int kStepsPerChunk = 4 / MB;         // an LDS chunk of the band is always 1024 vectors
	static constexpr int kChunkVecs = kStepsPerChunk * kStepVecs;
	static constexpr int kChunk = kChunkVecs * kEV;       // elements of K per LDS chunk of the band
	static constexpr int kPitchVecs = kChunkVecs + 1;     // LDS row pitch: 16 bytes of padding
	static constexpr int kNG = 32 / MR;                   // MFMA column groups per wave
};

// one store instruction at element alignment: rows of C need not be multiples of four elements long
typedef float4_t LooseFloat4 __attribute__((aligned(4)));
typedef half4_t LooseHalf4 __attribute__((aligned(2)));
__device__ __forceinline__ void store4(float* dst, const float4_t& v) { *reinterpret_cast<LooseFloat4*>(dst) = v; }
__device__ __forceinline__ void store4(half_t* dst, const float4_t& v)
{
	*reinterpret_cast<LooseHalf4*>(dst) = half4_t{(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
}

// Epilogue and store of one thread's sums.  Register 4 q + e of a lane: column 4 * grp + e (16-row form) or
// 8 q + 4 * grp + e (32-row form) of the MFMA column group, band row idx.
template <typename T, int MR, int MB, int EPI, typename Acc>
__device__ __forceinline__ void band_store(const Acc (*acc)[MB], const T* __restrict__ bias, T* __restrict__ C,
                                           int M, int64_t N, int64_t ldc, int64_t n0, int idx, int grp, float ep_param)
{
	using S = BandShape<T, MR, MB>;
	constexpr bool DUAL = (EPI == kEpiGeluMul);
	constexpr int kRegs = BandMma<T, MR>::kRegs;
#pragma unroll
	for (int b = 0; b < MB; ++b)
	{
		const int m = b * MR + idx;
		if (m >= M) continue;
#pragma unroll
		for (int j = 0; j < S::kNG; ++j)
#pragma unroll
			for (int q = 0; q < kRegs / 4; ++q)
			{
				const int64_t n = n0 + j * MR + (MR == 16 ? 4 * grp : 8 * q + 4 * grp);
				float4_t out;
#pragma unroll
				for (int e = 0; e < 4; ++e)
				{
					const float sum2 = DUAL ? acc[DUAL ? S::kNG + j : 0][b][4 * q + e] : 0.0f;
					const float bias_n = (EPI == kEpiBias && bias && n + e < N) ? (float)bias[n + e] : 0.0f;
					out[e] = finish_sum<EPI>(acc[j][b][4 * q + e], sum2, bias_n, ep_param);
				}
				T* dst = C + (int64_t)m * ldc + n;
				if (n + 4 <= N) store4(dst, out);
				else
				{
#pragma unroll
					for (int e = 0; e < 4; ++e)
						if (n + e < N) dst[e] = (T)out[e];
				}
			}
	}
}

// C[m, n] = finish(sum_k A[m, k] * B[n, k]), M <= MR * MB.  grid (tiles of 128 columns, splits of K);
// `chunks_per_split` LDS chunks of K per split.  With gridDim.y > 1 the sums of split y go to
// partial[tile][y][thread][register] and gemm_band_merge_kernel finishes.
template <typename T, int MR, int MB, int EPI>
__global__ __launch_bounds__(kBandThreads) void gemm_band_kernel(
	const T* __restrict__ A, const T* __restrict__ B, const T* __restrict__ B2, const T* __restrict__ bias,
	T* __restrict__ C, float* __restrict__ partial,
	int M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int chunks_per_split, float ep_param)
{
	using S = BandShape<T, MR, MB>;
	using Mma = BandMma<T, MR>;
	using Acc = typename Mma::Acc;
	constexpr bool DUAL = (EPI == kEpiGeluMul);
	constexpr int kW = S::kNG * (DUAL ? 2 : 1);          // weight rows per lane

	__shared__ Vec band[2][S::kRows * S::kPitchVecs];

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = tid >> 6;
	const int idx = lane % MR;                            // weight row (as W operand) / band row (as A operand)
	const int grp = lane / MR;
	const int64_t n0 = (int64_t)blockIdx.x * kBandCols + wave * 32;

	const int64_t kb = (int64_t)blockIdx.y * chunks_per_split * S::kChunk;
	const int64_t ke_want = kb + (int64_t)chunks_per_split * S::kChunk;
	const int64_t ke = ke_want < K ? ke_want : K;

	// weight row pointers of this lane; rows past the end are replaced by the last one (never stored)
	const T* wrow[kW];
#pragma unroll
	for (int j = 0; j < S::kNG; ++j)
	{
		int64_t n = n0 + j * MR + idx;
		n = n < N ? n : N - 1;
		wrow[j] = B + n * ldb;
		if constexpr (DUAL) wrow[S::kNG + j] = B2 + n * ldb;
	}

	// Weight vectors of one k step.  GUARDED: vectors at or past the end of the k range are fetched from the
	// start of the range instead (a valid address) and zeroed by mask_w before they are multiplied; the selects
	// sit at the use so that the loads stay in flight over the previous step.
	Vec wr[2][kW][4];
	const Vec zero = {0.0f, 0.0f, 0.0f, 0.0f};
	auto issue_w = [&](Vec (&dst)[kW][4], int64_t step, auto guarded) {
		const int64_t k0 = kb + step * S::kStep + grp * S::kEV;
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			const int64_t k = k0 + i * S::kGroups * S::kEV;
			const int64_t kk = (decltype(guarded)::value && k >= ke) ? kb : k;
#pragma unroll
			for (int j = 0; j < kW; ++j) dst[j][i] = *reinterpret_cast<const Vec*>(wrow[j] + kk);
		}
	};
	auto mask_w = [&](Vec (&w)[kW][4], int64_t step) {
		const int64_t k0 = kb + step * S::kStep + grp * S::kEV;
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			const bool valid = k0 + i * S::kGroups * S::kEV < ke;
#pragma unroll
			for (int j = 0; j < kW; ++j) w[j][i] = valid ? w[j][i] : zero;
		}
	};

	// the band chunk: kRows rows x kChunkVecs vectors = 1024 vectors, 4 per thread; rows past M and k past the
	// range are fetched from valid addresses and zeroed on their way into LDS
	Vec ar[4];
	auto issue_band = [&](int chunk) {
		const int64_t kc = kb + (int64_t)chunk * S::kChunk;
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			const int q = tid + kBandThreads * i;
			const int row = q / S::kChunkVecs;
			const int64_t k = kc + (q % S::kChunkVecs) * S::kEV;
			ar[i] = *reinterpret_cast<const Vec*>(A + (int64_t)(row < M ? row : M - 1) * lda + (k < ke ? k : kb));
		}
	};
	auto stage_band = [&](int slot, int chunk) {
		const int64_t kc = kb + (int64_t)chunk * S::kChunk;
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			const int q = tid + kBandThreads * i;
			const int row = q / S::kChunkVecs;
			const bool valid = row < M && kc + (q % S::kChunkVecs) * S::kEV < ke;
			band[slot & 1][row * S::kPitchVecs + (q % S::kChunkVecs)] = valid ? ar[i] : zero;
		}
	};

	Acc acc[kW][MB];
#pragma unroll
	for (int j = 0; j < kW; ++j)
#pragma unroll
		for (int b = 0; b < MB; ++b)
#pragma unroll
			for (int r = 0; r < Mma::kRegs; ++r) acc[j][b][r] = 0.0f;

	auto multiply = [&](const Vec (&w)[kW][4], int buf, int s) {
		Vec a[MB][4];
#pragma unroll
		for (int b = 0; b < MB; ++b)
		{
			const Vec* src = &band[buf][(b * MR + idx) * S::kPitchVecs + s * S::kStepVecs + grp];
#pragma unroll
			for (int i = 0; i < 4; ++i) a[b][i] = src[i * S::kGroups];
		}
#pragma unroll
		for (int i = 0; i < 4; ++i)
#pragma unroll
			for (int j = 0; j < kW; ++j)
#pragma unroll
				for (int b = 0; b < MB; ++b) Mma::mma(w[j][i], a[b][i], acc[j][b]);
	};

	using Plain = std::false_type;
	using Guarded = std::true_type;
	const int full_chunks = (int)((ke - kb) / S::kChunk);          // chunks whose every vector lies inside the range
	const bool tail = (ke - kb) % S::kChunk != 0;

	// Blocks walk the full chunks of their k range from different starting chunks and wrap around (the chunk with
	// the ragged end, if any, comes last for all): blocks that run side by side then read different parts of their
	// weight rows at any one time.  With weight rows a power of two apart, equal offsets in all rows are addresses
	// that share their low bits, and with them the memory channel.
	const int first = full_chunks > 1 ? (int)(((blockIdx.x + 977u * blockIdx.y) * 2654435761u >> 8) % (unsigned)full_chunks) : 0;
	auto chunk_at = [&](int i) {                            // i <= full_chunks; i == full_chunks: the chunk after them
		if (i >= full_chunks) return i;
		const int c = i + first;
		return c >= full_chunks ? c - full_chunks : c;
	};
	issue_band(chunk_at(0));
	if (full_chunks > 0) issue_w(wr[0], (int64_t)chunk_at(0) * S::kStepsPerChunk, Plain{});
	stage_band(0, chunk_at(0));
	__syncthreads();
	for (int c = 0; c < full_chunks; ++c)
	{
		const int64_t here = (int64_t)chunk_at(c) * S::kStepsPerChunk;       // first step of this chunk
		// after the last full step the same step is fetched again and dropped
		const int64_t after = c + 1 < full_chunks ? (int64_t)chunk_at(c + 1) * S::kStepsPerChunk : here + S::kStepsPerChunk - 1;
		issue_band(chunk_at(c + 1));             // past the end: zeros, staged into a buffer nobody reads
#pragma unroll
		for (int s = 0; s < S::kStepsPerChunk; ++s)
		{
			// the loads of the next step are issued before this step's MFMAs
			issue_w(wr[(s + 1) & 1], s + 1 < S::kStepsPerChunk ? here + s + 1 : after, Plain{});
			__builtin_amdgcn_sched_barrier(0);
			multiply(wr[s & 1], c & 1, s);
		}
		stage_band(c + 1, chunk_at(c + 1));
		__syncthreads();
	}
	if (tail)
	{
		const int c = full_chunks;
		issue_w(wr[0], (int64_t)c * S::kStepsPerChunk, Guarded{});
#pragma unroll
		for (int s = 0; s < S::kStepsPerChunk; ++s)
		{
			const int64_t step = (int64_t)c * S::kStepsPerChunk + s;
			issue_w(wr[(s + 1) & 1], step + 1, Guarded{});
			__builtin_amdgcn_sched_barrier(0);
			mask_w(wr[s & 1], step);
			multiply(wr[s & 1], c & 1, s);
		}
	}

	if (gridDim.y > 1)
	{
		constexpr int kAccFloats = kW * MB * Mma::kRegs;
		float* mine = partial + (((int64_t)blockIdx.x * gridDim.y + blockIdx.y) * kBandThreads + tid) * kAccFloats;
#pragma unroll
		for (int j = 0; j < kW; ++j)
#pragma unroll
			for (int b = 0; b < MB; ++b)
#pragma unroll
				for (int r = 0; r < Mma::kRegs; r += 4)
					*reinterpret_cast<float4_t*>(mine + (j * MB + b) * Mma::kRegs + r) =
						float4_t{acc[j][b][r], acc[j][b][r + 1], acc[j][b][r + 2], acc[j][b][r + 3]};
		return;
	}
	band_store<T, MR, MB, EPI>(acc, bias, C, M, N, ldc, n0, idx, grp, ep_param);
}

// Adds the partial sums of the `splits` K ranges in split order and finishes.  One thread per output vector of four
// columns (tile, thread of gemm_band_kernel, column group, row block, register quad), so that the short,
// latency-bound job is spread over many waves; the loads of four splits are in flight together and added in order.
template <typename T, int MR, int MB, int EPI>
__global__ __launch_bounds__(kBandThreads) void gemm_band_merge_kernel(
	const float* __restrict__ partial, const T* __restrict__ bias, T* __restrict__ C,
	int M, int64_t N, int64_t ldc, int splits, int64_t tiles, float ep_param)
{
	using S = BandShape<T, MR, MB>;
	using Mma = BandMma<T, MR>;
	constexpr bool DUAL = (EPI == kEpiGeluMul);
	constexpr int kMats = DUAL ? 2 : 1;
	constexpr int kQuads = Mma::kRegs / 4;
	constexpr int kItems = S::kNG * MB * kQuads;            // output vectors per thread of the product kernel
	constexpr int kAccFloats = kMats * kItems * 4;
	const int64_t item = (int64_t)blockIdx.x * kBandThreads + threadIdx.x;
	const int q = (int)(item % kItems);
	const int tid = (int)((item / kItems) % kBandThreads);
	const int64_t tile = item / (kItems * kBandThreads);
	if (tile >= tiles) return;
	const int j = q / (MB * kQuads), b = (q / kQuads) % MB, quad = q % kQuads;
	const int lane = tid & (kWaveSize - 1);
	const int m = b * MR + lane % MR;
	const int grp = lane / MR;
	const int64_t n = tile * kBandCols + (tid >> 6) * 32 + j * MR + (MR == 16 ? 4 * grp : 8 * quad + 4 * grp);
	if (m >= M || n >= N) return;

	const int64_t stride = (int64_t)kBandThreads * kAccFloats;
	const float* src = partial + (tile * splits * kBandThreads + tid) * kAccFloats + q * 4;
	float4_t sum[kMats];
#pragma unroll
	for (int w = 0; w < kMats; ++w) sum[w] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
	int sp = 0;
	for (; sp + 4 <= splits; sp += 4)
	{
		float4_t v[4][kMats];
#pragma unroll
		for (int i = 0; i < 4; ++i)
#pragma unroll
			for (int w = 0; w < kMats; ++w)
				v[i][w] = *reinterpret_cast<const float4_t*>(src + (sp + i) * stride + w * kItems * 4);
#pragma unroll
		for (int i = 0; i < 4; ++i)
#pragma unroll
			for (int w = 0; w < kMats; ++w) sum[w] += v[i][w];
	}
	for (; sp < splits; ++sp)
#pragma unroll
		for (int w = 0; w < kMats; ++w) sum[w] += *reinterpret_cast<const float4_t*>(src + sp * stride + w * kItems * 4);

	float4_t out;
#pragma unroll
	for (int e = 0; e < 4; ++e)
	{
		const float bias_n = (EPI == kEpiBias && bias && n + e < N) ? (float)bias[n + e] : 0.0f;
		out[e] = finish_sum<EPI>(sum[0][e], sum[kMats - 1][e], bias_n, ep_param);
	}
	T* dst = C + (int64_t)m * ldc + n;
	if (n + 4 <= N) store4(dst, out);
	else
	{
#pragma unroll
		for (int e = 0; e < 4; ++e)
			if (n + e < N) dst[e] = (T)out[e];
	}
}

template <typename T, int MR, int MB, int EPI>
hipError_t launch_band(const T* A, const T* B, const T* B2, const T* bias, T* C, int M, int64_t N, int64_t K,
                       int64_t lda, int64_t ldb, int64_t ldc, float ep_param, hipStream_t stream)
{
	using S = BandShape<T, MR, MB>;
	constexpr int kAccFloats = S::kNG * (EPI == kEpiGeluMul ? 2 : 1) * MB * BandMma<T, MR>::kRegs;
	const int64_t tiles = (N + kBandCols - 1) / kBandCols;
	SplitPlan plan;
	const hipError_t plan_err = plan_band_splits(tiles, K, S::kChunk, S::kRows, (int)sizeof(T), kAccFloats, stream, &plan);
	if (plan_err != hipSuccess) return plan_err;
	const int64_t splits = plan.splits, chunks_per_split = plan.chunks_per_split;
	float* partial = plan.partial;
	discard_stale_error();
	gemm_band_kernel<T, MR, MB, EPI><<<dim3((unsigned)tiles, (unsigned)splits), dim3(kBandThreads), 0, stream>>>(
		A, B, B2, bias, C, partial, M, N, K, lda, ldb, ldc, (int)chunks_per_split, ep_param);
	if (splits > 1)
	{
		const int64_t items = tiles * kBandThreads * (kAccFloats / (EPI == kEpiGeluMul ? 8 : 4));
		gemm_band_merge_kernel<T, MR, MB, EPI><<<dim3((unsigned)((items + kBandThreads - 1) / kBandThreads)), dim3(kBandThreads), 0, stream>>>(
			partial, bias, C, M, N, ldc, (int)splits, tiles, ep_param);
	}
	return hipGetLastError();
}

}  // namespace

// ---------------------------------------------------------------------------------------------
// Partial-sum workspaces, one per (device, stream) pair that has cut a product or been given one.
// ---------------------------------------------------------------------------------------------
namespace {

struct WorkspaceEntry
{
	float* base;
	size_t bytes;
	bool from_caller;
	uint64_t last_use;                        // value of use_clock at the entry's last acquisition
};

std::mutex workspace_lock;
std::map<std::pair<int, hipStream_t>, WorkspaceEntry> workspaces;
uint64_t use_clock = 0;
// The library keeps at most this many buffers of its own (ANYGPU_MAX_OWN_WORKSPACES in the header); a stream beyond that
// takes over the place of the one used longest ago.
constexpr size_t kMaxOwnWorkspaces = 8;

bool stream_is_capturing(hipStream_t stream)
{
	hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
	if (hipStreamIsCapturing(stream, &capture) != hipSuccess)
	{
		(void)hipGetLastError();
		return true;                          // (a stream whose state cannot be read is treated like one under capture)
	}
	return capture != hipStreamCaptureStatusNone;
}

}  // namespace

namespace {
thread_local size_t reserved_front = 0;      // bytes at the front of every workspace this thread's launches leave alone
}

band::WorkspaceReserve::WorkspaceReserve(size_t bytes) : previous_(reserved_front)
{
	reserved_front += (bytes + 255) / 256 * 256;
}

band::WorkspaceReserve::~WorkspaceReserve()
{
	reserved_front = previous_;
}

namespace {
// bytes the stream's workspace offers: a caller's buffer as it is; the library's own `own_bytes`, to eager launches only
size_t capacity_of(hipStream_t stream, size_t own_bytes)
{
	int device = 0;
	if (hipGetDevice(&device) != hipSuccess) return 0;
	size_t bytes = 0;
	bool fixed = false;
	{
		std::lock_guard<std::mutex> guard(workspace_lock);
		const auto found = workspaces.find(std::make_pair(device, stream));
		// a caller's buffer is what it is; so is the library's own while a launcher above holds pointers into it (a
		// reserved front): growing it would free what they point at
		if (found != workspaces.end() && (found->second.from_caller || reserved_front > 0))
		{
			bytes = found->second.bytes;
			fixed = true;
		}
	}
	if (!fixed) bytes = (stream_is_capturing(stream) || reserved_front > 0) ? 0 : own_bytes;
	return bytes > reserved_front ? bytes - reserved_front : 0;
}
}  // namespace

size_t band::workspace_capacity(hipStream_t stream) { return capacity_of(stream, kBandPartialBytes); }
size_t band::workspace_copy_capacity(hipStream_t stream) { return capacity_of(stream, kBandCopyBytes); }

hipError_t band::workspace_acquire(hipStream_t stream, float** base, size_t at_least)
{
	*base = nullptr;
	int device = 0;
	hipError_t err = hipGetDevice(&device);
	if (err != hipSuccess) return err;
	std::lock_guard<std::mutex> guard(workspace_lock);
	const auto key = std::make_pair(device, stream);
	// what the library's own buffer has to hold: the reserved front and `at_least` behind it, in whole steps
	size_t want = reserved_front + at_least;
	want = want <= kBandPartialBytes ? kBandPartialBytes : (want + kBandPartialBytes - 1) / kBandPartialBytes * kBandPartialBytes;
	const auto found = workspaces.find(key);
	if (found != workspaces.end())
	{
		if (found->second.from_caller || found->second.bytes >= want)
		{
			found->second.last_use = ++use_clock;
			*base = reinterpret_cast<float*>(reinterpret_cast<char*>(found->second.base) + reserved_front);
			return hipSuccess;
		}
		// the library's own buffer is too small for this copy: a larger one takes its place (never under a launcher
		// that holds pointers into it; the capacities above say so beforehand)
		if (reserved_front > 0) return hipErrorInvalidValue;
		const hipError_t freed = hipFree(found->second.base);
		if (freed != hipSuccess)
		{
			(void)hipGetLastError();
			return freed;
		}
		workspaces.erase(found);
	}
	// Streams come and go and the library does not see them go: when it already owns its limit of buffers, the one
	// used longest ago makes way.  hipFree waits for the device, so work that may still use that buffer has finished.
	size_t own = 0;
	auto oldest = workspaces.end();
	for (auto it = workspaces.begin(); it != workspaces.end(); ++it)
	{
		if (it->second.from_caller) continue;
		++own;
		if (oldest == workspaces.end() || it->second.last_use < oldest->second.last_use) oldest = it;
	}
	if (own >= kMaxOwnWorkspaces && oldest != workspaces.end())
	{
		int current = device;
		if (oldest->first.first != device) (void)hipSetDevice(oldest->first.first);
		const hipError_t freed = hipFree(oldest->second.base);
		if (oldest->first.first != device) (void)hipSetDevice(current);
		if (freed != hipSuccess)
		{
			(void)hipGetLastError();
			return freed;
		}
		workspaces.erase(oldest);
	}
	// First cut on this stream.  Another thread may be capturing some other stream in the global mode, in which an
	// allocation made anywhere invalidates its capture: this thread allocates in the relaxed mode.
	hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
	(void)hipThreadExchangeStreamCaptureMode(&mode);
	void* mem = nullptr;
	err = hipMalloc(&mem, want);
	(void)hipThreadExchangeStreamCaptureMode(&mode);
	if (err != hipSuccess)
	{
		(void)hipGetLastError();
		return err;
	}
	workspaces.emplace(key, WorkspaceEntry{static_cast<float*>(mem), want, false, ++use_clock});
	*base = reinterpret_cast<float*>(static_cast<char*>(mem) + reserved_front);
	return hipSuccess;
}

int band::workspace_set(hipStream_t stream, void* base, size_t bytes)
{
	int device = 0;
	const hipError_t err = hipGetDevice(&device);
	if (err != hipSuccess) return (int)err;
	std::lock_guard<std::mutex> guard(workspace_lock);
	const auto key = std::make_pair(device, stream);
	const auto found = workspaces.find(key);
	if (found != workspaces.end())
	{
		// the library's own buffer of this stream makes way (the caller has made sure that nothing on the stream
		// still uses it)
		if (!found->second.from_caller)
		{
			const hipError_t freed = hipFree(found->second.base);
			if (freed != hipSuccess) return (int)freed;
		}
		workspaces.erase(found);
	}
	if (base != nullptr && bytes > 0) workspaces.emplace(key, WorkspaceEntry{static_cast<float*>(base), bytes, true, ++use_clock});
	return ANYGPU_OK;
}

hipError_t band::workspace_release_all()
{
	std::lock_guard<std::mutex> guard(workspace_lock);
	hipError_t result = hipSuccess;
	for (auto& entry : workspaces)
	{
		if (entry.second.from_caller) continue;
		int current = 0;
		(void)hipGetDevice(&current);
		if (current != entry.first.first) (void)hipSetDevice(entry.first.first);
		const hipError_t freed = hipFree(entry.second.base);
		if (freed != hipSuccess) result = freed;
		if (current != entry.first.first) (void)hipSetDevice(current);
	}
	workspaces.clear();
	return result;
}

template <typename T>
bool gemm_band_applies(const T* A, const T* B, const T* B2, const T* C, int64_t M, int64_t N, int64_t K,
                       int64_t lda, int64_t ldb, int64_t ldc, int b_layout)
{
	constexpr int EV = 16 / (int)sizeof(T);
	if (b_layout != ANYGPU_B_COL_MAJOR) return false;
	if (M < (sizeof(T) == 4 ? kBandMinRowsF32 : kBandMinRows) || M > kBandMaxRows || N < 1 || K < 1) return false;
	if ((N + kBandCols - 1) / kBandCols > 0x7FFFFFFFLL) return false;
	// 33 .. 64 rows: two row blocks per weight register.  Worth it where the weights dominate and the columns or a
	// deep K give the chip enough blocks (256000 x 2304 fp32, 64 rows: 711 us against 1238 us through the tiles;
	// 2304 x 9216: 63 against 160); small weight matrices are quicker through the tile kernels.
	if (M > 32 && N < kBandEnoughBlocks * kBandCols && K < 4096) return false;
	// 16-byte loads along K from every row of A and B; C is stored at element alignment
	(void)C;
	(void)ldc;
	return K % EV == 0 && lda % EV == 0 && ldb % EV == 0 && band::aligned16(A) && band::aligned16(B) && band::aligned16(B2);
}

template <typename T>
hipError_t launch_gemm_band(const T* A, const T* B, const T* B2, const T* bias, T* C,
                            int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                            int epilogue, float ep_param, hipStream_t stream)
{
#define ANYGPU_BAND_ROWS(MR, MB) \
	switch (epilogue) \
	{ \
	case kEpiSoftcap: return launch_band<T, MR, MB, kEpiSoftcap>(A, B, B2, bias, C, (int)M, N, K, lda, ldb, ldc, ep_param, stream); \
	case kEpiGeluMul: return launch_band<T, MR, MB, kEpiGeluMul>(A, B, B2, bias, C, (int)M, N, K, lda, ldb, ldc, ep_param, stream); \
	default: return launch_band<T, MR, MB, kEpiBias>(A, B, B2, bias, C, (int)M, N, K, lda, ldb, ldc, ep_param, stream); \
	}
	if (M <= 16) { ANYGPU_BAND_ROWS(16, 1) }
	if (M <= 32) { ANYGPU_BAND_ROWS(32, 1) }
	ANYGPU_BAND_ROWS(32, 2)
#undef ANYGPU_BAND_ROWS
}

template bool gemm_band_applies<float>(const float*, const float*, const float*, const float*, int64_t, int64_t, int64_t,
                                       int64_t, int64_t, int64_t, int);
template bool gemm_band_applies<half_t>(const half_t*, const half_t*, const half_t*, const half_t*, int64_t, int64_t, int64_t,
                                        int64_t, int64_t, int64_t, int);
template hipError_t launch_gemm_band<float>(const float*, const float*, const float*, const float*, float*, int64_t, int64_t, int64_t,
                                            int64_t, int64_t, int64_t, int, float, hipStream_t);
template hipError_t launch_gemm_band<half_t>(const half_t*, const half_t*, const half_t*, const half_t*, half_t*, int64_t, int64_t, int64_t,
                                             int64_t, int64_t, int64_t, int, float, hipStream_t);

}  // namespace anygpu
