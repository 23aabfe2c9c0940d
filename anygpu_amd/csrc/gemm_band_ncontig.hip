// Bands of few left-operand rows (M <= 64) against n-contiguous fp32 weights (row-major B, [K, N]: the
// layout of the reference's own linear layers).  As in the k-contiguous form the weights go straight from
// memory into MFMA operand registers and the band of A rows is shared through LDS; what changes is which
// index the 16-byte vectors run along.
//
// A lane of the weight operand stands for one output column slot i and one k slot g of the MFMA.  It loads
// the four columns 4 i .. 4 i + 3 of row k = 4 g + t (t = 0 .. 3: four loads), so a load instruction reads
// 256 or 512 contiguous bytes of each of the 4 or 2 weight rows it touches.  Element e of such a vector is
// the operand of its own MFMA with its own accumulator: accumulator e holds the columns 4 i + e, i.e. the
// column index is permuted between lanes and accumulators, which costs nothing because the four
// accumulators of a lane end up holding four consecutive columns and are stored as one vector.  The A
// operand of all four is the same: lane (row m, k slot g) takes A[m][4 g + t] from a 16-byte LDS read.
//
// A wave covers 4 x 16 or 4 x 32 columns.  With many columns the 4 waves of a block sit side by side
// (256 or 512 columns per block); with few, all 4 take the same columns and a quarter of every band chunk's
// k range each, and add their sums up through LDS at the end, which gives four times the waves for the same
// partial-sum traffic.  On top of that K is split over blockIdx.y and merged by a second kernel exactly as in
// the k-contiguous form.
#include "gemm_band.hpp"
#include "anygpu_hip.h"

#include <type_traits>

namespace anygpu {

using namespace band;

namespace {

template <int MR, int MB, int EPI, bool KW, int SETS = 4>
struct RowBandShape
{
	static constexpr bool kDual = (EPI == kEpiGeluMul);
	static constexpr int kMats = kDual ? 2 : 1;
	static constexpr int kGroups = kWaveSize / MR;            // k slots of an MFMA = lane groups
	static constexpr int kStep = 4 * kGroups;                 // k per step: four loads per lane and weight matrix
	static constexpr int kRows = MR * MB;
	static constexpr int kChunkVecs = 1024 / kRows;           // an LDS chunk of the band is 1024 vectors
	static constexpr int kChunk = 4 * kChunkVecs;             // in elements of K
	static constexpr int kStepsPerChunk = kChunk / kStep;
	static constexpr int kWaveSteps = KW ? kStepsPerChunk / 4 : kStepsPerChunk;   // steps of a chunk one wave takes
	static constexpr int kSets = kWaveSteps < 4 ? 2 : SETS;   // register sets: the loads run kSets - 1 steps ahead
	static constexpr int kPitchVecs = kChunkVecs + 1;
	static constexpr int kWaveCols = 4 * MR;
	static constexpr int kBlockCols = KW ? kWaveCols : 4 * kWaveCols;
	static constexpr int kRegs = BandMma<float, MR>::kRegs;
	static constexpr int kAccFloats = kMats * 4 * MB * kRegs;
	static_assert(kWaveSteps % kSets == 0, "the register set of a step is a compile-time constant");
	static_assert(!KW || kWaveSize * kAccFloats * 4 <= 2 * kRows * kPitchVecs * 16, "the sums of a wave fit the band buffers");
};

// 16 bytes at element alignment: weight rows and rows of C need not be multiples of four elements long
typedef float4_t LooseVec __attribute__((aligned(4)));

template <int MR>
__device__ __forceinline__ void mma1(float w, float a, typename BandMma<float, MR>::Acc& acc)
{
	if constexpr (MR == 16) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w, a, acc, 0, 0, 0);
	else acc = __builtin_amdgcn_mfma_f32_32x32x2f32(w, a, acc, 0, 0, 0);
}

// Epilogue and store.  Register r of accumulator e of a lane: column slot s = 4 * grp + r (16-row form) or
// 8 * (r / 4) + 4 * grp + r % 4 (32-row form), column n0 + 4 s + e; band row idx of row block b.
template <int MR, int MB, int EPI, typename Acc>
__device__ __forceinline__ void row_band_store(const Acc (*acc)[4][MB], const float* __restrict__ bias, float* __restrict__ C,
                                               int M, int64_t N, int64_t ldc, int64_t n0, int idx, int grp, float ep_param)
{
	using S = RowBandShape<MR, MB, EPI, false>;
#pragma unroll
	for (int b = 0; b < MB; ++b)
	{
		const int m = b * MR + idx;
		if (m >= M) continue;
#pragma unroll
		for (int r = 0; r < S::kRegs; ++r)
		{
			const int slot = (MR == 16) ? 4 * grp + r : 8 * (r / 4) + 4 * grp + r % 4;
			int64_t n = n0 + 4 * slot;
			if (n >= N) continue;
			if (n + 4 > N) n = N - 4;             // the lane that loaded this slot took the last four columns instead
			float4_t out;
#pragma unroll
			for (int e = 0; e < 4; ++e)
			{
				const float sum2 = S::kDual ? acc[S::kDual ? 1 : 0][e][b][r] : 0.0f;
				const float bias_n = (EPI == kEpiBias && bias) ? bias[n + e] : 0.0f;
				out[e] = finish_sum<EPI>(acc[0][e][b][r], sum2, bias_n, ep_param);
			}
			*reinterpret_cast<LooseVec*>(C + (int64_t)m * ldc + n) = out;
		}
	}
}

// C[m, n] = finish(sum_k A[m, k] * B[k, n]), M <= MR * MB, N >= 4.  grid (column tiles, splits of K).
// KW: the waves of a block share their columns and divide K.  With gridDim.y > 1 the sums go to
// partial[wave tile][split][lane][register].
template <int MR, int MB, int EPI, bool KW, int SETS>
__global__ __launch_bounds__(kBandThreads) void gemm_band_ncontig_kernel(
	const float* __restrict__ A, const float* __restrict__ B, const float* __restrict__ B2, const float* __restrict__ bias,
	float* __restrict__ C, float* __restrict__ partial,
	int M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int chunks_per_split, float ep_param)
{
	using S = RowBandShape<MR, MB, EPI, KW, SETS>;
	using Acc = typename BandMma<float, MR>::Acc;

	__shared__ Vec band_lds[2][S::kRows * S::kPitchVecs];

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = tid >> 6;
	const int idx = lane % MR;
	const int grp = lane / MR;
	const int64_t wave_tile = KW ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * 4 + wave;
	const int64_t n0 = wave_tile * S::kWaveCols;
	const int first_step = KW ? wave * S::kWaveSteps : 0;     // this wave's steps inside every chunk

	const int64_t kb = (int64_t)blockIdx.y * chunks_per_split * S::kChunk;
	const int64_t ke_want = kb + (int64_t)chunks_per_split * S::kChunk;
	const int64_t ke = ke_want < K ? ke_want : K;

	// the four columns of this lane; a vector that would cross or lie past the end of a row is moved back to the last
	// four columns (crossing: stored there, with the same values as its neighbour's; past: never stored)
	int64_t n_lane = n0 + 4 * idx;
	n_lane = n_lane + 4 <= N ? n_lane : N - 4;
	const float* wcol[S::kMats];
	wcol[0] = B + n_lane;
	if constexpr (S::kDual) wcol[1] = B2 + n_lane;

	// Weight vectors of one k step; GUARDED: rows at or past the end of the k range are fetched from its first
	// row instead and zeroed by mask_w before they are multiplied.
	Vec wr[S::kSets][S::kMats][4];
	const Vec zero = {0.0f, 0.0f, 0.0f, 0.0f};
	// `wstep` counts the steps of this wave: step wstep % kWaveSteps of its share of chunk wstep / kWaveSteps
	auto step_k = [&](int64_t wstep) {
		return kb + (wstep / S::kWaveSteps) * S::kChunk + (first_step + wstep % S::kWaveSteps) * S::kStep + 4 * grp;
	};
	auto issue_w = [&](Vec (&dst)[S::kMats][4], int64_t wstep, auto guarded) {
		const int64_t k0 = step_k(wstep);
#pragma unroll
		for (int t = 0; t < 4; ++t)
		{
			const int64_t k = k0 + t;
			const int64_t kk = (decltype(guarded)::value && k >= ke) ? kb : k;
#pragma unroll
			for (int w = 0; w < S::kMats; ++w) dst[w][t] = __builtin_nontemporal_load(reinterpret_cast<const LooseVec*>(wcol[w] + kk * ldb));
		}
	};
	auto mask_w = [&](Vec (&v)[S::kMats][4], int64_t wstep) {
		const int64_t k0 = step_k(wstep);
#pragma unroll
		for (int t = 0; t < 4; ++t)
		{
			const bool valid = k0 + t < ke;
#pragma unroll
			for (int w = 0; w < S::kMats; ++w) v[w][t] = valid ? v[w][t] : zero;
		}
	};

	// the band chunk: kRows rows x kChunkVecs vectors, 4 per thread; rows past M and k past the range are fetched
	// from valid addresses and zeroed on their way into LDS
	Vec ar[4];
	auto issue_band = [&](int chunk) {
		const int64_t kc = kb + (int64_t)chunk * S::kChunk;
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			const int q = tid + kBandThreads * i;
			const int row = q / S::kChunkVecs;
			const int64_t k = kc + (q % S::kChunkVecs) * 4;
			ar[i] = *reinterpret_cast<const Vec*>(A + (int64_t)(row < M ? row : M - 1) * lda + (k < ke ? k : kb));
		}
	};
	auto stage_band = [&](int chunk) {
		const int64_t kc = kb + (int64_t)chunk * S::kChunk;
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			const int q = tid + kBandThreads * i;
			const int row = q / S::kChunkVecs;
			const bool valid = row < M && kc + (q % S::kChunkVecs) * 4 < ke;
			band_lds[chunk & 1][row * S::kPitchVecs + (q % S::kChunkVecs)] = valid ? ar[i] : zero;
		}
	};

	Acc acc[S::kMats][4][MB];
#pragma unroll
	for (int w = 0; w < S::kMats; ++w)
#pragma unroll
		for (int e = 0; e < 4; ++e)
#pragma unroll
			for (int b = 0; b < MB; ++b)
#pragma unroll
				for (int r = 0; r < S::kRegs; ++r) acc[w][e][b][r] = 0.0f;

	auto multiply = [&](const Vec (&v)[S::kMats][4], int buf, int s) {
		Vec a[MB];
#pragma unroll
		for (int b = 0; b < MB; ++b)
			a[b] = band_lds[buf][(b * MR + idx) * S::kPitchVecs + (first_step + s) * (S::kStep / 4) + grp];
#pragma unroll
		for (int t = 0; t < 4; ++t)
#pragma unroll
			for (int w = 0; w < S::kMats; ++w)
#pragma unroll
				for (int e = 0; e < 4; ++e)
#pragma unroll
					for (int b = 0; b < MB; ++b) mma1<MR>(v[w][t][e], a[b][t], acc[w][e][b]);
	};

	using Plain = std::false_type;
	using Guarded = std::true_type;
	const int full_chunks = (int)((ke - kb) / S::kChunk);
	const bool tail = (ke - kb) % S::kChunk != 0;
	const int64_t last_full_step = (int64_t)full_chunks * S::kWaveSteps - 1;

	constexpr int kAhead = S::kSets - 1;
	issue_band(0);
	if (full_chunks > 0)
	{
#pragma unroll
		for (int d = 0; d < kAhead; ++d) issue_w(wr[d], d < last_full_step ? d : last_full_step, Plain{});
	}
	stage_band(0);
	__syncthreads();
	for (int c = 0; c < full_chunks; ++c)
	{
		issue_band(c + 1);                       // past the end: zeros, staged into a buffer nobody reads
#pragma unroll
		for (int s = 0; s < S::kWaveSteps; ++s)
		{
			// the loads of step s + kAhead are issued before the MFMAs of step s; steps past the last full one
			// fetch that one again and are dropped
			const int64_t next = (int64_t)c * S::kWaveSteps + s + kAhead;
			issue_w(wr[(s + kAhead) % S::kSets], next < last_full_step ? next : last_full_step, Plain{});
			__builtin_amdgcn_sched_barrier(0);
			multiply(wr[s % S::kSets], c & 1, s);
		}
		stage_band(c + 1);
		__syncthreads();
	}
	if (tail)
	{
		const int c = full_chunks;
#pragma unroll
		for (int d = 0; d < kAhead; ++d) issue_w(wr[d], (int64_t)c * S::kWaveSteps + d, Guarded{});
#pragma unroll
		for (int s = 0; s < S::kWaveSteps; ++s)
		{
			const int64_t step = (int64_t)c * S::kWaveSteps + s;
			issue_w(wr[(s + kAhead) % S::kSets], step + kAhead, Guarded{});
			__builtin_amdgcn_sched_barrier(0);
			mask_w(wr[s % S::kSets], step);
			multiply(wr[s % S::kSets], c & 1, s);
		}
	}

	if constexpr (KW)
	{
		// waves 1 .. 3 hand their sums to wave 0, one after the other, through the band buffers
		float* pool = reinterpret_cast<float*>(&band_lds[0][0]);
		for (int giver = 1; giver < 4; ++giver)
		{
			__syncthreads();                     // the band (first round) or the previous round has been read
			if (wave == giver)
			{
#pragma unroll
				for (int w = 0; w < S::kMats; ++w)
#pragma unroll
					for (int e = 0; e < 4; ++e)
#pragma unroll
						for (int b = 0; b < MB; ++b)
#pragma unroll
							for (int r = 0; r < S::kRegs; ++r)
								pool[(((w * 4 + e) * MB + b) * S::kRegs + r) * kWaveSize + lane] = acc[w][e][b][r];
			}
			__syncthreads();
			if (wave == 0)
			{
#pragma unroll
				for (int w = 0; w < S::kMats; ++w)
#pragma unroll
					for (int e = 0; e < 4; ++e)
#pragma unroll
						for (int b = 0; b < MB; ++b)
#pragma unroll
							for (int r = 0; r < S::kRegs; ++r)
								acc[w][e][b][r] += pool[(((w * 4 + e) * MB + b) * S::kRegs + r) * kWaveSize + lane];
			}
		}
		if (wave != 0) return;
	}

	if (gridDim.y > 1)
	{
		// [matrix][row block][register][accumulator]: the four accumulators of a register are four consecutive columns
		float* mine = partial + ((wave_tile * gridDim.y + blockIdx.y) * kWaveSize + lane) * S::kAccFloats;
#pragma unroll
		for (int w = 0; w < S::kMats; ++w)
#pragma unroll
			for (int b = 0; b < MB; ++b)
#pragma unroll
				for (int r = 0; r < S::kRegs; ++r)
					*reinterpret_cast<float4_t*>(mine + ((w * MB + b) * S::kRegs + r) * 4) =
						float4_t{acc[w][0][b][r], acc[w][1][b][r], acc[w][2][b][r], acc[w][3][b][r]};
		return;
	}
	row_band_store<MR, MB, EPI>(acc, bias, C, M, N, ldc, n0, idx, grp, ep_param);
}

// Adds the partial sums of the `splits` K ranges in split order and finishes.  One thread per output vector of four
// columns (wave tile, lane, row block, register), so that the short, latency-bound job is spread over many waves;
// the loads of four splits are in flight together and added in order.
template <int MR, int MB, int EPI>
__global__ __launch_bounds__(kBandThreads) void gemm_band_ncontig_merge_kernel(
	const float* __restrict__ partial, const float* __restrict__ bias, float* __restrict__ C,
	int M, int64_t N, int64_t ldc, int splits, int64_t wave_tiles, float ep_param)
{
	using S = RowBandShape<MR, MB, EPI, false>;
	constexpr int kItems = MB * S::kRegs;                   // output vectors per lane
	const int64_t item = (int64_t)blockIdx.x * kBandThreads + threadIdx.x;
	const int q = (int)(item % kItems);
	const int lane = (int)((item / kItems) % kWaveSize);
	const int64_t wave_tile = item / (kItems * kWaveSize);
	if (wave_tile >= wave_tiles) return;
	const int b = q / S::kRegs, r = q % S::kRegs;
	const int m = b * MR + lane % MR;
	const int grp = lane / MR;
	const int slot = (MR == 16) ? 4 * grp + r : 8 * (r / 4) + 4 * grp + r % 4;
	int64_t n = wave_tile * S::kWaveCols + 4 * slot;
	if (m >= M || n >= N) return;
	if (n + 4 > N) n = N - 4;                     // as in row_band_store

	const int64_t stride = (int64_t)kWaveSize * S::kAccFloats;
	const float* src = partial + (wave_tile * splits * kWaveSize + lane) * S::kAccFloats + q * 4;
	float4_t sum[S::kMats];
#pragma unroll
	for (int w = 0; w < S::kMats; ++w) sum[w] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
	int sp = 0;
	for (; sp + 4 <= splits; sp += 4)
	{
		float4_t v[4][S::kMats];
#pragma unroll
		for (int i = 0; i < 4; ++i)
#pragma unroll
			for (int w = 0; w < S::kMats; ++w)
				v[i][w] = *reinterpret_cast<const float4_t*>(src + (sp + i) * stride + w * kItems * 4);
#pragma unroll
		for (int i = 0; i < 4; ++i)
#pragma unroll
			for (int w = 0; w < S::kMats; ++w) sum[w] += v[i][w];
	}
	for (; sp < splits; ++sp)
#pragma unroll
		for (int w = 0; w < S::kMats; ++w) sum[w] += *reinterpret_cast<const float4_t*>(src + sp * stride + w * kItems * 4);

	float4_t out;
#pragma unroll
	for (int e = 0; e < 4; ++e)
	{
		const float bias_n = (EPI == kEpiBias && bias) ? bias[n + e] : 0.0f;
		out[e] = finish_sum<EPI>(sum[0][e], sum[S::kMats - 1][e], bias_n, ep_param);
	}
	*reinterpret_cast<LooseVec*>(C + (int64_t)m * ldc + n) = out;
}

template <int MR, int MB, int EPI, bool KW, int SETS>
hipError_t launch_row_band_waves(const float* A, const float* B, const float* B2, const float* bias, float* C, int M, int64_t N,
                                 int64_t K, int64_t lda, int64_t ldb, int64_t ldc, float ep_param, hipStream_t stream)
{
	using S = RowBandShape<MR, MB, EPI, KW, SETS>;
	const int64_t tiles = (N + S::kBlockCols - 1) / S::kBlockCols;
	const int64_t wave_tiles = (N + S::kWaveCols - 1) / S::kWaveCols;
	// one wave's worth of sums per wave tile and split: a quarter of a 256-thread block's
	SplitPlan plan;
	const hipError_t plan_err = plan_band_splits(tiles, K, S::kChunk, S::kRows, (int)sizeof(float), S::kAccFloats / (KW ? 4 : 1), stream, &plan);
	if (plan_err != hipSuccess) return plan_err;
	discard_stale_error();
	gemm_band_ncontig_kernel<MR, MB, EPI, KW, SETS><<<dim3((unsigned)tiles, (unsigned)plan.splits), dim3(kBandThreads), 0, stream>>>(
		A, B, B2, bias, C, plan.partial, M, N, K, lda, ldb, ldc, (int)plan.chunks_per_split, ep_param);
	if (plan.splits > 1)
	{
		const int64_t items = wave_tiles * kWaveSize * MB * S::kRegs;
		gemm_band_ncontig_merge_kernel<MR, MB, EPI><<<dim3((unsigned)((items + kBandThreads - 1) / kBandThreads)), dim3(kBandThreads), 0, stream>>>(
			plan.partial, bias, C, M, N, ldc, (int)plan.splits, wave_tiles, ep_param);
	}
	return hipGetLastError();
}

template <int MR, int MB, int EPI>
hipError_t launch_row_band(const float* A, const float* B, const float* B2, const float* bias, float* C, int M, int64_t N, int64_t K,
                           int64_t lda, int64_t ldb, int64_t ldc, float ep_param, hipStream_t stream)
{
	// waves side by side when that alone gives the chip enough blocks, else the waves of a block divide K
	if ((N + 16 * MR - 1) / (16 * MR) >= kBandEnoughBlocks)
		return launch_row_band_waves<MR, MB, EPI, false, 4>(A, B, B2, bias, C, M, N, K, lda, ldb, ldc, ep_param, stream);
	// 32 rows of one product, waves dividing K: with two register sets for the weights instead of four (loads one step
	// ahead instead of three) three waves fit a SIMD instead of two, which hides more of the matrix cores' time than the
	// deeper queue does (32 x 4096 -> 6144: 37 -> 32 us, 4096 -> 11008: 48 -> 45.7); with 200 tiles and more, or a K of 16384 and
	// more, the deeper queue stays ahead (24 x 5120 -> 65536: 224 against 234, 32 x 36864 -> 4608: 123 against 139)
	if constexpr (MR == 32 && MB == 1 && EPI != kEpiGeluMul)
	{
		if ((N + 4 * MR - 1) / (4 * MR) < 200 && K < 16384)
			return launch_row_band_waves<MR, MB, EPI, true, 2>(A, B, B2, bias, C, M, N, K, lda, ldb, ldc, ep_param, stream);
	}
	return launch_row_band_waves<MR, MB, EPI, true, 4>(A, B, B2, bias, C, M, N, K, lda, ldb, ldc, ep_param, stream);
}

}  // namespace

bool gemm_band_ncontig_applies(const float* A, const float* B, const float* B2, const float* C, int64_t M, int64_t N, int64_t K,
                               int64_t lda, int64_t ldb, int64_t ldc, bool dual)
{
	if (M < 1 || M > kBandMaxRows || N < 4 || K < 1) return false;
	if (N / 64 > 0x7FFFFFFFLL) return false;
	if (M > 32 && (dual || (N < kBandEnoughBlocks * 512 && K < 4096))) return false;
	// 16-byte loads along K from A; the loads along N from B and the stores to C are 16 bytes at element alignment, and
	// with N no multiple of four the vector that would cross the end of a row is moved back to end with it
	(void)B;
	(void)B2;
	(void)C;
	(void)ldb;
	(void)ldc;
	return K % 4 == 0 && lda % 4 == 0 && aligned16(A);
}

hipError_t launch_gemm_band_ncontig(const float* A, const float* B, const float* B2, const float* bias, float* C,
                                    int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                    int epilogue, float ep_param, hipStream_t stream)
{
#define ANYGPU_ROW_BAND(MR, MB, EPI) \
	return launch_row_band<MR, MB, EPI>(A, B, B2, bias, C, (int)M, N, K, lda, ldb, ldc, ep_param, stream)
	if (epilogue == kEpiGeluMul)
	{
		if (M <= 16) ANYGPU_ROW_BAND(16, 1, kEpiGeluMul);
		ANYGPU_ROW_BAND(32, 1, kEpiGeluMul);
	}
	if (epilogue == kEpiSoftcap)
	{
		if (M <= 16) ANYGPU_ROW_BAND(16, 1, kEpiSoftcap);
		if (M <= 32) ANYGPU_ROW_BAND(32, 1, kEpiSoftcap);
		ANYGPU_ROW_BAND(32, 2, kEpiSoftcap);
	}
	if (M <= 16) ANYGPU_ROW_BAND(16, 1, kEpiBias);
	if (M <= 32) ANYGPU_ROW_BAND(32, 1, kEpiBias);
	ANYGPU_ROW_BAND(32, 2, kEpiBias);
#undef ANYGPU_ROW_BAND
}

}  // namespace anygpu
