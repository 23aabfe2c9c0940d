// Bands of few left-operand rows (M <= 64) against n-contiguous fp16 weights (row-major B, [K, N]: the layout of the
// reference's own linear layers, srcs/ops/mm_ops.hpp:205-232) with very many columns: the weight matrix is streamed
// once, straight from memory into MFMA operand registers, in whole 256-byte pieces of its rows.
//
// v_mfma_f32_16x16x32_f16 wants, per lane, eight consecutive k of ONE column; a 16-byte vector of an n-contiguous row
// holds ONE k of eight consecutive columns.  A lane (column slot i = lane % 16, k group g = lane / 16) therefore loads
// eight vectors, rows k0 + 8 g + j (j = 0 .. 7) of columns n0 + 8 i .. + 7: an 8 x 8 block of halves, which it transposes
// in its own registers (v_perm_b32 picks the low or the high halves of two dwords: four per operand).  Column e of the
// block is the operand of MFMA e with its own accumulator, so the column index is permuted between lanes and
// accumulators (MFMA e covers columns n0 + 8 s + e, s = 0 .. 15), which costs nothing: with the weights as the first
// operand a lane ends up with the slots 4 g + r of one band row, and its eight accumulators of a slot are eight
// consecutive columns, one 16-byte store.  A load instruction of a wave reads 256 contiguous bytes of each of four rows.
// The band of A rows sits in LDS (chunks of 128 k, two buffers) and is the second operand of every MFMA of a step.
//
// A wave covers 128 columns.  With very many columns the four waves of a block sit side by side (512 columns per block);
// with fewer all four take the same 128 columns and every fourth 32-deep step of K each and add their sums up through
// LDS at the end, which gives four times the blocks.  No cut along K over blocks: the kernel is for weight matrices whose
// columns give every CU work (output heads: 32000 to 256000 columns), everything else stays with the tile kernels.
#include "gemm_band.hpp"
#include "anygpu_hip.h"

namespace anygpu {

using namespace band;

namespace {

constexpr int kKnChunk = 128;                      // k per LDS chunk of the band
constexpr int kKnStep = 32;                        // k per MFMA step
constexpr int kKnPitch = kKnChunk + 8;             // halves per band row in LDS: rows 272 bytes apart, no bank conflicts
constexpr int kKnWaveCols = 128;
constexpr int kKnBlockCols = 4 * kKnWaveCols;
constexpr int kKnSets = 2;                         // weight register sets: loads run a step ahead (two steps: no faster)

// MB: row blocks of 16 (M <= 16 MB).  EPI: kEpiBias (nothing added: the fp16 bias form goes elsewhere) or kEpiSoftcap.
// KW: the waves of a block share their columns and divide K.
template <int MB, int EPI, bool KW>
__global__ __launch_bounds__(kBandThreads) void gemm_band_kn_f16_kernel(
	const half_t* __restrict__ A, const half_t* __restrict__ B, half_t* __restrict__ C,
	int M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, float ep_param)
{
	constexpr int kRows = 16 * MB;
	constexpr int kVecsPerThread = kRows * (kKnChunk / 8) / kBandThreads;       // band vectors a thread stages per chunk
	static_assert(kRows * (kKnChunk / 8) % kBandThreads == 0, "whole vectors per thread");
	__shared__ __align__(16) half_t band_lds[2][kRows * kKnPitch];

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = tid >> 6;
	const int slot = lane & 15;
	const int grp = lane >> 4;
	const int64_t n0 = (KW ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * 4 + wave) * kKnWaveCols;
	const bool active = n0 < N;                                // (a wave past the last column still stages the band)
	// this lane's eight columns; a vector past the end of a row is moved back to the last eight columns (never stored)
	int64_t n_lane = n0 + 8 * slot;
	if (n_lane + 8 > N) n_lane = N - 8;
	const half_t* __restrict__ wcol = B + n_lane;

	const int64_t steps = K / kKnStep;
	Vec wr[kKnSets][8];
	auto issue_w = [&](Vec (&dst)[8], int64_t step) {
		const int64_t k0 = step * kKnStep + 8 * grp;
#pragma unroll
		for (int j = 0; j < 8; ++j) dst[j] = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(wcol + (k0 + j) * ldb));
	};

	// the band chunk: kRows rows x 16 vectors; rows past M and k past K come from valid addresses and are zeroed
	Vec ar[kVecsPerThread];
	const Vec zero = {0.0f, 0.0f, 0.0f, 0.0f};
	auto issue_band = [&](int64_t chunk) {
		const int64_t kc = chunk * kKnChunk;
#pragma unroll
		for (int i = 0; i < kVecsPerThread; ++i)
		{
			const int q = tid + kBandThreads * i;
			const int row = q / (kKnChunk / 8);
			const int64_t k = kc + (q % (kKnChunk / 8)) * 8;
			ar[i] = *reinterpret_cast<const Vec*>(A + (int64_t)(row < M ? row : M - 1) * lda + (k < K ? k : 0));
		}
	};
	auto stage_band = [&](int64_t chunk) {
		const int64_t kc = chunk * kKnChunk;
#pragma unroll
		for (int i = 0; i < kVecsPerThread; ++i)
		{
			const int q = tid + kBandThreads * i;
			const int row = q / (kKnChunk / 8);
			const bool valid = row < M && kc + (q % (kKnChunk / 8)) * 8 < K;
			*reinterpret_cast<Vec*>(&band_lds[chunk & 1][row * kKnPitch + (q % (kKnChunk / 8)) * 8]) = valid ? ar[i] : zero;
		}
	};

	float4_t acc[8][MB];
#pragma unroll
	for (int e = 0; e < 8; ++e)
#pragma unroll
		for (int b = 0; b < MB; ++b) acc[e][b] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

	auto multiply = [&](const Vec (&v)[8], int buf, int s) {
		half8_t a[MB];
#pragma unroll
		for (int b = 0; b < MB; ++b)
			a[b] = *reinterpret_cast<const half8_t*>(&band_lds[buf][(16 * b + slot) * kKnPitch + s * kKnStep + 8 * grp]);
		typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
		uint4v raw[8];
#pragma unroll
		for (int j = 0; j < 8; ++j) raw[j] = __builtin_bit_cast(uint4v, v[j]);
#pragma unroll
		for (int e = 0; e < 8; ++e)
		{
			// operand dword d = halves e of rows 2 d and 2 d + 1 of the block
			uint4v op;
#pragma unroll
			for (int d = 0; d < 4; ++d)
				op[d] = __builtin_amdgcn_perm(raw[2 * d + 1][e / 2], raw[2 * d][e / 2], (e & 1) ? 0x07060302u : 0x05040100u);
			const half8_t w = __builtin_bit_cast(half8_t, op);
#pragma unroll
			for (int b = 0; b < MB; ++b) acc[e][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, a[b], acc[e][b], 0, 0, 0);
		}
	};

	const int64_t chunks = (K + kKnChunk - 1) / kKnChunk;
	constexpr int kStepsPerChunk = kKnChunk / kKnStep;
	constexpr int kWaveSteps = KW ? 1 : kStepsPerChunk;    // steps of a chunk one wave takes: all, or step number `wave`
	constexpr int kAhead = kKnSets - 1;
	// step q of this wave's own sequence, as a step of K
	auto own_step = [&](int64_t q) { return KW ? q * kStepsPerChunk + wave : q; };
	issue_band(0);
	if (active)
	{
#pragma unroll
		for (int d = 0; d < kAhead; ++d) issue_w(wr[d], own_step(d) < steps ? own_step(d) : steps - 1);
	}
	stage_band(0);
	__syncthreads();
	// (the register set of a step has to be a compile-time constant: three chunks per trip)
	for (int64_t c0 = 0; c0 < chunks; c0 += kKnSets)
	{
#pragma unroll
		for (int cc = 0; cc < kKnSets; ++cc)
		{
			const int64_t c = c0 + cc;
			if (c < chunks)                                    // block-uniform
			{
				issue_band(c + 1);                             // past the end: zeros, staged into a buffer nobody reads
#pragma unroll
				for (int sl = 0; sl < kWaveSteps; ++sl)
				{
					const int s = KW ? wave : sl;              // step inside the chunk
					const int64_t q = c * kWaveSteps + sl;     // its number in this wave's sequence
					const int set = (cc * kWaveSteps + sl) % kKnSets;
					if (active && c * kStepsPerChunk + s < steps)
					{
						const int64_t next = own_step(q + kAhead);
						issue_w(wr[(set + kAhead) % kKnSets], next < steps ? next : steps - 1);
						__builtin_amdgcn_sched_barrier(0);
						multiply(wr[set], (int)(c & 1), s);
					}
				}
				stage_band(c + 1);
				__syncthreads();
			}
		}
	}
	if constexpr (KW)
	{
		// waves 1 .. 3 hand their sums to wave 0, one after the other, through the band buffers
		static_assert(sizeof(band_lds) >= kWaveSize * 32 * MB * sizeof(float), "the sums of a wave fit the band buffers");
		float* pool = reinterpret_cast<float*>(&band_lds[0][0]);
		for (int giver = 1; giver < 4; ++giver)
		{
			__syncthreads();                               // the band (first round) or the previous round has been read
			if (wave == giver)
			{
#pragma unroll
				for (int e = 0; e < 8; ++e)
#pragma unroll
					for (int b = 0; b < MB; ++b)
#pragma unroll
						for (int r = 0; r < 4; ++r) pool[((e * MB + b) * 4 + r) * kWaveSize + lane] = acc[e][b][r];
			}
			__syncthreads();
			if (wave == 0)
			{
#pragma unroll
				for (int e = 0; e < 8; ++e)
#pragma unroll
					for (int b = 0; b < MB; ++b)
#pragma unroll
						for (int r = 0; r < 4; ++r) acc[e][b][r] += pool[((e * MB + b) * 4 + r) * kWaveSize + lane];
			}
		}
		if (wave != 0) return;
	}
	if (!active) return;

	// lane (band row slot, k group g) holds, of row block b, the column slots 4 g + r; accumulator e is column 8 s + e
#pragma unroll
	for (int b = 0; b < MB; ++b)
	{
		const int m = 16 * b + slot;
		if (m >= M) continue;
#pragma unroll
		for (int r = 0; r < 4; ++r)
		{
			const int64_t n = n0 + 8 * (4 * grp + r);
			if (n + 8 > N) continue;
			half8_t out;
#pragma unroll
			for (int e = 0; e < 8; ++e) out[e] = (half_t)finish_sum<EPI, true>(acc[e][b][r], 0.0f, 0.0f, ep_param);
			*reinterpret_cast<half8_t*>(C + (int64_t)m * ldc + n) = out;
		}
	}
}

// Blocks of 512 columns from which the waves of a block sit side by side (measured against the tile kernels and the
// vendor library at 2304 and 4096 deep: 160 blocks win at every row count, 128 lose), and the columns from which the
// waves share their columns and divide K instead (up to 32 rows; at 64 rows the hand-over of the sums through LDS
// costs what the extra blocks bring, at 32000 columns the tile kernels are faster at every row count).
constexpr int64_t kKnWideBlocks = 160;
constexpr int64_t kKnSharedMinCols = 49152;
constexpr int64_t kKnSharedMaxRows = 32;

template <int MB>
hipError_t launch_rows(const half_t* A, const half_t* B, half_t* C, int M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                       int64_t ldc, int epilogue, float ep_param, hipStream_t stream)
{
	const bool wide = (N + kKnBlockCols - 1) / kKnBlockCols >= kKnWideBlocks;
	const int64_t cols = wide ? kKnBlockCols : kKnWaveCols;
	const dim3 grid((unsigned)((N + cols - 1) / cols));
	discard_stale_error();
#define ANYGPU_KN_LAUNCH(EPI, KW) \
	gemm_band_kn_f16_kernel<MB, EPI, KW><<<grid, dim3(kBandThreads), 0, stream>>>(A, B, C, M, N, K, lda, ldb, ldc, ep_param)
	if (epilogue == kEpiSoftcap)
	{
		if (wide) ANYGPU_KN_LAUNCH(kEpiSoftcap, false);
		else ANYGPU_KN_LAUNCH(kEpiSoftcap, true);
	}
	else
	{
		if (wide) ANYGPU_KN_LAUNCH(kEpiBias, false);
		else ANYGPU_KN_LAUNCH(kEpiBias, true);
	}
#undef ANYGPU_KN_LAUNCH
	return hipGetLastError();
}

}  // namespace

// The kernel streams the weights without a cut along K over blocks, so it is for matrices whose columns give the chip
// enough blocks.
bool gemm_band_kn_f16_applies(const void* A, const void* B, const void* C, int64_t M, int64_t N, int64_t K,
                              int64_t lda, int64_t ldb, int64_t ldc)
{
	if (M < 1 || M > 64 || K < kKnStep || K % kKnStep != 0 || N % 8 != 0) return false;
	const bool wide = (N + kKnBlockCols - 1) / kKnBlockCols >= kKnWideBlocks;
	if (!wide && (N < kKnSharedMinCols || M > kKnSharedMaxRows)) return false;
	if ((N + kKnWaveCols - 1) / kKnWaveCols > 0x7FFFFFFFLL) return false;
	return lda % 8 == 0 && ldb % 8 == 0 && ldc % 8 == 0 && aligned16(A) && aligned16(B) && aligned16(C);
}

hipError_t launch_gemm_band_kn_f16(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                                   int64_t lda, int64_t ldb, int64_t ldc, int epilogue, float ep_param, hipStream_t stream)
{
	const half_t* a = static_cast<const half_t*>(A);
	const half_t* b = static_cast<const half_t*>(B);
	half_t* c = static_cast<half_t*>(C);
	if (M <= 16) return launch_rows<1>(a, b, c, (int)M, N, K, lda, ldb, ldc, epilogue, ep_param, stream);
	if (M <= 32) return launch_rows<2>(a, b, c, (int)M, N, K, lda, ldb, ldc, epilogue, ep_param, stream);
	return launch_rows<4>(a, b, c, (int)M, N, K, lda, ldb, ldc, epilogue, ep_param, stream);
}

}  // namespace anygpu
