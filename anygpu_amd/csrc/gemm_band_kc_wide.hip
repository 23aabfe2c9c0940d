// Bands of few left-operand rows (M <= 64) against k-contiguous weights (B stored [N, K], "weights as [out, in]": the
// layout of the Gemma2 output head, srcs/models/gemma2/gemma_linsoftcap.cu:11-33) with the many columns of an output
// head, fp32 and fp16: the weight matrix is streamed once, in whole 128-byte lines per row and load instruction.
//
// The MFMA operand of the weights wants lane (c = lane % 16, g = lane / 16) to hold 16 bytes of weight row c.  Loaded
// that way, an instruction reads 64 bytes of each of 16 rows: half lines.  Here a lane (i = lane % 8, h = lane / 8)
// loads chunk h (16 bytes) of the 128-byte segment of row i, and again of row i + 8: whole lines of eight rows per
// instruction.  h = 2 g + (bit 3 of the lane), so a lane and its partner lane ^ 8 hold, of the two rows c = lane % 16
// stands for in the two of them, the even and the odd chunk of their k group: each sends the partner the vector it
// needs (one DPP row rotation by 8) and keeps the other, after which every lane holds chunks 2 g and 2 g + 1 of row c.
// The k index inside an MFMA is a dummy index, so the k slot of lane group g simply stands for that chunk's k (the band
// operand is read from LDS with the same mapping: 32 consecutive bytes of band row m per lane).
// fp16: a chunk is the 8 k of one v_mfma_f32_16x16x32_f16 operand, two MFMAs per 128-byte step; fp32: element e of a
// chunk feeds its own v_mfma_f32_16x16x4_f32, eight per step.
//
// A wave covers 64 columns (four MFMA column tiles), the four waves of a block sit side by side; no cut along K: the
// kernel is for weight matrices whose columns alone fill the chip, everything else stays with the other band kernels
// and the tile kernels.
#include "gemm_band.hpp"
#include "anygpu_hip.h"

#include <type_traits>

namespace anygpu {

using namespace band;

namespace {

constexpr int kWideStepBytes = 128;                // bytes of a weight row (and of a band row) per step
constexpr int kWideStepsPerChunk = 2;              // steps per LDS chunk of the band (64 rows x 2 buffers: 35 KB)
constexpr int kWideChunkBytes = kWideStepBytes * kWideStepsPerChunk;
constexpr int kWidePitchBytes = kWideChunkBytes + 16;   // band rows 272 bytes apart in LDS: no bank conflicts
constexpr int kWideTiles = 4;                      // MFMA column tiles of 16 per wave
constexpr int kWideWaveCols = 16 * kWideTiles;
constexpr int kWideBlockCols = 4 * kWideWaveCols;
constexpr int kWideSets = 2;                       // weight register sets: loads run a step ahead (three sets: 3 % slower,
                                                   // the registers cost a wave per SIMD)

typedef int int4v __attribute__((ext_vector_type(4)));

// the vector of lane ^ 8 (a rotation by 8 inside each row of 16 lanes)
__device__ __forceinline__ int4v from_partner(const int4v& v)
{
	int4v r;
#pragma unroll
	for (int d = 0; d < 4; ++d) r[d] = __builtin_amdgcn_update_dpp(0, v[d], 0x128 /* row_ror:8 */, 0xF, 0xF, true);
	return r;
}

// MB: row blocks of 16 (M <= 16 MB).  EPI: kEpiBias (+ bias[n] when bias != NULL) or kEpiSoftcap.
// PARTIAL: blockIdx.y walks ranges of k_split elements of K (whole LDS chunks) and the raw fp32 sums of range y go to
// plane y ([M, N] floats) of `partial`; the merge kernel below adds the planes and applies the epilogue.
template <typename T, int MB, int EPI, bool PARTIAL>
__global__ __launch_bounds__(kBandThreads) void gemm_band_kc_wide_kernel(
	const T* __restrict__ A, const T* __restrict__ B, const T* __restrict__ bias, T* __restrict__ C,
	int M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, float ep_param,
	float* __restrict__ partial, int64_t k_split)
{
	if constexpr (PARTIAL)
	{
		const int64_t k_begin = (int64_t)blockIdx.y * k_split;
		A += k_begin;
		B += k_begin;
		K = K - k_begin < k_split ? K - k_begin : k_split;
	}
	constexpr int EPC = 16 / (int)sizeof(T);                       // elements per 16-byte chunk
	constexpr int kStep = kWideStepBytes / (int)sizeof(T);         // k per step
	constexpr int kChunk = kStep * kWideStepsPerChunk;             // k per LDS chunk of the band
	constexpr int kRows = 16 * MB;
	constexpr int kVecsPerRow = kWideChunkBytes / 16;
	constexpr int kVecsPerThread = kRows * kVecsPerRow / kBandThreads;
	static_assert(kRows * kVecsPerRow % kBandThreads == 0, "whole vectors per thread");
	__shared__ __align__(16) char band_lds[2][kRows * kWidePitchBytes];

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = tid >> 6;
	const int col = lane & 15;                       // MFMA side: weight row (output column) slot, band row
	const int grp = lane >> 4;                       //            k group
	const int row8 = lane & 7;                       // load side: weight row inside a half tile
	const int chunk = lane >> 3;                     //            16-byte chunk of the step's 128 bytes
	const bool upper = (lane & 8) != 0;
	const int64_t n0 = ((int64_t)blockIdx.x * 4 + wave) * kWideWaveCols;
	const bool active = n0 < N;                      // (a wave past the last column still stages the band)

	// weight rows of this lane: rows past the end are replaced by the last one (never stored)
	const T* wrow[kWideTiles][2];
#pragma unroll
	for (int t = 0; t < kWideTiles; ++t)
#pragma unroll
		for (int h = 0; h < 2; ++h)
		{
			int64_t n = n0 + 16 * t + 8 * h + row8;
			if (n >= N) n = N - 1;
			wrow[t][h] = B + n * ldb + chunk * EPC;
		}

	const int64_t steps = K / kStep;
	Vec wr[kWideSets][kWideTiles][2];
	auto issue_w = [&](Vec (&dst)[kWideTiles][2], int64_t step) {
#pragma unroll
		for (int t = 0; t < kWideTiles; ++t)
#pragma unroll
			for (int h = 0; h < 2; ++h) dst[t][h] = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(wrow[t][h] + step * kStep));
	};

	// the band chunk: kRows rows x 16 vectors; rows past M and k past K come from valid addresses and are zeroed
	Vec ar[kVecsPerThread];
	const Vec zero = {0.0f, 0.0f, 0.0f, 0.0f};
	auto issue_band = [&](int64_t c) {
		const int64_t kc = c * kChunk;
#pragma unroll
		for (int i = 0; i < kVecsPerThread; ++i)
		{
			const int q = tid + kBandThreads * i;
			const int row = q / kVecsPerRow;
			const int64_t k = kc + (q % kVecsPerRow) * EPC;
			ar[i] = *reinterpret_cast<const Vec*>(A + (int64_t)(row < M ? row : M - 1) * lda + (k < K ? k : 0));
		}
	};
	auto stage_band = [&](int64_t slot, int64_t c) {
		const int64_t kc = c * kChunk;
#pragma unroll
		for (int i = 0; i < kVecsPerThread; ++i)
		{
			const int q = tid + kBandThreads * i;
			const int row = q / kVecsPerRow;
			const bool valid = row < M && kc + (q % kVecsPerRow) * EPC < K;
			*reinterpret_cast<Vec*>(&band_lds[slot & 1][row * kWidePitchBytes + (q % kVecsPerRow) * 16]) = valid ? ar[i] : zero;
		}
	};

	float4_t acc[kWideTiles][MB];
#pragma unroll
	for (int t = 0; t < kWideTiles; ++t)
#pragma unroll
		for (int b = 0; b < MB; ++b) acc[t][b] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

	auto multiply = [&](const Vec (&v)[kWideTiles][2], int buf, int s) {
		// chunks 2 g and 2 g + 1 of band row m: 32 consecutive bytes
		Vec a_even[MB], a_odd[MB];
#pragma unroll
		for (int b = 0; b < MB; ++b)
		{
			const char* src = &band_lds[buf][(16 * b + col) * kWidePitchBytes + s * kWideStepBytes + 32 * grp];
			a_even[b] = *reinterpret_cast<const Vec*>(src);
			a_odd[b] = *reinterpret_cast<const Vec*>(src + 16);
		}
#pragma unroll
		for (int t = 0; t < kWideTiles; ++t)
		{
			const int4v x0 = __builtin_bit_cast(int4v, v[t][0]), x1 = __builtin_bit_cast(int4v, v[t][1]);
			const int4v got = from_partner(upper ? x0 : x1);
			const Vec w_even = __builtin_bit_cast(Vec, upper ? got : x0);
			const Vec w_odd = __builtin_bit_cast(Vec, upper ? x1 : got);
#pragma unroll
			for (int b = 0; b < MB; ++b)
			{
				if constexpr (sizeof(T) == 2)
				{
					acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, w_even), __builtin_bit_cast(half8_t, a_even[b]), acc[t][b], 0, 0, 0);
					acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, w_odd), __builtin_bit_cast(half8_t, a_odd[b]), acc[t][b], 0, 0, 0);
				}
				else
				{
#pragma unroll
					for (int e = 0; e < 4; ++e) acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(w_even[e], a_even[b][e], acc[t][b], 0, 0, 0);
#pragma unroll
					for (int e = 0; e < 4; ++e) acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(w_odd[e], a_odd[b][e], acc[t][b], 0, 0, 0);
				}
			}
		}
	};

	const int64_t chunks = (K + kChunk - 1) / kChunk;
	constexpr int kAhead = kWideSets - 1;
	// Blocks start at different chunks of K and wrap around: blocks that run side by side then read different parts of
	// their weight rows at any one time (with rows a power of two apart, equal offsets in all rows are addresses that
	// share their low bits, and with them the memory channel).  Whole chunks only: with a half chunk at the end of K the
	// order stays 0, 1, 2, ...
	const int64_t first = steps % kWideStepsPerChunk == 0 ? (int64_t)(((blockIdx.x + 977u * blockIdx.y) * 2654435761u) >> 8) % chunks : 0;
	auto chunk_at = [&](int64_t i) { const int64_t c = i + first; return c >= chunks ? c - chunks : c; };   // i <= chunks
	auto step_at = [&](int64_t i) { const int64_t t = i + first * kWideStepsPerChunk; return t >= steps ? t - steps : t; };
	issue_band(chunk_at(0));
	if (active)
	{
#pragma unroll
		for (int d = 0; d < kAhead; ++d) issue_w(wr[d], step_at(d < steps ? d : steps - 1));
	}
	stage_band(0, chunk_at(0));
	__syncthreads();
	// (the register set of a step has to be a compile-time constant: six steps, three chunks, per trip)
	for (int64_t c0 = 0; c0 < chunks; c0 += kWideSets)
	{
#pragma unroll
		for (int cc = 0; cc < kWideSets; ++cc)
		{
			const int64_t c = c0 + cc;
			if (c < chunks)                                    // block-uniform
			{
				issue_band(chunk_at(c + 1));                   // after the last chunk: staged into a buffer nobody reads
#pragma unroll
				for (int s = 0; s < kWideStepsPerChunk; ++s)
				{
					const int64_t step = c * kWideStepsPerChunk + s;
					const int set = (cc * kWideStepsPerChunk + s) % kWideSets;
					if (active && step < steps)
					{
						const int64_t next = step + kAhead;
						issue_w(wr[(set + kAhead) % kWideSets], step_at(next < steps ? next : steps - 1));
						__builtin_amdgcn_sched_barrier(0);
						multiply(wr[set], (int)(c & 1), s);
					}
				}
				stage_band(c + 1, chunk_at(c + 1));
				__syncthreads();
			}
		}
	}
	if (!active) return;

	// lane (band row slot, k group g) holds, of row block b and column tile t, the columns 16 t + 4 g + r
	typedef T OutVec __attribute__((ext_vector_type(4)));
#pragma unroll
	for (int b = 0; b < MB; ++b)
	{
		const int m = 16 * b + col;
		if (m >= M) continue;
#pragma unroll
		for (int t = 0; t < kWideTiles; ++t)
		{
			const int64_t n = n0 + 16 * t + 4 * grp;
			if (n + 4 > N) continue;
			if constexpr (PARTIAL)
			{
				*reinterpret_cast<float4_t*>(partial + ((int64_t)blockIdx.y * M + m) * N + n) = acc[t][b];
				continue;
			}
			OutVec out;
#pragma unroll
			for (int r = 0; r < 4; ++r)
			{
				const float bias_n = (EPI == kEpiBias && bias) ? (float)bias[n + r] : 0.0f;
				out[r] = (T)finish_sum<EPI, sizeof(T) == 2>(acc[t][b][r], 0.0f, bias_n, ep_param);
			}
			*reinterpret_cast<OutVec*>(C + (int64_t)m * ldc + n) = out;
		}
	}
}

// C[m, n .. n + 3] = finish(sum over the planes, in order), one thread per four columns
template <typename T, int EPI>
__global__ __launch_bounds__(256) void gemm_band_kc_wide_merge_kernel(
	const float* __restrict__ partial, const T* __restrict__ bias, T* __restrict__ C, int M, int64_t N, int64_t ldc,
	int splits, float ep_param)
{
	const int64_t per_row = N / 4;
	const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (item >= (int64_t)M * per_row) return;
	const int64_t m = item / per_row, n = (item % per_row) * 4;
	const float* src = partial + m * N + n;
	const int64_t plane = (int64_t)M * N;
	float4_t sum = {0.0f, 0.0f, 0.0f, 0.0f};
	int sp = 0;
	for (; sp + 4 <= splits; sp += 4)
	{
		float4_t v[4];
#pragma unroll
		for (int i = 0; i < 4; ++i) v[i] = *reinterpret_cast<const float4_t*>(src + (sp + i) * plane);
#pragma unroll
		for (int i = 0; i < 4; ++i) sum += v[i];
	}
	for (; sp < splits; ++sp) sum += *reinterpret_cast<const float4_t*>(src + sp * plane);
	typedef T OutVec __attribute__((ext_vector_type(4)));
	OutVec out;
#pragma unroll
	for (int r = 0; r < 4; ++r)
	{
		const float bias_n = (EPI == kEpiBias && bias) ? (float)bias[n + r] : 0.0f;
		out[r] = (T)finish_sum<EPI, sizeof(T) == 2>(sum[r], 0.0f, bias_n, ep_param);
	}
	*reinterpret_cast<OutVec*>(C + m * ldc + n) = out;
}

// How a product whose columns alone do not fill the chip is cut along K: ranges of whole LDS chunks, as few as give
// every CU (nearly) two blocks with no more than 15 % of the CUs idle in the last round, every range at least
// kWideMinChunks chunks deep (16 x 3584 -> 18944 fp32 in ten ranges of six chunks: 58 us, the other band kernel 51),
// the planes within `room` bytes.  0: no such cut.  17 - 32 rows (where the matrix cores' time comes close to the
// memory's in fp32 and the other band kernel is as fast on most shapes) only in three ranges or more.
constexpr int64_t kWideMinChunks = 12;
template <typename T>
int64_t wide_split_chunks(int64_t M, int64_t N, int64_t K, size_t room)
{
	constexpr int kChunk = kWideChunkBytes / (int)sizeof(T);
	const int64_t chunks = (K + kChunk - 1) / kChunk;
	const int64_t blocks = (N + kWideBlockCols - 1) / kWideBlockCols;
	const int64_t cus = device_cu_count();
	for (int64_t s = 2; s <= 16; ++s)
	{
		const int64_t per = (chunks + s - 1) / s;
		if (per < kWideMinChunks) break;
		const int64_t ranges = (chunks + per - 1) / per;
		if ((size_t)ranges * (size_t)M * (size_t)N * sizeof(float) > room) break;
		const int64_t total = blocks * ranges, rounds = (total + cus - 1) / cus;
		if (total * 20 < cus * 38 || total * 100 < rounds * cus * 85) continue;
		if (M > 16 && M <= 32 && ranges < 3) return 0;
		return per;
	}
	return 0;
}

template <typename T, int MB>
hipError_t launch_rows(const T* A, const T* B, const T* bias, T* C, int M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                       int64_t ldc, int epilogue, float ep_param, hipStream_t stream, int64_t split_chunks)
{
	const unsigned blocks = (unsigned)((N + kWideBlockCols - 1) / kWideBlockCols);
	discard_stale_error();
	if (split_chunks > 0)
	{
		constexpr int kChunk = kWideChunkBytes / (int)sizeof(T);
		const int64_t k_split = split_chunks * kChunk;
		const int ranges = (int)((K + k_split - 1) / k_split);
		float* partial = nullptr;
		const hipError_t err = workspace_acquire(stream, &partial);
		if (err != hipSuccess) return err;
		gemm_band_kc_wide_kernel<T, MB, kEpiBias, true><<<dim3(blocks, (unsigned)ranges), dim3(kBandThreads), 0, stream>>>(
			A, B, nullptr, C, M, N, K, lda, ldb, ldc, 0.0f, partial, k_split);
		const dim3 grid((unsigned)(((int64_t)M * (N / 4) + 255) / 256));
		if (epilogue == kEpiSoftcap)
			gemm_band_kc_wide_merge_kernel<T, kEpiSoftcap><<<grid, dim3(256), 0, stream>>>(partial, bias, C, M, N, ldc, ranges, ep_param);
		else
			gemm_band_kc_wide_merge_kernel<T, kEpiBias><<<grid, dim3(256), 0, stream>>>(partial, bias, C, M, N, ldc, ranges, ep_param);
		return hipGetLastError();
	}
	if (epilogue == kEpiSoftcap)
		gemm_band_kc_wide_kernel<T, MB, kEpiSoftcap, false><<<dim3(blocks), dim3(kBandThreads), 0, stream>>>(A, B, bias, C, M, N, K, lda, ldb, ldc, ep_param, nullptr, 0);
	else
		gemm_band_kc_wide_kernel<T, MB, kEpiBias, false><<<dim3(blocks), dim3(kBandThreads), 0, stream>>>(A, B, bias, C, M, N, K, lda, ldb, ldc, ep_param, nullptr, 0);
	return hipGetLastError();
}

// what both forms assume of the operands
template <typename T>
bool wide_operands_ok(const T* A, const T* B, const T* C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t max_rows)
{
	constexpr int EPC = 16 / (int)sizeof(T);
	constexpr int kStep = kWideStepBytes / (int)sizeof(T);
	if (M < 1 || M > max_rows || M > 64 || K < kStep || K % kStep != 0 || N % 4 != 0) return false;
	if ((N + kWideBlockCols - 1) / kWideBlockCols > 0x7FFFFFFFLL) return false;
	return lda % EPC == 0 && ldb % EPC == 0 && ldc % 4 == 0 && aligned16(A) && aligned16(B) &&
	       reinterpret_cast<uintptr_t>(C) % (4 * sizeof(T)) == 0;
}

}  // namespace

// Whole 128-byte steps of K, rows of the operands at 16-byte boundaries, four output columns per store, and a block
// count that suits a kernel without a cut along K: (nearly) two blocks of 256 columns per CU or more (eight waves a CU
// keep enough loads in flight; 128256 columns on 256 CUs are 1.96), and no more than 15 % of the CUs idle while the
// others work on their last block (98304 columns are 1.5 blocks per CU: half the CUs would run two, half one).
template <typename T>
bool gemm_band_kc_wide_applies(const T* A, const T* B, const T* C, int64_t M, int64_t N, int64_t K,
                               int64_t lda, int64_t ldb, int64_t ldc, int64_t max_rows)
{
	if (!wide_operands_ok(A, B, C, M, N, K, lda, ldb, ldc, max_rows)) return false;
	const int64_t blocks = (N + kWideBlockCols - 1) / kWideBlockCols;
	const int64_t cus = device_cu_count();
	const int64_t rounds = (blocks + cus - 1) / cus;
	return cus > 0 && blocks * 20 >= cus * 38 && blocks * 100 >= rounds * cus * 85;
}

// The same with fewer columns, where a cut along K brings the block count there (see wide_split_chunks)
template <typename T>
bool gemm_band_kc_wide_split_applies(const T* A, const T* B, const T* C, int64_t M, int64_t N, int64_t K,
                                     int64_t lda, int64_t ldb, int64_t ldc, int64_t max_rows, hipStream_t stream)
{
	if (!wide_operands_ok(A, B, C, M, N, K, lda, ldb, ldc, max_rows)) return false;
	if (gemm_band_kc_wide_applies(A, B, C, M, N, K, lda, ldb, ldc, max_rows)) return false;
	return wide_split_chunks<T>(M, N, K, workspace_capacity(stream)) > 0;
}

template <typename T>
hipError_t launch_gemm_band_kc_wide(const T* A, const T* B, const T* bias, T* C, int64_t M, int64_t N, int64_t K,
                                    int64_t lda, int64_t ldb, int64_t ldc, int epilogue, float ep_param, hipStream_t stream)
{
	const int64_t split_chunks = gemm_band_kc_wide_applies(A, B, C, M, N, K, lda, ldb, ldc, 64) ? 0 : wide_split_chunks<T>(M, N, K, workspace_capacity(stream));
	if (M <= 16) return launch_rows<T, 1>(A, B, bias, C, (int)M, N, K, lda, ldb, ldc, epilogue, ep_param, stream, split_chunks);
	if (M <= 32) return launch_rows<T, 2>(A, B, bias, C, (int)M, N, K, lda, ldb, ldc, epilogue, ep_param, stream, split_chunks);
	if (M <= 48) return launch_rows<T, 3>(A, B, bias, C, (int)M, N, K, lda, ldb, ldc, epilogue, ep_param, stream, split_chunks);
	return launch_rows<T, 4>(A, B, bias, C, (int)M, N, K, lda, ldb, ldc, epilogue, ep_param, stream, split_chunks);
}

template bool gemm_band_kc_wide_applies<float>(const float*, const float*, const float*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t);
template bool gemm_band_kc_wide_applies<half_t>(const half_t*, const half_t*, const half_t*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t);
template bool gemm_band_kc_wide_split_applies<float>(const float*, const float*, const float*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, hipStream_t);
template bool gemm_band_kc_wide_split_applies<half_t>(const half_t*, const half_t*, const half_t*, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, hipStream_t);
template hipError_t launch_gemm_band_kc_wide<float>(const float*, const float*, const float*, float*, int64_t, int64_t, int64_t,
                                                    int64_t, int64_t, int64_t, int, float, hipStream_t);
template hipError_t launch_gemm_band_kc_wide<half_t>(const half_t*, const half_t*, const half_t*, half_t*, int64_t, int64_t, int64_t,
                                                     int64_t, int64_t, int64_t, int, float, hipStream_t);

}  // namespace anygpu
