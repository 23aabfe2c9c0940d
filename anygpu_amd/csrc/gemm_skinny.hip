// Products with very few left-operand rows (M <= 8: the single-token decode step of a language
// model, where every linear layer is a matrix-vector product).  A 64 x 64 MFMA tile would be
// 1/64 .. 1/8 full and the launch would have N / 64 blocks; the job is to stream the weight matrix
// from HBM once, at full bandwidth, so these kernels are plain FMA loops built around the loads.
//
//   k-contiguous weights (column-major B, [N, K]): one wave per pair of output columns; the lanes
//   stride over K with 16-byte loads, the A rows come out of L1 / L2, a DPP all-reduce finishes.
//
//   n-contiguous weights (row-major B, [K, N]): a block of 16 waves owns 32 lanes' worth of
//   columns; each half wave takes every 32nd weight row (128 contiguous bytes per load, 16 loads
//   in flight per lane).  The A rows are staged in LDS chunk by chunk, transposed to [k][m], so
//   that a lane gets all M values of its row with one broadcast LDS read; the partial sums of
//   the 32 row slices meet in LDS.
//
// Sums are fp32 whatever the element type; the order of summation differs from a sequential
// loop and stays inside the tolerance of the tile kernels.
#include "device_utils.hpp"
#include "gemm_epilogue.hpp"
#include "launch.hpp"
#include "anygpu_hip.h"

namespace anygpu {

namespace {

template <typename T> struct Vec16;
template <> struct Vec16<float> { typedef float4_t type; static constexpr int kLen = 4; };
template <> struct Vec16<half_t> { typedef half8_t type; static constexpr int kLen = 8; };

template <typename T> struct Vec4B;
template <> struct Vec4B<float> { typedef float type; static constexpr int kLen = 1; };
template <> struct Vec4B<half_t> { typedef half2_t type; static constexpr int kLen = 2; };

__device__ __forceinline__ float elem(float v, int) { return v; }
__device__ __forceinline__ float elem(half2_t v, int i) { return (float)v[i]; }

// output columns per wave of the k-contiguous kernel: more columns amortise the A loads over more FMAs
constexpr int skinny_cols_per_wave(int mrows) { return mrows >= 8 ? 8 : mrows >= 4 ? 4 : 2; }

// acc + sum_e a[e] * b[e] over one 16-byte vector, fp32 sums
__device__ __forceinline__ float dot_acc(float4_t a, float4_t b, float acc)
{
#pragma unroll
	for (int e = 0; e < 4; ++e) acc = __builtin_fmaf(a[e], b[e], acc);
	return acc;
}

// half inputs: v_dot2_f32_f16 forms both fp16 x fp16 products exactly and adds them to the fp32 sum
__device__ __forceinline__ float dot_acc(half8_t a, half8_t b, float acc)
{
#pragma unroll
	for (int e = 0; e < 8; e += 2)
		acc = __builtin_amdgcn_fdot2(half2_t{a[e], a[e + 1]}, half2_t{b[e], b[e + 1]}, acc, false);
	return acc;
}

// C[m, n] = finish(sum_k A[m, k] * B[n, k])
template <typename T, int MROWS, int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_kcontig_kernel(
	const T* __restrict__ A, const T* __restrict__ B, const T* __restrict__ B2, const T* __restrict__ bias,
	T* __restrict__ C, int M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, float ep_param)
{
	typedef typename Vec16<T>::type vec_t;
	constexpr int VEC = Vec16<T>::kLen;
	constexpr int NC = skinny_cols_per_wave(MROWS) / (EPI == kEpiGeluMul ? 2 : 1);
	constexpr bool DUAL = (EPI == kEpiGeluMul);
	const int lane = threadIdx.x & (kWaveSize - 1);
	const int wave = threadIdx.x >> 6;
	const int64_t n0 = ((int64_t)blockIdx.x * 4 + wave) * NC;
	if (n0 >= N) return;                       // the whole wave leaves; the kernel has no barrier

	const T* b_row[NC];
	const T* a_row[MROWS];
#pragma unroll
	for (int c = 0; c < NC; ++c) b_row[c] = B + (n0 + c < N ? n0 + c : n0) * ldb;
#pragma unroll
	for (int m = 0; m < MROWS; ++m) a_row[m] = A + (int64_t)(m < M ? m : M - 1) * lda;
	const int64_t b2_shift = DUAL ? (B2 - B) : 0;

	float acc[NC][MROWS], acc2[DUAL ? NC : 1][DUAL ? MROWS : 1];
#pragma unroll
	for (int c = 0; c < NC; ++c)
#pragma unroll
		for (int m = 0; m < MROWS; ++m)
		{
			acc[c][m] = 0.0f;
			if constexpr (DUAL) acc2[c][m] = 0.0f;
		}

#pragma unroll 2
	for (int64_t k = (int64_t)lane * VEC; k < K; k += kWaveSize * VEC)
	{
		vec_t b[NC], b2[DUAL ? NC : 1];
#pragma unroll
		for (int c = 0; c < NC; ++c)
		{
			b[c] = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(b_row[c] + k));
			if constexpr (DUAL) b2[c] = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(b_row[c] + b2_shift + k));
		}
#pragma unroll
		for (int m = 0; m < MROWS; ++m)
		{
			const vec_t a = *reinterpret_cast<const vec_t*>(a_row[m] + k);
#pragma unroll
			for (int c = 0; c < NC; ++c)
			{
				acc[c][m] = dot_acc(a, b[c], acc[c][m]);
				if constexpr (DUAL) acc2[c][m] = dot_acc(a, b2[c], acc2[c][m]);
			}
		}
	}

#pragma unroll
	for (int c = 0; c < NC; ++c)
#pragma unroll
		for (int m = 0; m < MROWS; ++m)
		{
			const float sum = wave_allreduce(acc[c][m], SumOp());
			float sum2 = 0.0f;
			if constexpr (DUAL) sum2 = wave_allreduce(acc2[c][m], SumOp());
			const int64_t n = n0 + c;
			if (lane == 0 && m < M && n < N)
			{
				const float bias_n = (EPI == kEpiBias && bias) ? (float)bias[n] : 0.0f;
				C[(int64_t)m * ldc + n] = (T)finish_sum<EPI>(sum, sum2, bias_n, ep_param);
			}
		}
}

constexpr int kSkinnySlices = 32;          // row slices per block: 16 waves x 2 halves
constexpr int kSkinnyDepth = 16;           // weight loads in flight per lane

// C[m, n] = finish(sum_k A[m, k] * B[k, n])
template <typename T, int MROWS, int EPI>
__global__ __launch_bounds__(1024) void gemm_skinny_ncontig_kernel(
	const T* __restrict__ A, const T* __restrict__ B, const T* __restrict__ B2, const T* __restrict__ bias,
	T* __restrict__ C, int M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, float ep_param)
{
	typedef typename Vec4B<T>::type vec_t;
	typedef float xvec_t __attribute__((ext_vector_type(MROWS)));
	constexpr int VECN = Vec4B<T>::kLen;
	constexpr int COLS = 32 * VECN;            // columns per block
	constexpr bool DUAL = (EPI == kEpiGeluMul);
	constexpr int NSUM = DUAL ? 2 : 1;
	constexpr int KC = 8192 / MROWS;           // A rows per LDS chunk (32 KB of floats), a multiple of 512
	constexpr int kRedFloats = 16 * NSUM * MROWS * VECN * 32;
	// first the A chunk as [k][m]; afterwards the partial sums of the 16 waves as [wave][sum][m][v][column lane]
	__shared__ __align__(16) float lds[kRedFloats > 8192 ? kRedFloats : 8192];

	const int lane = threadIdx.x & (kWaveSize - 1);
	const int wave = threadIdx.x >> 6;
	const int col_lane = lane & 31;
	const int slice = wave * 2 + (lane >> 5);
	const int64_t col = (int64_t)blockIdx.x * COLS + col_lane * VECN;
	// a vector that would cross or lie past the end of a row is moved back to the last VECN columns (crossing: stored
	// there, with the same values as its neighbour's; past: never stored); loads are made at element alignment
	typedef vec_t loose_t __attribute__((aligned(sizeof(T))));
	const int64_t col_load = col + VECN <= N ? col : N - VECN;
	const T* b_col = B + col_load;
	const int64_t b2_shift = DUAL ? (B2 - B) : 0;

	float acc[NSUM][MROWS][VECN];
#pragma unroll
	for (int s = 0; s < NSUM; ++s)
#pragma unroll
		for (int m = 0; m < MROWS; ++m)
#pragma unroll
			for (int v = 0; v < VECN; ++v) acc[s][m][v] = 0.0f;

	for (int64_t k0 = 0; k0 < K; k0 += KC)
	{
		if (k0 > 0) __syncthreads();           // everybody is done with the previous chunk
		// stage A[0..M)[k0 .. k0 + KC) as floats, zero past M and past K
		for (int idx = threadIdx.x; idx < KC * MROWS; idx += 1024)
		{
			const int m = idx / KC, kk = idx % KC;           // consecutive threads walk along k
			const float x = (m < M && k0 + kk < K) ? (float)A[(int64_t)m * lda + k0 + kk] : 0.0f;
			lds[kk * MROWS + m] = x;
		}
		__syncthreads();

		const int64_t chunk_rows = K - k0 < KC ? K - k0 : KC;
		for (int64_t kk = slice; kk < chunk_rows; kk += kSkinnySlices * kSkinnyDepth)
		{
			vec_t w[kSkinnyDepth], w2[DUAL ? kSkinnyDepth : 1];
#pragma unroll
			for (int d = 0; d < kSkinnyDepth; ++d)
			{
				int64_t row = k0 + kk + d * kSkinnySlices;
				row = row < K ? row : K - 1;                 // the A values of such a row are zero
				w[d] = __builtin_nontemporal_load(reinterpret_cast<const loose_t*>(b_col + row * ldb));
				if constexpr (DUAL) w2[d] = __builtin_nontemporal_load(reinterpret_cast<const loose_t*>(b_col + b2_shift + row * ldb));
			}
#pragma unroll
			for (int d = 0; d < kSkinnyDepth; ++d)
			{
				// kk + d * 32 stays inside its 512-row group and KC is a multiple of 512: r < KC
				const int r = (int)kk + d * kSkinnySlices;
				const xvec_t x = *reinterpret_cast<const xvec_t*>(&lds[r * MROWS]);
#pragma unroll
				for (int m = 0; m < MROWS; ++m)
				{
					const float xm = x[m];
#pragma unroll
					for (int v = 0; v < VECN; ++v)
					{
						acc[0][m][v] = __builtin_fmaf(xm, elem(w[d], v), acc[0][m][v]);
						if constexpr (DUAL) acc[NSUM - 1][m][v] = __builtin_fmaf(xm, elem(w2[DUAL ? d : 0], v), acc[NSUM - 1][m][v]);
					}
				}
			}
		}
	}
	__syncthreads();                               // the A chunk gives way to the partial sums

	auto red = [&](int w, int s, int m, int v, int cl) -> float& { return lds[(((w * NSUM + s) * MROWS + m) * VECN + v) * 32 + cl]; };
#pragma unroll
	for (int s = 0; s < NSUM; ++s)
#pragma unroll
		for (int m = 0; m < MROWS; ++m)
#pragma unroll
			for (int v = 0; v < VECN; ++v)
			{
				const float other = __shfl_xor(acc[s][m][v], 32);      // the wave's other row slice, same columns
				if (lane < 32) red(wave, s, m, v, col_lane) = acc[s][m][v] + other;
			}
	__syncthreads();

	// one thread per (m, v, column lane) adds the 16 partial sums
	for (int idx = threadIdx.x; idx < MROWS * VECN * 32; idx += 1024)
	{
		const int cl = idx & 31;
		const int v = (idx >> 5) % VECN;
		const int m = idx / (32 * VECN);
		float sum = 0.0f, sum2 = 0.0f;
#pragma unroll
		for (int w = 0; w < 16; ++w)
		{
			sum += red(w, 0, m, v, cl);
			if constexpr (DUAL) sum2 += red(w, NSUM - 1, m, v, cl);
		}
		int64_t n_vec = (int64_t)blockIdx.x * COLS + cl * VECN;
		if (n_vec < N && n_vec + VECN > N) n_vec = N - VECN;        // as col_load of that lane
		const int64_t n = n_vec + v;
		if (m < M && n < N)
		{
			const float bias_n = (EPI == kEpiBias && bias) ? (float)bias[n] : 0.0f;
			C[(int64_t)m * ldc + n] = (T)finish_sum<EPI>(sum, sum2, bias_n, ep_param);
		}
	}
}

template <typename T, int MROWS, int EPI>
hipError_t launch_rows(const T* A, const T* B, const T* B2, const T* bias, T* C, int M, int64_t N, int64_t K,
                       int64_t lda, int64_t ldb, int64_t ldc, int b_layout, float ep_param, hipStream_t stream)
{
	discard_stale_error();
	if (b_layout == ANYGPU_B_COL_MAJOR)
	{
		constexpr int kColsPerBlock = 4 * skinny_cols_per_wave(MROWS) / (EPI == kEpiGeluMul ? 2 : 1);
		const int64_t blocks = (N + kColsPerBlock - 1) / kColsPerBlock;
		gemm_skinny_kcontig_kernel<T, MROWS, EPI><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
			A, B, B2, bias, C, M, N, K, lda, ldb, ldc, ep_param);
	}
	else
	{
		constexpr int COLS = 32 * Vec4B<T>::kLen;
		gemm_skinny_ncontig_kernel<T, MROWS, EPI><<<dim3((unsigned)((N + COLS - 1) / COLS)), dim3(1024), 0, stream>>>(
			A, B, B2, bias, C, M, N, K, lda, ldb, ldc, ep_param);
	}
	return hipGetLastError();
}

template <typename T>
bool aligned_to(const T* p, size_t bytes) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % bytes == 0; }

}  // namespace

template <typename T>
bool gemm_skinny_applies(const T* A, const T* B, const T* B2, int64_t M, int64_t N, int64_t K,
                         int64_t lda, int64_t ldb, int b_layout)
{
	if (M < 1 || M > kSkinnyMaxRows || N < 1 || K < 1) return false;
	if (b_layout == ANYGPU_B_COL_MAJOR)
	{
		// 16-byte loads along K from every row of A and B
		constexpr int VEC = Vec16<T>::kLen;
		if (N > (int64_t)0x7FFFFFFF * 4) return false;       // grid of at most N / 4 blocks
		return K % VEC == 0 && lda % VEC == 0 && ldb % VEC == 0 && aligned_to(A, 16) && aligned_to(B, 16) && aligned_to(B2, 16);
	}
	// 4-byte loads along N at element alignment
	constexpr int VECN = Vec4B<T>::kLen;
	return N >= VECN;
}

template <typename T>
hipError_t launch_gemm_skinny(const T* A, const T* B, const T* B2, const T* bias, T* C,
                              int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                              int b_layout, int epilogue, float ep_param, hipStream_t stream)
{
	const int rows = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : 8;
#define ANYGPU_SKINNY_ROWS(R) \
	switch (epilogue) \
	{ \
	case kEpiSoftcap: return launch_rows<T, R, kEpiSoftcap>(A, B, B2, bias, C, (int)M, N, K, lda, ldb, ldc, b_layout, ep_param, stream); \
	case kEpiGeluMul: return launch_rows<T, R, kEpiGeluMul>(A, B, B2, bias, C, (int)M, N, K, lda, ldb, ldc, b_layout, ep_param, stream); \
	default: return launch_rows<T, R, kEpiBias>(A, B, B2, bias, C, (int)M, N, K, lda, ldb, ldc, b_layout, ep_param, stream); \
	}
	switch (rows)
	{
	case 1: ANYGPU_SKINNY_ROWS(1)
	case 2: ANYGPU_SKINNY_ROWS(2)
	case 4: ANYGPU_SKINNY_ROWS(4)
	default: ANYGPU_SKINNY_ROWS(8)
	}
#undef ANYGPU_SKINNY_ROWS
}

template bool gemm_skinny_applies<float>(const float*, const float*, const float*, int64_t, int64_t, int64_t, int64_t, int64_t, int);
template bool gemm_skinny_applies<half_t>(const half_t*, const half_t*, const half_t*, int64_t, int64_t, int64_t, int64_t, int64_t, int);
template hipError_t launch_gemm_skinny<float>(const float*, const float*, const float*, const float*, float*, int64_t, int64_t, int64_t,
                                              int64_t, int64_t, int64_t, int, int, float, hipStream_t);
template hipError_t launch_gemm_skinny<half_t>(const half_t*, const half_t*, const half_t*, const half_t*, half_t*, int64_t, int64_t, int64_t,
                                               int64_t, int64_t, int64_t, int, int, float, hipStream_t);

}  // namespace anygpu
