// fp32 GEMM (+ optional bias) for gfx950 on the fp32 MFMA path (v_mfma_f32_32x32x2_f32: every
// lane supplies one A and one B value per instruction, lanes 0-31 the even and lanes 32-63
// the odd k of a 2-deep step).  True fp32 products and sums; no reduced-precision tricks.
//
// Block tile 128 x 128 x 16, 4 waves, each wave a 64 x 64 patch (2 x 2 MFMA tiles).  A is
// staged in LDS as [m][16 k] rows, B as [16 k][n] rows for the row-major layout (lanes walk
// n) or as [n][16 k] rows for the column-major layout.  Inside a slab the lower lane half
// consumes k = 0..7 and the upper half k = 8..15, one per instruction, so a lane reads its 8
// A values with two 16-byte LDS loads.
// The same kernel serves any shape: FULL = true assumes whole tiles and 16-byte aligned
// rows (vector global loads), FULL = false guards every global access.
#include "device_utils.hpp"
#include "launch.hpp"
#include "anygpu_hip.h"

namespace anygpu {

constexpr int kBM = 128, kBN = 128, kBK = 16;
constexpr int kPitchK = kBK + 4;     // floats per [row][k] LDS row: 80 bytes, keeps 16-byte alignment
constexpr int kPitchN = kBN + 4;     // floats per [k][n] LDS row

template <int B_LAYOUT, bool FULL>
__global__ __launch_bounds__(256) void gemm_f32_kernel(
	const float* __restrict__ A, const float* __restrict__ B, const float* __restrict__ bias, float* __restrict__ C,
	int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc)
{
	__shared__ __align__(16) float a_lds[2][kBM * kPitchK];
	__shared__ __align__(16) float b_lds[2][(B_LAYOUT == ANYGPU_B_COL_MAJOR) ? kBN * kPitchK : kBK * kPitchN];

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = tid >> 6;
	const int wm = wave >> 1, wn = wave & 1;
	const int64_t m0 = (int64_t)blockIdx.y * kBM;
	const int64_t n0 = (int64_t)blockIdx.x * kBN;

	// staging registers: A slab 128 x 16 = 512 float4 -> 2 per thread; B slab likewise
	float4_t ra[2], rb[2];

	auto load_a = [&](int64_t k0) {
#pragma unroll
		for (int i = 0; i < 2; ++i)
		{
			const int q = tid + 256 * i;         // float4 index: row q / 4, k-quad q % 4
			const int r = q >> 2, c = (q & 3) * 4;
			const int64_t m = m0 + r;
			if (FULL)
			{
				ra[i] = *reinterpret_cast<const float4_t*>(A + m * lda + k0 + c);
			}
			else
			{
#pragma unroll
				for (int e = 0; e < 4; ++e)
					ra[i][e] = (m < M && k0 + c + e < K) ? A[m * lda + k0 + c + e] : 0.0f;
			}
		}
	};
	auto load_b = [&](int64_t k0) {
#pragma unroll
		for (int i = 0; i < 2; ++i)
		{
			const int q = tid + 256 * i;
			if (B_LAYOUT == ANYGPU_B_COL_MAJOR)
			{
				const int r = q >> 2, c = (q & 3) * 4;   // row = n, quad along k
				const int64_t n = n0 + r;
				if (FULL)
				{
					rb[i] = *reinterpret_cast<const float4_t*>(B + n * ldb + k0 + c);
				}
				else
				{
#pragma unroll
					for (int e = 0; e < 4; ++e)
						rb[i][e] = (n < N && k0 + c + e < K) ? B[n * ldb + k0 + c + e] : 0.0f;
				}
			}
			else
			{
				const int r = q >> 5, c = (q & 31) * 4;  // row = k, quad along n
				const int64_t k = k0 + r;
				if (FULL)
				{
					rb[i] = *reinterpret_cast<const float4_t*>(B + k * ldb + n0 + c);
				}
				else
				{
#pragma unroll
					for (int e = 0; e < 4; ++e)
						rb[i][e] = (k < K && n0 + c + e < N) ? B[k * ldb + n0 + c + e] : 0.0f;
				}
			}
		}
	};
	auto store_slab = [&](int buf) {
#pragma unroll
		for (int i = 0; i < 2; ++i)
		{
			const int q = tid + 256 * i;
			{
				const int r = q >> 2, c = (q & 3) * 4;
				*reinterpret_cast<float4_t*>(&a_lds[buf][r * kPitchK + c]) = ra[i];
			}
			if (B_LAYOUT == ANYGPU_B_COL_MAJOR)
			{
				const int r = q >> 2, c = (q & 3) * 4;
				*reinterpret_cast<float4_t*>(&b_lds[buf][r * kPitchK + c]) = rb[i];
			}
			else
			{
				const int r = q >> 5, c = (q & 31) * 4;
				*reinterpret_cast<float4_t*>(&b_lds[buf][r * kPitchN + c]) = rb[i];
			}
		}
	};

	float16_t acc[2][2];
#pragma unroll
	for (int i = 0; i < 2; ++i)
#pragma unroll
		for (int j = 0; j < 2; ++j)
#pragma unroll
			for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

	const int frag_row = lane & 31;
	const int kb = (lane >> 5) * 8;          // this lane half's k range inside the slab
	const int64_t ktiles = (K + kBK - 1) / kBK;

	if (ktiles > 0)
	{
		load_a(0);
		load_b(0);
		store_slab(0);
	}
	__syncthreads();

	for (int64_t kt = 0; kt < ktiles; ++kt)
	{
		const int buf = (int)(kt & 1);
		if (kt + 1 < ktiles)
		{
			load_a((kt + 1) * kBK);
			load_b((kt + 1) * kBK);
		}

		float av[2][8], bv[2][8];
#pragma unroll
		for (int i = 0; i < 2; ++i)
		{
			const float* src = &a_lds[buf][(wm * 64 + i * 32 + frag_row) * kPitchK + kb];
			const float4_t lo = *reinterpret_cast<const float4_t*>(src);
			const float4_t hi = *reinterpret_cast<const float4_t*>(src + 4);
#pragma unroll
			for (int e = 0; e < 4; ++e) { av[i][e] = lo[e]; av[i][4 + e] = hi[e]; }
		}
#pragma unroll
		for (int j = 0; j < 2; ++j)
		{
			const int n = wn * 64 + j * 32 + frag_row;
			if (B_LAYOUT == ANYGPU_B_COL_MAJOR)
			{
				const float* src = &b_lds[buf][n * kPitchK + kb];
				const float4_t lo = *reinterpret_cast<const float4_t*>(src);
				const float4_t hi = *reinterpret_cast<const float4_t*>(src + 4);
#pragma unroll
				for (int e = 0; e < 4; ++e) { bv[j][e] = lo[e]; bv[j][4 + e] = hi[e]; }
			}
			else
			{
#pragma unroll
				for (int e = 0; e < 8; ++e) bv[j][e] = b_lds[buf][(kb + e) * kPitchN + n];
			}
		}
#pragma unroll
		for (int e = 0; e < 8; ++e)
#pragma unroll
			for (int i = 0; i < 2; ++i)
#pragma unroll
				for (int j = 0; j < 2; ++j)
					acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[j][e], av[i][e], acc[i][j], 0, 0, 0);

		if (kt + 1 < ktiles) store_slab(buf ^ 1);
		__syncthreads();
	}

	// register r of lane l: C[m = l % 32][n = 8 * (r / 4) + 4 * (l / 32) + r % 4] of a 32 x 32 tile
#pragma unroll
	for (int i = 0; i < 2; ++i)
	{
		const int64_t m = m0 + wm * 64 + i * 32 + frag_row;
#pragma unroll
		for (int j = 0; j < 2; ++j)
		{
#pragma unroll
			for (int g = 0; g < 4; ++g)
			{
				const int64_t n = n0 + wn * 64 + j * 32 + 8 * g + 4 * (lane >> 5);
				if (FULL)
				{
					float4_t out;
#pragma unroll
					for (int e = 0; e < 4; ++e) out[e] = acc[i][j][4 * g + e] + (bias ? bias[n + e] : 0.0f);
					*reinterpret_cast<float4_t*>(C + m * ldc + n) = out;
				}
				else if (m < M)
				{
#pragma unroll
					for (int e = 0; e < 4; ++e)
						if (n + e < N) C[m * ldc + n + e] = acc[i][j][4 * g + e] + (bias ? bias[n + e] : 0.0f);
				}
			}
		}
	}
}

template <int B_LAYOUT>
static hipError_t launch_layout(const float* A, const float* B, const float* bias, float* C,
                                int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                hipStream_t stream)
{
	const dim3 grid((unsigned)((N + kBN - 1) / kBN), (unsigned)((M + kBM - 1) / kBM));
	const bool aligned = (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(B) % 16 == 0) &&
	                     (reinterpret_cast<uintptr_t>(C) % 16 == 0) && (lda % 4 == 0) && (ldb % 4 == 0) && (ldc % 4 == 0);
	const bool full = aligned && (M % kBM == 0) && (N % kBN == 0) && (K % kBK == 0);
	discard_stale_error();
	if (full)
		gemm_f32_kernel<B_LAYOUT, true><<<grid, dim3(256), 0, stream>>>(A, B, bias, C, M, N, K, lda, ldb, ldc);
	else
		gemm_f32_kernel<B_LAYOUT, false><<<grid, dim3(256), 0, stream>>>(A, B, bias, C, M, N, K, lda, ldb, ldc);
	return hipGetLastError();
}

hipError_t launch_gemm_f32(const float* A, const float* B, const float* bias, float* C,
                           int64_t M, int64_t N, int64_t K,
                           int64_t lda, int64_t ldb, int64_t ldc, int b_layout, hipStream_t stream)
{
	if (M == 0 || N == 0) return hipSuccess;
	if (b_layout == ANYGPU_B_COL_MAJOR)
		return launch_layout<ANYGPU_B_COL_MAJOR>(A, B, bias, C, M, N, K, lda, ldb, ldc, stream);
	return launch_layout<ANYGPU_B_ROW_MAJOR>(A, B, bias, C, M, N, K, lda, ldb, ldc, stream);
}

}  // namespace anygpu
