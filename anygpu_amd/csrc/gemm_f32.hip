// fp32 GEMM (+ optional bias) for gfx950 on the fp32 MFMA path (v_mfma_f32_32x32x2_f32: every
// lane supplies one A and one B value per instruction, lanes 0-31 the even and lanes 32-63
// the odd k of a 2-deep step).  True fp32 products and sums; no reduced-precision tricks.
//
// Block tile 128 x 128 x 16, 4 waves, each wave a 64 x 64 patch (2 x 2 MFMA tiles).  An
// operand slab is staged in LDS in the orientation it has in memory: "k-contiguous" operands
// (row-major A, column-major B) as [row][16 k] rows, "row-contiguous" operands (column-major
// A, row-major B) as [16 k][row] rows.  Inside a slab the lower lane half consumes k = 0..7
// and the upper half k = 8..15, one per instruction, so a lane reads its 8 values of a
// k-contiguous operand with two 16-byte LDS loads and of a row-contiguous operand with eight
// conflict-free 4-byte loads.
// The same kernel serves any shape: FULL = true assumes whole tiles and 16-byte aligned
// rows (vector global loads), FULL = false guards every global access.
#include "device_utils.hpp"
#include "launch.hpp"
#include "anygpu_hip.h"

namespace anygpu {

constexpr int kBM = 128, kBN = 128, kBK = 16;
constexpr int kPitchK = kBK + 4;     // floats per [row][k] LDS row: 80 bytes, keeps 16-byte alignment
constexpr int kPitchR = 128 + 4;     // floats per [k][row] LDS row

// One 128-row x 16-deep operand slab.  KCONTIG: element (row, k) at base[row * ld + k];
// otherwise at base[k * ld + row].  `rows` / `depth` are the valid extents from the slab origin.
template <bool KCONTIG, bool FULL>
struct Slab
{
	static constexpr int kLdsFloats = KCONTIG ? 128 * kPitchK : kBK * kPitchR;

	// global -> registers: 512 float4 per slab, 2 per thread
	__device__ static void load(float4_t (&reg)[2], const float* __restrict__ base, int64_t ld,
	                            int64_t rows, int64_t depth, int tid)
	{
#pragma unroll
		for (int i = 0; i < 2; ++i)
		{
			const int q = tid + 256 * i;
			const int r = KCONTIG ? (q >> 2) : (q & 31) * 4;       // first row covered
			const int k = KCONTIG ? (q & 3) * 4 : (q >> 5);        // first k covered
			if (FULL)
			{
				reg[i] = *reinterpret_cast<const float4_t*>(KCONTIG ? base + r * ld + k : base + k * ld + r);
			}
			else
			{
#pragma unroll
				for (int e = 0; e < 4; ++e)
				{
					const int rr = KCONTIG ? r : r + e;
					const int kk = KCONTIG ? k + e : k;
					reg[i][e] = (rr < rows && kk < depth) ? (KCONTIG ? base[rr * ld + kk] : base[kk * ld + rr]) : 0.0f;
				}
			}
		}
	}

	__device__ static void store(float* lds, const float4_t (&reg)[2], int tid)
	{
#pragma unroll
		for (int i = 0; i < 2; ++i)
		{
			const int q = tid + 256 * i;
			if (KCONTIG)
				*reinterpret_cast<float4_t*>(&lds[(q >> 2) * kPitchK + (q & 3) * 4]) = reg[i];
			else
				*reinterpret_cast<float4_t*>(&lds[(q >> 5) * kPitchR + (q & 31) * 4]) = reg[i];
		}
	}

	// the 8 values row `row` contributes for k = kb .. kb + 7
	__device__ static void fragment(float (&v)[8], const float* lds, int row, int kb)
	{
		if (KCONTIG)
		{
			const float* src = &lds[row * kPitchK + kb];
			const float4_t lo = *reinterpret_cast<const float4_t*>(src);
			const float4_t hi = *reinterpret_cast<const float4_t*>(src + 4);
#pragma unroll
			for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[4 + e] = hi[e]; }
		}
		else
		{
#pragma unroll
			for (int e = 0; e < 8; ++e) v[e] = lds[(kb + e) * kPitchR + row];
		}
	}
};

template <int A_LAYOUT, int B_LAYOUT, bool FULL>
__global__ __launch_bounds__(256) void gemm_f32_kernel(
	const float* __restrict__ A, const float* __restrict__ B, const float* __restrict__ bias, float* __restrict__ C,
	int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
	int64_t stride_a, int64_t stride_b, int64_t stride_c)
{
	A += (int64_t)blockIdx.z * stride_a;
	B += (int64_t)blockIdx.z * stride_b;
	C += (int64_t)blockIdx.z * stride_c;
	using SlabA = Slab<A_LAYOUT == ANYGPU_A_ROW_MAJOR, FULL>;
	using SlabB = Slab<B_LAYOUT == ANYGPU_B_COL_MAJOR, FULL>;
	__shared__ __align__(16) float a_lds[2][SlabA::kLdsFloats];
	__shared__ __align__(16) float b_lds[2][SlabB::kLdsFloats];

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = tid >> 6;
	const int wm = wave >> 1, wn = wave & 1;
	const int64_t m0 = (int64_t)blockIdx.y * kBM;
	const int64_t n0 = (int64_t)blockIdx.x * kBN;

	const float* a_base = (A_LAYOUT == ANYGPU_A_ROW_MAJOR) ? A + m0 * lda : A + m0;
	const float* b_base = (B_LAYOUT == ANYGPU_B_COL_MAJOR) ? B + n0 * ldb : B + n0;
	auto a_at = [&](int64_t k0) { return (A_LAYOUT == ANYGPU_A_ROW_MAJOR) ? a_base + k0 : a_base + k0 * lda; };
	auto b_at = [&](int64_t k0) { return (B_LAYOUT == ANYGPU_B_COL_MAJOR) ? b_base + k0 : b_base + k0 * ldb; };

	float4_t ra[2], rb[2];

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
		SlabA::load(ra, a_at(0), lda, M - m0, K, tid);
		SlabB::load(rb, b_at(0), ldb, N - n0, K, tid);
		SlabA::store(a_lds[0], ra, tid);
		SlabB::store(b_lds[0], rb, tid);
	}
	__syncthreads();

	for (int64_t kt = 0; kt < ktiles; ++kt)
	{
		const int buf = (int)(kt & 1);
		if (kt + 1 < ktiles)
		{
			const int64_t k1 = (kt + 1) * kBK;
			SlabA::load(ra, a_at(k1), lda, M - m0, K - k1, tid);
			SlabB::load(rb, b_at(k1), ldb, N - n0, K - k1, tid);
		}

		float av[2][8], bv[2][8];
#pragma unroll
		for (int i = 0; i < 2; ++i) SlabA::fragment(av[i], a_lds[buf], wm * 64 + i * 32 + frag_row, kb);
#pragma unroll
		for (int j = 0; j < 2; ++j) SlabB::fragment(bv[j], b_lds[buf], wn * 64 + j * 32 + frag_row, kb);
#pragma unroll
		for (int e = 0; e < 8; ++e)
#pragma unroll
			for (int i = 0; i < 2; ++i)
#pragma unroll
				for (int j = 0; j < 2; ++j)
					acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[j][e], av[i][e], acc[i][j], 0, 0, 0);

		if (kt + 1 < ktiles)
		{
			SlabA::store(a_lds[buf ^ 1], ra, tid);
			SlabB::store(b_lds[buf ^ 1], rb, tid);
		}
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

template <int A_LAYOUT, int B_LAYOUT>
static hipError_t launch_layout(const float* A, const float* B, const float* bias, float* C,
                                int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                                hipStream_t stream)
{
	const dim3 grid((unsigned)((N + kBN - 1) / kBN), (unsigned)((M + kBM - 1) / kBM), (unsigned)batch);
	const bool aligned = (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(B) % 16 == 0) &&
	                     (reinterpret_cast<uintptr_t>(C) % 16 == 0) && (lda % 4 == 0) && (ldb % 4 == 0) && (ldc % 4 == 0) &&
	                     (stride_a % 4 == 0) && (stride_b % 4 == 0) && (stride_c % 4 == 0);
	const bool full = aligned && (M % kBM == 0) && (N % kBN == 0) && (K % kBK == 0);
	discard_stale_error();
	if (full)
		gemm_f32_kernel<A_LAYOUT, B_LAYOUT, true><<<grid, dim3(256), 0, stream>>>(A, B, bias, C, M, N, K, lda, ldb, ldc,
		                                                                            stride_a, stride_b, stride_c);
	else
		gemm_f32_kernel<A_LAYOUT, B_LAYOUT, false><<<grid, dim3(256), 0, stream>>>(A, B, bias, C, M, N, K, lda, ldb, ldc,
		                                                                            stride_a, stride_b, stride_c);
	return hipGetLastError();
}

hipError_t launch_gemm_f32(const float* A, const float* B, const float* bias, float* C,
                           int64_t M, int64_t N, int64_t K,
                           int64_t lda, int64_t ldb, int64_t ldc,
                           int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                           int a_layout, int b_layout, hipStream_t stream)
{
	if (M == 0 || N == 0 || batch == 0) return hipSuccess;
	if (a_layout == ANYGPU_A_ROW_MAJOR)
	{
		if (b_layout == ANYGPU_B_COL_MAJOR)
			return launch_layout<ANYGPU_A_ROW_MAJOR, ANYGPU_B_COL_MAJOR>(A, B, bias, C, M, N, K, lda, ldb, ldc,
		                                                             stride_a, stride_b, stride_c, batch, stream);
		return launch_layout<ANYGPU_A_ROW_MAJOR, ANYGPU_B_ROW_MAJOR>(A, B, bias, C, M, N, K, lda, ldb, ldc,
		                                                             stride_a, stride_b, stride_c, batch, stream);
	}
	if (b_layout == ANYGPU_B_COL_MAJOR)
		return launch_layout<ANYGPU_A_COL_MAJOR, ANYGPU_B_COL_MAJOR>(A, B, bias, C, M, N, K, lda, ldb, ldc,
		                                                             stride_a, stride_b, stride_c, batch, stream);
	return launch_layout<ANYGPU_A_COL_MAJOR, ANYGPU_B_ROW_MAJOR>(A, B, bias, C, M, N, K, lda, ldb, ldc,
		                                                             stride_a, stride_b, stride_c, batch, stream);
}

}  // namespace anygpu
