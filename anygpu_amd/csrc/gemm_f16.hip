// fp16 x fp16 -> fp32-accumulate -> fp16 GEMM for gfx950 on the MFMA units
// (v_mfma_f32_32x32x16_f16: 32x32 output tile, 16-deep, 8 halves per lane per operand).
//
// Tile kernel ("NT": A [M,K] and B [N,K], both K-contiguous): a block owns a BM x BN tile of C,
// stages BM x BK and BN x BK slabs of A and B in LDS, double-buffered, and each wave
// accumulates a (BM/WM) x (BN/WN) sub-tile in registers.  LDS rows are BK halves (128 bytes)
// long; the 16-byte chunk index is XOR-swizzled with the row so that the 8 lanes that read
// the same logical chunk of 8 consecutive rows hit 8 different bank groups.
// The products are formed transposed (operand "A" of the instruction is the B slab), which
// leaves every lane with 4 consecutive columns of one row of C: 8-byte stores.
//
// Edge kernel: 64 x 64 tiles, guarded scalar loads and stores, either B layout, any
// shape, stride and alignment.
#include "device_utils.hpp"
#include "launch.hpp"
#include "anygpu_hip.h"

namespace anygpu {

// ---------------------------------------------------------------------------------------------
// Tile -> block mapping.  Workgroups are dealt round-robin to the 8 XCDs (each with its own
// L2), so block b runs on XCD b % 8.  Blocks of one XCD are given a contiguous range of tile
// numbers, and tile numbers walk the tile grid in column-strips of GROUP_M rows, so an XCD
// works on a compact patch of C and re-uses A and B slabs out of its own L2.
// ---------------------------------------------------------------------------------------------
constexpr int kNumXcd = 8;
constexpr int kGroupM = 4;

__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn)
{
	const int total = tiles_m * tiles_n;
	int id = bid;
	if (total % kNumXcd == 0)
	{
		id = (bid % kNumXcd) * (total / kNumXcd) + bid / kNumXcd;
	}
	const int per_group = kGroupM * tiles_n;
	const int g = id / per_group;
	const int first_m = g * kGroupM;
	const int rows = min(kGroupM, tiles_m - first_m);
	const int in_group = id - g * per_group;
	tm = first_m + in_group % rows;
	tn = in_group / rows;
}

template <int BM, int BN, int BK, int WM, int WN>
struct TileCfg
{
	static constexpr int kThreads = WM * WN * kWaveSize;
	static constexpr int kWaveM = BM / WM;
	static constexpr int kWaveN = BN / WN;
	static constexpr int kTilesM = kWaveM / 32;
	static constexpr int kTilesN = kWaveN / 32;
	static constexpr int kChunks = BK / 8;                   // 16-byte chunks per LDS row
	static constexpr int kVecA = BM * kChunks / kThreads;    // 16-byte global loads per thread per slab
	static constexpr int kVecB = BN * kChunks / kThreads;
	static constexpr int kSlabBytes = (BM + BN) * BK * 2;
	static constexpr int kLdsBytes = 2 * kSlabBytes;
	static_assert(BK == 64, "the swizzle below assumes 8 chunks per row");
	static_assert(BM * kChunks % kThreads == 0 && BN * kChunks % kThreads == 0, "slab must divide over the block");
};

__device__ __forceinline__ int swizzled_offset(int row, int chunk)
{
	return row * 128 + ((chunk ^ (row & 7)) << 4);
}

template <int BM, int BN, int BK, int WM, int WN>
__global__ __launch_bounds__(WM * WN * kWaveSize) void gemm_f16_nt_tile_kernel(
	const half_t* __restrict__ A, const half_t* __restrict__ B, half_t* __restrict__ C,
	int K, int64_t lda, int64_t ldb, int64_t ldc, int tiles_m, int tiles_n)
{
	using Cfg = TileCfg<BM, BN, BK, WM, WN>;
	extern __shared__ __align__(16) char lds[];

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = tid >> 6;
	const int wm = wave / WN;
	const int wn = wave % WN;

	int tile_m, tile_n;
	tile_of_block(blockIdx.x, tiles_m, tiles_n, tile_m, tile_n);
	const int64_t m0 = (int64_t)tile_m * BM;
	const int64_t n0 = (int64_t)tile_n * BN;

	// global -> register staging: vector q = tid + kThreads * i covers (row q / 8, chunk q % 8)
	const int ld_row = tid / Cfg::kChunks;
	const int ld_chunk = tid % Cfg::kChunks;
	constexpr int kRowStep = Cfg::kThreads / Cfg::kChunks;
	const half_t* a_src = A + (m0 + ld_row) * lda + ld_chunk * 8;
	const half_t* b_src = B + (n0 + ld_row) * ldb + ld_chunk * 8;

	half8_t ra[Cfg::kVecA], rb[Cfg::kVecB];

	auto load_slab = [&](int kt) {
		const int64_t koff = (int64_t)kt * BK;
#pragma unroll
		for (int i = 0; i < Cfg::kVecA; ++i)
			ra[i] = *reinterpret_cast<const half8_t*>(a_src + (int64_t)i * kRowStep * lda + koff);
#pragma unroll
		for (int i = 0; i < Cfg::kVecB; ++i)
			rb[i] = *reinterpret_cast<const half8_t*>(b_src + (int64_t)i * kRowStep * ldb + koff);
	};
	auto store_slab = [&](int buf) {
		char* a_lds = lds + buf * Cfg::kSlabBytes;
		char* b_lds = a_lds + BM * BK * 2;
#pragma unroll
		for (int i = 0; i < Cfg::kVecA; ++i)
			*reinterpret_cast<half8_t*>(a_lds + swizzled_offset(ld_row + i * kRowStep, ld_chunk)) = ra[i];
#pragma unroll
		for (int i = 0; i < Cfg::kVecB; ++i)
			*reinterpret_cast<half8_t*>(b_lds + swizzled_offset(ld_row + i * kRowStep, ld_chunk)) = rb[i];
	};

	float16_t acc[Cfg::kTilesM][Cfg::kTilesN];
#pragma unroll
	for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
		for (int j = 0; j < Cfg::kTilesN; ++j)
#pragma unroll
			for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

	const int frag_row = lane & 31;
	const int frag_half = lane >> 5;
	const int ktiles = K / BK;

	load_slab(0);
	store_slab(0);
	__syncthreads();

	for (int kt = 0; kt < ktiles; ++kt)
	{
		const int buf = kt & 1;
		if (kt + 1 < ktiles) load_slab(kt + 1);

		const char* a_lds = lds + buf * Cfg::kSlabBytes;
		const char* b_lds = a_lds + BM * BK * 2;
#pragma unroll
		for (int kk = 0; kk < BK / 16; ++kk)
		{
			const int chunk = kk * 2 + frag_half;
			half8_t af[Cfg::kTilesM], bf[Cfg::kTilesN];
#pragma unroll
			for (int i = 0; i < Cfg::kTilesM; ++i)
				af[i] = *reinterpret_cast<const half8_t*>(
					a_lds + swizzled_offset(wm * Cfg::kWaveM + i * 32 + frag_row, chunk));
#pragma unroll
			for (int j = 0; j < Cfg::kTilesN; ++j)
				bf[j] = *reinterpret_cast<const half8_t*>(
					b_lds + swizzled_offset(wn * Cfg::kWaveN + j * 32 + frag_row, chunk));
#pragma unroll
			for (int i = 0; i < Cfg::kTilesM; ++i)
#pragma unroll
				for (int j = 0; j < Cfg::kTilesN; ++j)
					acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
		}

		if (kt + 1 < ktiles) store_slab(buf ^ 1);
		__syncthreads();
	}

	// Epilogue.  With the B slab as the first operand, register r of lane l holds
	// C[m = l % 32][n = 8 * (r / 4) + 4 * (l / 32) + r % 4] of the 32 x 32 tile.
#pragma unroll
	for (int i = 0; i < Cfg::kTilesM; ++i)
	{
		const int64_t m = m0 + wm * Cfg::kWaveM + i * 32 + frag_row;
#pragma unroll
		for (int j = 0; j < Cfg::kTilesN; ++j)
		{
			const int64_t nb = n0 + wn * Cfg::kWaveN + j * 32 + 4 * frag_half;
#pragma unroll
			for (int g = 0; g < 4; ++g)
			{
				half4_t out;
#pragma unroll
				for (int e = 0; e < 4; ++e) out[e] = (half_t)acc[i][j][4 * g + e];
				*reinterpret_cast<half4_t*>(C + m * ldc + nb + 8 * g) = out;
			}
		}
	}
}

// ---------------------------------------------------------------------------------------------
// Edge kernel: 64 x 64 tile, 4 waves, one 32 x 32 MFMA tile per wave, 16-deep steps.
// Every global access is guarded and scalar; K tails are zero-filled in LDS.
// ---------------------------------------------------------------------------------------------
template <int B_LAYOUT>
__global__ __launch_bounds__(256) void gemm_f16_edge_kernel(
	const half_t* __restrict__ A, const half_t* __restrict__ B, half_t* __restrict__ C,
	int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc)
{
	__shared__ half_t a_lds[64][16 + 8];
	__shared__ half_t b_lds[64][16 + 8];

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = tid >> 6;
	const int64_t m0 = (int64_t)blockIdx.y * 64;
	const int64_t n0 = (int64_t)blockIdx.x * 64;
	const int wm = wave >> 1, wn = wave & 1;

	float16_t acc;
#pragma unroll
	for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

	for (int64_t k0 = 0; k0 < K; k0 += 16)
	{
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			const int q = tid + 256 * i;      // 0..1023
			{
				const int r = q / 16, c = q % 16;
				const int64_t m = m0 + r, k = k0 + c;
				a_lds[r][c] = (m < M && k < K) ? A[m * lda + k] : (half_t)0.0f;
			}
			if (B_LAYOUT == ANYGPU_B_COL_MAJOR)
			{
				const int r = q / 16, c = q % 16;
				const int64_t n = n0 + r, k = k0 + c;
				b_lds[r][c] = (n < N && k < K) ? B[n * ldb + k] : (half_t)0.0f;
			}
			else
			{
				const int c = q / 64, r = q % 64;  // consecutive threads walk n
				const int64_t n = n0 + r, k = k0 + c;
				b_lds[r][c] = (n < N && k < K) ? B[k * ldb + n] : (half_t)0.0f;
			}
		}
		__syncthreads();

		half8_t af, bf;
		const int kb = (lane >> 5) * 8;
#pragma unroll
		for (int e = 0; e < 8; ++e)
		{
			af[e] = a_lds[wm * 32 + (lane & 31)][kb + e];
			bf[e] = b_lds[wn * 32 + (lane & 31)][kb + e];
		}
		acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf, af, acc, 0, 0, 0);
		__syncthreads();
	}

	const int64_t m = m0 + wm * 32 + (lane & 31);
	if (m < M)
	{
#pragma unroll
		for (int r = 0; r < 16; ++r)
		{
			const int64_t n = n0 + wn * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
			if (n < N) C[m * ldc + n] = (half_t)acc[r];
		}
	}
}

template <int BM, int BN, int BK, int WM, int WN>
static hipError_t launch_tile(const half_t* A, const half_t* B, half_t* C, int64_t M, int64_t N, int64_t K,
                              int64_t lda, int64_t ldb, int64_t ldc, hipStream_t stream)
{
	using Cfg = TileCfg<BM, BN, BK, WM, WN>;
	auto kernel = gemm_f16_nt_tile_kernel<BM, BN, BK, WM, WN>;
	static bool configured = false;
	discard_stale_error();
	if (!configured)
	{
		hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
		                                   hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::kLdsBytes);
		if (e != hipSuccess) return e;
		configured = true;
	}
	const int tiles_m = (int)(M / BM), tiles_n = (int)(N / BN);
	kernel<<<dim3((unsigned)(tiles_m * tiles_n)), dim3(Cfg::kThreads), Cfg::kLdsBytes, stream>>>(
		A, B, C, (int)K, lda, ldb, ldc, tiles_m, tiles_n);
	return hipGetLastError();
}

hipError_t launch_gemm_f16(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                           int64_t lda, int64_t ldb, int64_t ldc, int b_layout, hipStream_t stream)
{
	if (M == 0 || N == 0) return hipSuccess;
	const half_t* a = static_cast<const half_t*>(A);
	const half_t* b = static_cast<const half_t*>(B);
	half_t* c = static_cast<half_t*>(C);

	const bool aligned = (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(B) % 16 == 0) &&
	                     (reinterpret_cast<uintptr_t>(C) % 8 == 0) && (lda % 8 == 0) && (ldb % 8 == 0) && (ldc % 4 == 0);
	if (b_layout == ANYGPU_B_COL_MAJOR && aligned && K > 0 && K % 64 == 0 && M % 256 == 0 && N % 256 == 0 &&
	    (M / 256) * (N / 256) <= 0x7FFFFFFFLL)
	{
		return launch_tile<256, 256, 64, 2, 4>(a, b, c, M, N, K, lda, ldb, ldc, stream);
	}

	const dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64));
	discard_stale_error();
	if (b_layout == ANYGPU_B_COL_MAJOR)
		gemm_f16_edge_kernel<ANYGPU_B_COL_MAJOR><<<grid, dim3(256), 0, stream>>>(a, b, c, M, N, K, lda, ldb, ldc);
	else
		gemm_f16_edge_kernel<ANYGPU_B_ROW_MAJOR><<<grid, dim3(256), 0, stream>>>(a, b, c, M, N, K, lda, ldb, ldc);
	return hipGetLastError();
}

}  // namespace anygpu
