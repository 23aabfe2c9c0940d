// fp32 GEMM (+ optional bias) for gfx950 on the fp32 MFMA path (v_mfma_f32_32x32x2_f32: every
// lane supplies one A and one B value per instruction, lanes 0-31 the even and lanes 32-63
// the odd k of a 2-deep step).  True fp32 products and sums; no reduced-precision tricks.
//
// Block tile 128 x 128 x 16 or 64 x 64 x 16, 4 waves in a 2 x 2 arrangement.  An
// operand slab is staged in LDS in the orientation it has in memory: "k-contiguous" operands
// (row-major A, column-major B) as [row][16 k] rows, "row-contiguous" operands (column-major
// A, row-major B) as [16 k][row] rows.  Inside a slab the lower lane half consumes k = 0..7
// and the upper half k = 8..15, one per instruction, so a lane reads its 8 values of a
// k-contiguous operand with two 16-byte LDS loads and of a row-contiguous operand with eight
// conflict-free 4-byte loads.
// The same kernel serves any shape through its access mode: whole tiles and 16-byte aligned rows
// (vector loads, no tests), aligned rows but ragged extents (vector loads from clamped rows, the
// last vectors of a row or column guarded, vector stores where they fit), or anything (the same
// with the vectors at element alignment).
#include "device_utils.hpp"
#include "gemm_epilogue.hpp"
#include "launch.hpp"
#include "gemm_band.hpp"
#include "gemm_f32_ring.hpp"
#include "anygpu_hip.h"

#include <type_traits>

namespace anygpu {

// how the kernel may touch global memory
constexpr int kAccessFull = 0;      // whole tiles, aligned: no tests
constexpr int kAccessAligned = 1;   // 16-byte aligned rows and leading dimensions, ragged M / N / K
constexpr int kAccessAny = 2;       // nothing assumed: vectors at element alignment, guarded ends
constexpr int kAccessPadded = 3;    // operands as in kAccessFull (aligned copies padded with zeros to whole tiles), C as in kAccessAny

constexpr int kBK = 16;
constexpr int kPitchK = kBK + 4;     // floats per [row][k] LDS row: 80 bytes, keeps 16-byte alignment

// Scheduling-group masks of __builtin_amdgcn_sched_group_barrier
constexpr int kSchedMfma = 0x008;
constexpr int kSchedVmemRead = 0x020;
constexpr int kSchedDsRead = 0x100;
constexpr int kSchedDsWrite = 0x200;

// One ROWS-row x 16-deep operand slab (ROWS = 64 or 128).  KCONTIG: element (row, k) at
// base[row * ld + k]; otherwise at base[k * ld + row].  `rows` / `depth` are the valid extents
// from the slab origin.
template <bool KCONTIG, int ACCESS, int ROWS>
struct Slab
{
	static constexpr bool FULL = (ACCESS == kAccessFull || ACCESS == kAccessPadded);
	static constexpr bool kKContig = KCONTIG;
	static constexpr int kPitchR = ROWS + 4;                 // floats per [k][row] LDS row
	static constexpr int kLdsFloats = KCONTIG ? ROWS * kPitchK : kBK * kPitchR;
	static constexpr int kVecs = ROWS * kBK / 4 / 256;       // float4 per thread per slab
	static constexpr int kQuadsPerK = ROWS / 4;              // float4 along a [k][row] row

	// global -> registers
	__device__ static void load(float4_t (&reg)[kVecs], const float* __restrict__ base, int64_t ld,
	                            int64_t rows, int64_t depth, int tid)
	{
#pragma unroll
		for (int i = 0; i < kVecs; ++i)
		{
			const int q = tid + 256 * i;
			const int r = KCONTIG ? (q >> 2) : (q % kQuadsPerK) * 4;       // first row covered
			const int k = KCONTIG ? (q & 3) * 4 : (q / kQuadsPerK);        // first k covered
			if (FULL)
			{
				reg[i] = *reinterpret_cast<const float4_t*>(KCONTIG ? base + r * ld + k : base + k * ld + r);
			}
			else if (KCONTIG ? (k + 4 <= depth) : (k < depth && r + 4 <= rows))
			{
				// the vector lies inside the operand along its own axis; across it, rows past the end are
				// replaced by the last row (they only feed results that are not stored).  Without the
				// alignment guarantee the same 16 bytes are fetched at element alignment.
				typedef float4_t LooseVec __attribute__((aligned(4)));
				const int64_t rc = KCONTIG ? (r < rows ? r : rows - 1) : r;
				const float* src = KCONTIG ? base + rc * ld + k : base + k * ld + r;
				if (ACCESS == kAccessAligned) reg[i] = *reinterpret_cast<const float4_t*>(src);
				else reg[i] = *reinterpret_cast<const LooseVec*>(src);
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

	__device__ static void store(float* lds, const float4_t (&reg)[kVecs], int tid)
	{
#pragma unroll
		for (int i = 0; i < kVecs; ++i)
		{
			const int q = tid + 256 * i;
			if (KCONTIG)
				*reinterpret_cast<float4_t*>(&lds[(q >> 2) * kPitchK + (q & 3) * 4]) = reg[i];
			else
				*reinterpret_cast<float4_t*>(&lds[(q / kQuadsPerK) * kPitchR + (q % kQuadsPerK) * 4]) = reg[i];
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

template <int A_LAYOUT, int B_LAYOUT, int ACCESS, int BM, int BN, int EPI>
__global__ __launch_bounds__(256) void gemm_f32_kernel(
	const float* __restrict__ A, const float* __restrict__ B, const float* __restrict__ B2,
	const float* __restrict__ bias, float* __restrict__ C,
	int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
	int64_t stride_a, int64_t stride_b, int64_t stride_c, float ep_param, int64_t k_split)
{
	constexpr bool DUAL = (EPI == kEpiGeluMul);
	constexpr bool FULL = (ACCESS == kAccessFull);                                  // no test anywhere
	constexpr bool FULL_IN = FULL || ACCESS == kAccessPadded;                       // none on the operand side
	if (k_split > 0)
	{
		// blockIdx.z counts ranges of K of one product instead of products: the strides step along K
		const int64_t left = K - (int64_t)blockIdx.z * k_split;
		K = left < k_split ? left : k_split;
	}
	A += (int64_t)blockIdx.z * stride_a;
	B += (int64_t)blockIdx.z * stride_b;
	C += (int64_t)blockIdx.z * stride_c;
	using SlabA = Slab<A_LAYOUT == ANYGPU_A_ROW_MAJOR, ACCESS, BM>;
	using SlabB = Slab<B_LAYOUT == ANYGPU_B_COL_MAJOR, ACCESS, BN>;
	constexpr int WTM = BM / 2, WTN = BN / 2;       // wave patch (2 x 2 waves)
	constexpr int TM = WTM / 32, TN = WTN / 32;     // MFMA tiles per wave
	__shared__ __align__(16) float a_lds[2][SlabA::kLdsFloats];
	__shared__ __align__(16) float b_lds[2][SlabB::kLdsFloats];
	__shared__ __align__(16) float b2_lds[DUAL ? 2 : 1][DUAL ? SlabB::kLdsFloats : 4];

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = tid >> 6;
	const int wm = wave >> 1, wn = wave & 1;
	const int64_t m0 = (int64_t)blockIdx.y * BM;
	const int64_t n0 = (int64_t)blockIdx.x * BN;

	const float* a_base = (A_LAYOUT == ANYGPU_A_ROW_MAJOR) ? A + m0 * lda : A + m0;
	const float* b_base = (B_LAYOUT == ANYGPU_B_COL_MAJOR) ? B + n0 * ldb : B + n0;
	auto a_at = [&](int64_t k0) { return (A_LAYOUT == ANYGPU_A_ROW_MAJOR) ? a_base + k0 : a_base + k0 * lda; };
	auto b_at = [&](int64_t k0) { return (B_LAYOUT == ANYGPU_B_COL_MAJOR) ? b_base + k0 : b_base + k0 * ldb; };
	const int64_t b2_shift = DUAL ? (B2 - B) : 0;   // the second right operand has the layout and pitch of the first

	float4_t ra[2][SlabA::kVecs], rb[2][SlabB::kVecs], rb2[2][DUAL ? SlabB::kVecs : 1];   // two staging sets

	float16_t acc[TM][TN], acc2[DUAL ? TM : 1][DUAL ? TN : 1];
#pragma unroll
	for (int i = 0; i < TM; ++i)
#pragma unroll
		for (int j = 0; j < TN; ++j)
#pragma unroll
			for (int r = 0; r < 16; ++r)
			{
				acc[i][j][r] = 0.0f;
				if constexpr (DUAL) acc2[i][j][r] = 0.0f;
			}

	const int frag_row = lane & 31;
	const int kb = (lane >> 5) * 8;          // this lane half's k range inside the slab
	const int64_t ktiles = (K + kBK - 1) / kBK;

	// Five tiles are in flight: tile t is multiplied out of one fragment register set while the
	// fragments of tile t + 1 are read from LDS into the other set, tile t + 2 moves from a
	// staging register set into the LDS buffer tile t has left, tile t + 3 is on its way from
	// memory into the other staging set and the global loads of tile t + 4 are issued (two tile
	// times cover the memory latency).  One barrier per tile separates a buffer's last read from
	// its next write.  Tile indices past the end are clamped to the last tile: its data is
	// fetched and staged again into a buffer nobody multiplies from, which keeps the loop body
	// free of branches.
	float av[2][TM][8], bv[2][TN][8], bv2[2][DUAL ? TN : 1][8];
	const int64_t last = ktiles - 1;

	auto fetch = [&](auto set, int64_t kt) {
		constexpr int S = decltype(set)::value;
		const int64_t k0 = (kt < last ? kt : last) * kBK;
		SlabA::load(ra[S], a_at(k0), lda, M - m0, K - k0, tid);
		SlabB::load(rb[S], b_at(k0), ldb, N - n0, K - k0, tid);
		if constexpr (DUAL) SlabB::load(rb2[S], b_at(k0) + b2_shift, ldb, N - n0, K - k0, tid);
	};
	auto stage = [&](auto set) {               // staging set S -> LDS buffer S
		constexpr int S = decltype(set)::value;
		SlabA::store(a_lds[S], ra[S], tid);
		SlabB::store(b_lds[S], rb[S], tid);
		if constexpr (DUAL) SlabB::store(b2_lds[S], rb2[S], tid);
	};
	auto read_frags = [&](auto set) {          // LDS buffer S -> fragment set S
		constexpr int S = decltype(set)::value;
#pragma unroll
		for (int i = 0; i < TM; ++i) SlabA::fragment(av[S][i], a_lds[S], wm * WTM + i * 32 + frag_row, kb);
#pragma unroll
		for (int j = 0; j < TN; ++j) SlabB::fragment(bv[S][j], b_lds[S], wn * WTN + j * 32 + frag_row, kb);
		if constexpr (DUAL)
		{
#pragma unroll
			for (int j = 0; j < TN; ++j) SlabB::fragment(bv2[S][j], b2_lds[S], wn * WTN + j * 32 + frag_row, kb);
		}
	};
	auto multiply = [&](auto set) {
		constexpr int S = decltype(set)::value;
#pragma unroll
		for (int e = 0; e < 8; ++e)
#pragma unroll
			for (int i = 0; i < TM; ++i)
#pragma unroll
				for (int j = 0; j < TN; ++j)
				{
					acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[S][j][e], av[S][i][e], acc[i][j], 0, 0, 0);
					if constexpr (DUAL)
						acc2[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv2[S][j][e], av[S][i][e], acc2[i][j], 0, 0, 0);
				}
	};
	using Set0 = std::integral_constant<int, 0>;
	using Set1 = std::integral_constant<int, 1>;

	// even tiles live in set / buffer 0, odd tiles in set / buffer 1
	auto step = [&](int64_t kt, auto set) {
		using Other = std::integral_constant<int, decltype(set)::value ^ 1>;
		read_frags(Other{});                       // tile kt + 1
		multiply(set);                             // tile kt
		stage(set);                                // tile kt + 2
		fetch(set, kt + 4);
		if constexpr (FULL_IN)
		{
			// Issue order inside the step: the LDS reads ride on the first half of the MFMAs, the
			// LDS writes and then the global loads (which reuse the registers just written out) on
			// the second half, and the last MFMAs run into the barrier.
			constexpr int kMfma = 8 * TM * TN * (DUAL ? 2 : 1);
			constexpr int kReads = TM * (SlabA::kKContig ? 2 : 4) + (DUAL ? 2 : 1) * TN * (SlabB::kKContig ? 2 : 4);
			constexpr int kMoves = SlabA::kVecs + (DUAL ? 2 : 1) * SlabB::kVecs;
			constexpr int kHalf = kMfma / 2;
			constexpr int kReadsPer = (kReads + kHalf - 1) / kHalf;
			constexpr int kQuarter = kMfma / 4;
			constexpr int kMovesPer = (kMoves + kQuarter - 1) / kQuarter;
#pragma unroll
			for (int i = 0; i < kHalf; ++i)
			{
				__builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
				__builtin_amdgcn_sched_group_barrier(kSchedDsRead, kReadsPer, 0);
			}
#pragma unroll
			for (int i = 0; i < kQuarter; ++i)
			{
				__builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
				__builtin_amdgcn_sched_group_barrier(kSchedDsWrite, kMovesPer, 0);
			}
#pragma unroll
			for (int i = 0; i < kQuarter; ++i)
			{
				__builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
				__builtin_amdgcn_sched_group_barrier(kSchedVmemRead, kMovesPer, 0);
			}
		}
		__syncthreads();
	};

	if (ktiles > 0)
	{
		fetch(Set0{}, 0);
		fetch(Set1{}, 1);
		stage(Set0{});
		fetch(Set0{}, 2);
		stage(Set1{});
		fetch(Set1{}, 3);
		__syncthreads();
		read_frags(Set0{});
		__syncthreads();                           // buffer 0 is overwritten by the first step

		int64_t kt = 0;
		for (; kt + 1 < ktiles; kt += 2)
		{
			step(kt, Set0{});
			step(kt + 1, Set1{});
		}
		if (kt < ktiles) multiply(Set0{});
	}

	// register r of lane l: C[m = l % 32][n = 8 * (r / 4) + 4 * (l / 32) + r % 4] of a 32 x 32 tile
#pragma unroll
	for (int i = 0; i < TM; ++i)
	{
		const int64_t m = m0 + wm * WTM + i * 32 + frag_row;
#pragma unroll
		for (int j = 0; j < TN; ++j)
		{
#pragma unroll
			for (int g = 0; g < 4; ++g)
			{
				const int64_t n = n0 + wn * WTN + j * 32 + 8 * g + 4 * (lane >> 5);
				auto finish = [&](int e) {
					const float sum2 = DUAL ? acc2[DUAL ? i : 0][DUAL ? j : 0][4 * g + e] : 0.0f;
					const float bias_n = (EPI == kEpiBias && bias) ? bias[n + e] : 0.0f;
					return finish_sum<EPI>(acc[i][j][4 * g + e], sum2, bias_n, ep_param);
				};
				if (FULL || (m < M && n + 4 <= N))
				{
					typedef float4_t LooseVec __attribute__((aligned(4)));
					float4_t out;
#pragma unroll
					for (int e = 0; e < 4; ++e) out[e] = finish(e);
					if (ACCESS == kAccessAny || ACCESS == kAccessPadded) *reinterpret_cast<LooseVec*>(C + m * ldc + n) = out;
					else *reinterpret_cast<float4_t*>(C + m * ldc + n) = out;
				}
				else if (m < M)
				{
#pragma unroll
					for (int e = 0; e < 4; ++e)
						if (n + e < N) C[m * ldc + n + e] = finish(e);
				}
			}
		}
	}
}

// One launch of the tile kernel.  k_split > 0: `batch` ranges of K (k_split deep) of a single product, see the kernel.
template <int A_LAYOUT, int B_LAYOUT, int BM, int BN, int EPI>
static hipError_t launch_tiles_once(const float* A, const float* B, const float* B2, const float* bias, float* C,
                                    int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                    int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                                    float ep_param, int64_t k_split, hipStream_t stream, bool padded = false)
{
	// k-contiguous operands in whole 32-deep slabs, one product per tile: the four-wave kernel (gemm_f32_ring.hpp), which
	// keeps the matrix cores busier than this file's kernel does around its barriers (2048^3: 131 -> see the header)
	if constexpr (A_LAYOUT == ANYGPU_A_ROW_MAJOR && BM == BN && EPI != kEpiGeluMul)
	{
		if (gemm_f32_ring_applies(A, B, M, N, K, lda, ldb, stride_a, stride_b, batch, k_split, BM, B_LAYOUT, padded))
			return launch_gemm_f32_ring<BM / 64, EPI, B_LAYOUT == ANYGPU_B_ROW_MAJOR>(A, B, bias, C, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c,
			                                                                        batch, ep_param, k_split, stream, padded);
	}
	const dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM), (unsigned)batch);
	const bool aligned_in = (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(B) % 16 == 0) &&
	                        (reinterpret_cast<uintptr_t>(B2) % 16 == 0) && (lda % 4 == 0) && (ldb % 4 == 0) &&
	                        (stride_a % 4 == 0) && (stride_b % 4 == 0);
	const bool aligned = aligned_in && (reinterpret_cast<uintptr_t>(C) % 16 == 0) && (ldc % 4 == 0) && (stride_c % 4 == 0);
	const bool full = aligned && (M % BM == 0) && (N % BN == 0) && (K % kBK == 0) && (k_split % kBK == 0);
	// padded: the operands are aligned copies that reach, filled with zeros, to the end of the last tile in every direction
	const bool padded_in = padded && aligned_in && (K % kBK == 0) && (k_split % kBK == 0);
	discard_stale_error();
	if (full)
		gemm_f32_kernel<A_LAYOUT, B_LAYOUT, kAccessFull, BM, BN, EPI><<<grid, dim3(256), 0, stream>>>(
			A, B, B2, bias, C, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, ep_param, k_split);
	else if (padded_in)
		gemm_f32_kernel<A_LAYOUT, B_LAYOUT, kAccessPadded, BM, BN, EPI><<<grid, dim3(256), 0, stream>>>(
			A, B, B2, bias, C, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, ep_param, k_split);
	else if (aligned)
		gemm_f32_kernel<A_LAYOUT, B_LAYOUT, kAccessAligned, BM, BN, EPI><<<grid, dim3(256), 0, stream>>>(
			A, B, B2, bias, C, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, ep_param, k_split);
	else
		gemm_f32_kernel<A_LAYOUT, B_LAYOUT, kAccessAny, BM, BN, EPI><<<grid, dim3(256), 0, stream>>>(
			A, B, B2, bias, C, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, ep_param, k_split);
	return hipGetLastError();
}

// C[m, n] = finish(sum over splits of partial[split][m][n]), one thread per four columns, splits added in order
template <int EPI, bool VEC>
__global__ __launch_bounds__(256) void gemm_f32_split_merge_kernel(
	const float* __restrict__ partial, const float* __restrict__ bias, float* __restrict__ C,
	int64_t M, int64_t N, int64_t ldc, int splits, float ep_param)
{
	const int64_t quads = (N + 3) / 4;
	const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
	const int64_t m = item / quads;
	const int64_t n = (item % quads) * 4;
	if (m >= M) return;
	const int64_t plane = M * N;
	const float* src = partial + m * N + n;
	float4_t sum = {0.0f, 0.0f, 0.0f, 0.0f};
	if (VEC)
	{
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
	}
	else
	{
		for (int sp = 0; sp < splits; ++sp)
#pragma unroll
			for (int e = 0; e < 4; ++e)
				if (n + e < N) sum[e] += src[sp * plane + e];
	}
#pragma unroll
	for (int e = 0; e < 4; ++e)
	{
		const float bias_n = (EPI == kEpiBias && bias && n + e < N) ? bias[n + e] : 0.0f;
		sum[e] = finish_sum<EPI>(sum[e], 0.0f, bias_n, ep_param);
	}
	if (VEC) *reinterpret_cast<float4_t*>(C + m * ldc + n) = sum;
	else
	{
#pragma unroll
		for (int e = 0; e < 4; ++e)
			if (n + e < N) C[m * ldc + n + e] = sum[e];
	}
}

// Tiling plan.  A CU works on the blocks it was given side by side, so a launch of 288 tiles takes as long as one
// of 512: some CUs have two blocks.  Two remedies, both priced by a small model of the launch: the smaller tile,
// and for a single product a cut along K.  The model counts "rounds" (blocks per CU) times the 16-deep slabs times
// the time per slab and round, 1.0 us for a 128 x 128 tile and 0.36 us for a 64 x 64 one (2048^3 at 131 us and
// 183 us).  Rounds are whole numbers for the big tile; the small one, of which a CU holds several at once, was
// measured to follow the average beyond two per CU (per slab: 64 tiles 0.32 us, 288 0.64, 576 0.83, 1024 1.43).  Every range of K is then a launch "batch" that writes raw sums to its own [M, N]
// plane of the stream's workspace and a merge kernel adds the planes in order and applies the epilogue; the model
// charges it the merge launch and the traffic of the planes.
struct TilePlan
{
	int tile;          // 128 or 64
	int64_t splits;    // ranges of K, 1 = no cut
	double cost;       // modelled time in us
};

constexpr int64_t kSplitMinDepth = 256;
constexpr int64_t kSplitMax = 16;
// the number of CUs is the device's (256 on an MI355X)
static inline int64_t chip_cus() { return device_cu_count(); }

// four_wave: the product takes the kernels of gemm_f32_ring.hpp, which run at the matrix cores' pace at either tile size
// (per 16 of K and round: 128 x 128 0.9 us, 2048^3 in 123 us; 64 x 64 0.225 us)
static TilePlan plan_tiles(int tile, int64_t M, int64_t N, int64_t K, int64_t batch, bool may_split, size_t workspace_bytes,
                           bool four_wave = false)
{
	const double slab_us = four_wave ? (tile == 128 ? 0.9 : 0.225) : (tile == 128 ? 1.0 : 0.36);
	const int64_t tiles = ((M + tile - 1) / tile) * ((N + tile - 1) / tile) * batch;
	const int64_t slabs = (K + kBK - 1) / kBK;
	// (the four-wave kernels hold two small tiles per CU at most, each then at half pace: whole rounds at either size)
	const auto rounds_of = [tile, four_wave](int64_t blocks) {
		if (tile == 64 && !four_wave && blocks > 2 * chip_cus()) return (double)blocks / (double)chip_cus();
		return (double)((blocks + chip_cus() - 1) / chip_cus());
	};
	// (with a short K the time a block takes to start and to store its tile counts: a CU holds one big tile, whose loads
	// and stores nothing overlaps, or several small ones; 32 x 1024 x 128 . 128 x 1024 batched: 119 -> 111 us, 8192 x 64 -> 8192:
	// 143 -> 133.  From K = 512 on the slab prices alone choose better.)
	const double store_us = (four_wave && K <= 256) ? (tile == 128 ? 3.0 : 0.4) : 0.0;
	TilePlan best{tile, 1, rounds_of(tiles) * ((double)slabs * slab_us + store_us)};
	if (!may_split || batch != 1) return best;
	const int64_t room = (int64_t)(workspace_bytes / ((size_t)M * N * sizeof(float)));
	for (int64_t s = 2; s <= kSplitMax && s <= K / kSplitMinDepth && s <= room; ++s)
	{
		const double rounds = rounds_of(tiles * s);
		// (the planes are written by the product's last waves and read back by a launch that only does that: priced at
		// 6 TB/s, and a cut has to promise 3 % — with 3 TB/s and 10 % products of 48 to 128 rows against wide weight
		// matrices stayed uncut that run 15 % faster in three or four ranges: 64 x 2304 -> 18432 75 -> 63 us)
		const double planes_us = 8.0 * (double)s * (double)M * (double)N / 6.0e6;
		const double cost = rounds * ((double)slabs / (double)s + 5.0) * slab_us + 3.0 + planes_us;
		if (cost < best.cost * 0.97) best = TilePlan{tile, s, cost};
	}
	return best;
}

template <int A_LAYOUT, int B_LAYOUT, int BM, int BN, int EPI>
static hipError_t launch_tiles(const float* A, const float* B, const float* B2, const float* bias, float* C,
                                int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                                float ep_param, int64_t splits, hipStream_t stream, bool padded = false)
{
	if constexpr (EPI != kEpiGeluMul)
	{
		if (splits > 1)
		{
			int64_t k_split = (K + splits - 1) / splits;
			k_split = (k_split + 31) / 32 * 32;             // whole slabs of either kernel family
			splits = (K + k_split - 1) / k_split;
			if (splits > 1)
			{
				float* partial = nullptr;
				const hipError_t ws_err = band::workspace_acquire(stream, &partial);
				if (ws_err != hipSuccess) return ws_err;
				const int64_t step_a = (A_LAYOUT == ANYGPU_A_ROW_MAJOR) ? k_split : k_split * lda;
				const int64_t step_b = (B_LAYOUT == ANYGPU_B_COL_MAJOR) ? k_split : k_split * ldb;
				const hipError_t err = launch_tiles_once<A_LAYOUT, B_LAYOUT, BM, BN, kEpiBias>(
					A, B, nullptr, nullptr, partial, M, N, K, lda, ldb, N, step_a, step_b, M * N, splits, 0.0f, k_split, stream, padded);
				if (err != hipSuccess) return err;
				const int64_t items = M * ((N + 3) / 4);
				const dim3 grid((unsigned)((items + 255) / 256));
				const bool vec = (N % 4 == 0) && (ldc % 4 == 0) && (reinterpret_cast<uintptr_t>(C) % 16 == 0);
				if (vec)
					gemm_f32_split_merge_kernel<EPI, true><<<grid, dim3(256), 0, stream>>>(partial, bias, C, M, N, ldc, (int)splits, ep_param);
				else
					gemm_f32_split_merge_kernel<EPI, false><<<grid, dim3(256), 0, stream>>>(partial, bias, C, M, N, ldc, (int)splits, ep_param);
				return hipGetLastError();
			}
		}
	}
	return launch_tiles_once<A_LAYOUT, B_LAYOUT, BM, BN, EPI>(A, B, B2, bias, C, M, N, K, lda, ldb, ldc,
	                                                          stride_a, stride_b, stride_c, batch, ep_param, 0, stream, padded);
}

template <int A_LAYOUT, int B_LAYOUT, int EPI>
static hipError_t launch_layout(const float* A, const float* B, const float* B2, const float* bias, float* C,
                                int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                                float ep_param, hipStream_t stream, bool padded = false)
{
	const bool may_split = (EPI != kEpiGeluMul);
	// (what the stream's workspace holds bounds the cuts along K: the caller's, or the library's own for eager launches;
	// a stream under capture without a caller's workspace has none and runs uncut)
	const size_t ws_bytes = (may_split && batch == 1) ? band::workspace_capacity(stream) : 0;
	const bool four_wave = A_LAYOUT == ANYGPU_A_ROW_MAJOR && EPI != kEpiGeluMul &&
	                       gemm_f32_ring_applies(A, B, M, N, K, lda, ldb, stride_a, stride_b, batch, 0, 64, B_LAYOUT, padded);
	const TilePlan big = plan_tiles(128, M, N, K, batch, may_split, ws_bytes, four_wave);
	const TilePlan small = plan_tiles(64, M, N, K, batch, may_split, ws_bytes, four_wave);
	if constexpr (EPI != kEpiGeluMul)
	{
		// A product of big tiles that fills whole rounds and a bit, e.g. 576 tiles = 2.25 rounds, pays three rounds.  It
		// is divided by columns into the whole rounds, launched as they are, and the rest, which as a product of its
		// own is cut along K by the plan above (1024 x 2304 x 9216: 411 us as one launch).
		const int64_t tiles_m = (M + 127) / 128, tiles_n = (N + 127) / 128;
		const int64_t whole = tiles_m * tiles_n / chip_cus() * chip_cus();
		const int64_t head_cols = whole / tiles_m;                      // tile columns of the first part
		if (batch == 1 && whole > 0 && head_cols > 0 && head_cols < tiles_n)
		{
			const int64_t n_head = head_cols * 128, n_tail = N - n_head;
			const TilePlan head = plan_tiles(128, M, n_head, K, 1, false, 0, four_wave);
			const TilePlan tail_big = plan_tiles(128, M, n_tail, K, 1, true, ws_bytes, four_wave);
			const TilePlan tail_small = plan_tiles(64, M, n_tail, K, 1, true, ws_bytes, four_wave);
			const TilePlan& tail = tail_big.cost <= tail_small.cost ? tail_big : tail_small;
			const double best_whole = big.cost <= small.cost ? big.cost : small.cost;
			if (head.cost + tail.cost + 3.0 < 0.96 * best_whole)
			{
				const hipError_t err = launch_tiles<A_LAYOUT, B_LAYOUT, 128, 128, EPI>(
					A, B, B2, bias, C, M, n_head, K, lda, ldb, ldc, 0, 0, 0, 1, ep_param, 1, stream, padded);
				if (err != hipSuccess) return err;
				const float* b_tail = (B_LAYOUT == ANYGPU_B_COL_MAJOR) ? B + n_head * ldb : B + n_head;
				const float* bias_tail = bias ? bias + n_head : nullptr;
				if (tail.tile == 128)
					return launch_tiles<A_LAYOUT, B_LAYOUT, 128, 128, EPI>(A, b_tail, nullptr, bias_tail, C + n_head, M, n_tail, K,
					                                                       lda, ldb, ldc, 0, 0, 0, 1, ep_param, tail.splits, stream, padded);
				return launch_tiles<A_LAYOUT, B_LAYOUT, 64, 64, EPI>(A, b_tail, nullptr, bias_tail, C + n_head, M, n_tail, K,
				                                                     lda, ldb, ldc, 0, 0, 0, 1, ep_param, tail.splits, stream, padded);
			}
		}
	}
	if (big.cost <= small.cost)
		return launch_tiles<A_LAYOUT, B_LAYOUT, 128, 128, EPI>(A, B, B2, bias, C, M, N, K, lda, ldb, ldc,
		                                                       stride_a, stride_b, stride_c, batch, ep_param, big.splits, stream, padded);
	return launch_tiles<A_LAYOUT, B_LAYOUT, 64, 64, EPI>(A, B, B2, bias, C, M, N, K, lda, ldb, ldc,
	                                                     stride_a, stride_b, stride_c, batch, ep_param, small.splits, stream, padded);
}

// rows from which (below: the skinny kernels, as for the other band kernel) and up to which (three row blocks of 16;
// with four the fp32 matrix cores, not the memory, are what the product waits for, and the band kernel with the cut
// along K is as fast) the wide band kernel takes fp32 output heads
constexpr int64_t kWideMinRowsF32 = 3;
constexpr int64_t kWideMaxRowsF32 = 48;
// (and with fewer columns where a cut along K fills the chip: 16 x 4096 -> 32000 106 -> 85 us, 16 x 4608 -> 36864 167 -> 120,
// 48 x 5120 -> 65536 367 -> 330)
constexpr int64_t kWideSplitMaxRowsF32 = 48;

hipError_t launch_gemm_f32(const float* A, const float* B, const float* bias, float* C,
                           int64_t M, int64_t N, int64_t K,
                           int64_t lda, int64_t ldb, int64_t ldc,
                           int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                           int a_layout, int b_layout, hipStream_t stream)
{
	if (M == 0 || N == 0 || batch == 0) return hipSuccess;
	// Rows that end a little past a multiple of 64 make a whole further row of tiles, which in fp32 costs matrix-core
	// time, where the few rows past the multiple would only cost another pass over the weights through the few-row
	// kernels: where the plans' prices say so, the product is divided into the multiples of 64 and the rest
	// (65 x 4096 -> 14336: 123 us whole, 67 + 37 divided; 80 x 2304 -> 9216: 57 -> 47; vendor 95 / 39).
	// (a rest of 17 - 32 rows only behind the first 64: 160 x 4096 -> 14336 as 128 + 32 got 3 % slower)
	if (batch == 1 && a_layout == ANYGPU_A_ROW_MAJOR && M > 64 && M % 64 != 0 && M % 64 <= (M < 128 ? 32 : 16))
	{
		const int64_t m_body = M / 64 * 64, m_tail = M - m_body;
		const bool ring = gemm_f32_ring_applies(A, B, M, N, K, lda, ldb, stride_a, stride_b, batch, 0, 64, b_layout, false);
		const size_t ws_bytes = band::workspace_capacity(stream);
		const auto tiles_us = [&](int64_t rows) {
			return std::min(plan_tiles(128, rows, N, K, 1, true, ws_bytes, ring).cost, plan_tiles(64, rows, N, K, 1, true, ws_bytes, ring).cost) + 6.0;
		};
		// the rest: one pass over the weights at what the few-row kernels reach, or its products where those take longer
		const double rest_us = std::max(4.0 * ((double)N + (double)m_tail) * (double)K / 6.0e6,
		                                2.0 * (double)((m_tail + 15) / 16 * 16) * (double)N * (double)K / 1.0e8) + 4.0;
		// (up to 16 rows the few-row kernels reliably run at the pace of the weights: taken at par; beyond, a margin)
		if (tiles_us(m_body) + rest_us < (m_tail <= 16 ? 1.0 : 0.95) * tiles_us(M))
		{
			const hipError_t err = launch_gemm_f32(A, B, bias, C, m_body, N, K, lda, ldb, ldc, 0, 0, 0, 1, a_layout, b_layout, stream);
			if (err != hipSuccess) return err;
			return launch_gemm_f32(A + m_body * lda, B, bias, C + m_body * ldc, m_tail, N, K, lda, ldb, ldc, 0, 0, 0, 1, a_layout, b_layout, stream);
		}
	}
	// Operands that start at an odd address or have an odd row pitch would be fetched element by element, and operands
	// that end inside a tile make the kernel test every vector it fetches (2047^3: 69 TFLOP/s, 2044^3: 70, against 119
	// for 2048^3).  From 128 rows on (fewer rows stream the weights once, which a copy would triple), for products worth two more launches, such operands are copied into the stream's
	// workspace in their own layout, aligned and filled with zeros up to whole tiles of 128 in every direction, and the
	// tile kernels fetch the copies without tests; only the stores into C are guarded.
	const bool a_odd = reinterpret_cast<uintptr_t>(A) % 16 != 0 || lda % 4 != 0;
	const bool b_odd = reinterpret_cast<uintptr_t>(B) % 16 != 0 || ldb % 4 != 0;
	// (the four-wave kernels fetch ragged M and N through their offset tables: no copies where they take the operands as
	// they lie; 270 x 4096 -> 4100: 149 us with copies, 93 without)
	const bool ring_takes = a_layout == ANYGPU_A_ROW_MAJOR && gemm_f32_ring_applies(A, B, M, N, K, lda, ldb, stride_a, stride_b, batch, 0, 64, b_layout, false);
	const bool ragged = !ring_takes && (M % 128 != 0 || N % 128 != 0 || K % kBK != 0);
	if ((a_odd || b_odd || ragged) && batch == 1 && M >= 128 && (double)M * (double)N * (double)K >= (double)(1 << 29))
	{
		const int64_t m_pad = (M + 127) / 128 * 128, n_pad = (N + 127) / 128 * 128, k_pad = (K + 127) / 128 * 128;
		const bool copy_a = a_odd || M % 128 != 0 || K % kBK != 0, copy_b = b_odd || N % 128 != 0 || K % kBK != 0;
		const bool a_rows_m = a_layout == ANYGPU_A_ROW_MAJOR, b_rows_n = b_layout == ANYGPU_B_COL_MAJOR;
		const size_t bytes_a = copy_a ? (size_t)m_pad * k_pad * 4 : 0;
		const size_t bytes_b = copy_b ? (size_t)n_pad * k_pad * 4 : 0;
		if (bytes_a + bytes_b <= band::workspace_copy_capacity(stream))
		{
			float* front = nullptr;
			hipError_t err = band::workspace_acquire(stream, &front, bytes_a + bytes_b);
			if (err != hipSuccess) return err;
			float* a_copy = front;
			float* b_copy = reinterpret_cast<float*>(reinterpret_cast<char*>(front) + bytes_a);
			if (copy_a)
			{
				err = a_rows_m ? launch_repack_rows(A, lda, M, K, a_copy, k_pad, 4, stream, m_pad)
				               : launch_repack_rows(A, lda, K, M, a_copy, m_pad, 4, stream, k_pad);
				if (err != hipSuccess) return err;
			}
			if (copy_b)
			{
				err = b_rows_n ? launch_repack_rows(B, ldb, N, K, b_copy, k_pad, 4, stream, n_pad)
				               : launch_repack_rows(B, ldb, K, N, b_copy, n_pad, 4, stream, k_pad);
				if (err != hipSuccess) return err;
			}
			// (an operand that is used as it lies is whole and aligned already; K grows to the zeros only where both
			// operands have them)
			const int64_t k_used = K % kBK != 0 ? k_pad : K;
			const float* a_use = copy_a ? a_copy : A;
			const float* b_use = copy_b ? b_copy : B;
			const int64_t lda_use = copy_a ? (a_rows_m ? k_pad : m_pad) : lda, ldb_use = copy_b ? (b_rows_n ? k_pad : n_pad) : ldb;
			const band::WorkspaceReserve keep(bytes_a + bytes_b);
#define ANYGPU_F32_PADDED(AL, BL) \
			return launch_layout<AL, BL, kEpiBias>(a_use, b_use, nullptr, bias, C, M, N, k_used, lda_use, ldb_use, ldc, 0, 0, 0, 1, 0.0f, stream, true)
			if (a_rows_m && b_rows_n) ANYGPU_F32_PADDED(ANYGPU_A_ROW_MAJOR, ANYGPU_B_COL_MAJOR);
			if (a_rows_m) ANYGPU_F32_PADDED(ANYGPU_A_ROW_MAJOR, ANYGPU_B_ROW_MAJOR);
			if (b_rows_n) ANYGPU_F32_PADDED(ANYGPU_A_COL_MAJOR, ANYGPU_B_COL_MAJOR);
			ANYGPU_F32_PADDED(ANYGPU_A_COL_MAJOR, ANYGPU_B_ROW_MAJOR);
#undef ANYGPU_F32_PADDED
		}
	}
	// From 33 rows on (where the band kernels go from two row blocks of 16 to two of 32), k-contiguous weights in whole
	// slabs go to the four-wave 64 x 64 tiles cut along K rather than to the band kernels (64 x 4096 -> 6144: 45 us as a
	// band, 37 us in tiles; 40 x 9216 -> 2304: 44 against 28.5, 40 x 4096 -> 14336: 80 against 65; 17 - 32 rows of the
	// same: 48 us as a band, 64 in tiles).
	// ([K, N] weights alike, up to 65536 columns: 48 x 4096 -> 14336 94 us through the band kernel for that layout, 66 in
	// tiles; 9216 -> 2304 59 against 29; with the 256000 columns of an output head the band kernel stays 5 % ahead)
		// (small [K, N] weights, up to 6 M elements, from 17 rows on: 32 x 2048 -> 2048 14.2 -> 11.5 us, 4096 -> 1024 14.5 -> 12)
	const int64_t tiles_first_rows = (b_layout == ANYGPU_B_ROW_MAJOR && (double)K * (double)N <= 6.0e6) ? 17 : 33;
	const bool tiles_first = a_layout == ANYGPU_A_ROW_MAJOR && M >= tiles_first_rows && (b_layout == ANYGPU_B_COL_MAJOR || N <= 65536) &&
	                         gemm_f32_ring_applies(A, B, M, N, K, lda, ldb, stride_a, stride_b, batch, 0, 64, b_layout);
	// few rows against k-contiguous weights with the columns of an output head: whole lines per row and load instruction
	if (batch == 1 && a_layout == ANYGPU_A_ROW_MAJOR && b_layout == ANYGPU_B_COL_MAJOR && M >= kWideMinRowsF32 &&
	    gemm_band_kc_wide_applies<float>(A, B, C, M, N, K, lda, ldb, ldc, kWideMaxRowsF32))
		return launch_gemm_band_kc_wide<float>(A, B, bias, C, M, N, K, lda, ldb, ldc, kEpiBias, 0.0f, stream);
	if (batch == 1 && a_layout == ANYGPU_A_ROW_MAJOR && b_layout == ANYGPU_B_COL_MAJOR && M >= kWideMinRowsF32 &&
	    gemm_band_kc_wide_split_applies<float>(A, B, C, M, N, K, lda, ldb, ldc, kWideSplitMaxRowsF32, stream))
		return launch_gemm_band_kc_wide<float>(A, B, bias, C, M, N, K, lda, ldb, ldc, kEpiBias, 0.0f, stream);
	if (batch == 1 && !tiles_first && a_layout == ANYGPU_A_ROW_MAJOR && gemm_band_applies<float>(A, B, nullptr, C, M, N, K, lda, ldb, ldc, b_layout))
		return launch_gemm_band<float>(A, B, nullptr, bias, C, M, N, K, lda, ldb, ldc, kEpiBias, 0.0f, stream);
	if (batch == 1 && !tiles_first && a_layout == ANYGPU_A_ROW_MAJOR && b_layout == ANYGPU_B_ROW_MAJOR &&
	    gemm_band_ncontig_applies(A, B, nullptr, C, M, N, K, lda, ldb, ldc, false))
		return launch_gemm_band_ncontig(A, B, nullptr, bias, C, M, N, K, lda, ldb, ldc, kEpiBias, 0.0f, stream);
	if (batch == 1 && a_layout == ANYGPU_A_ROW_MAJOR && gemm_skinny_applies<float>(A, B, nullptr, M, N, K, lda, ldb, b_layout))
		return launch_gemm_skinny<float>(A, B, nullptr, bias, C, M, N, K, lda, ldb, ldc, b_layout, kEpiBias, 0.0f, stream);
#define ANYGPU_F32_LAYOUT(AL, BL) \
	return launch_layout<AL, BL, kEpiBias>(A, B, nullptr, bias, C, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, batch, 0.0f, stream)
	if (a_layout == ANYGPU_A_ROW_MAJOR)
	{
		if (b_layout == ANYGPU_B_COL_MAJOR) ANYGPU_F32_LAYOUT(ANYGPU_A_ROW_MAJOR, ANYGPU_B_COL_MAJOR);
		ANYGPU_F32_LAYOUT(ANYGPU_A_ROW_MAJOR, ANYGPU_B_ROW_MAJOR);
	}
	if (b_layout == ANYGPU_B_COL_MAJOR) ANYGPU_F32_LAYOUT(ANYGPU_A_COL_MAJOR, ANYGPU_B_COL_MAJOR);
	ANYGPU_F32_LAYOUT(ANYGPU_A_COL_MAJOR, ANYGPU_B_ROW_MAJOR);
#undef ANYGPU_F32_LAYOUT
}

hipError_t launch_gemm_f32_softcap(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K,
                                   int64_t lda, int64_t ldb, int64_t ldc, int b_layout, float softcap, hipStream_t stream)
{
	if (M == 0 || N == 0) return hipSuccess;
	if (b_layout == ANYGPU_B_COL_MAJOR && M >= kWideMinRowsF32 && gemm_band_kc_wide_applies<float>(A, B, C, M, N, K, lda, ldb, ldc, kWideMaxRowsF32))
		return launch_gemm_band_kc_wide<float>(A, B, nullptr, C, M, N, K, lda, ldb, ldc, kEpiSoftcap, softcap, stream);
	if (b_layout == ANYGPU_B_COL_MAJOR && M >= kWideMinRowsF32 && gemm_band_kc_wide_split_applies<float>(A, B, C, M, N, K, lda, ldb, ldc, kWideSplitMaxRowsF32, stream))
		return launch_gemm_band_kc_wide<float>(A, B, nullptr, C, M, N, K, lda, ldb, ldc, kEpiSoftcap, softcap, stream);
	if (gemm_band_applies<float>(A, B, nullptr, C, M, N, K, lda, ldb, ldc, b_layout))
		return launch_gemm_band<float>(A, B, nullptr, nullptr, C, M, N, K, lda, ldb, ldc, kEpiSoftcap, softcap, stream);
	if (b_layout == ANYGPU_B_ROW_MAJOR && gemm_band_ncontig_applies(A, B, nullptr, C, M, N, K, lda, ldb, ldc, false))
		return launch_gemm_band_ncontig(A, B, nullptr, nullptr, C, M, N, K, lda, ldb, ldc, kEpiSoftcap, softcap, stream);
	if (gemm_skinny_applies<float>(A, B, nullptr, M, N, K, lda, ldb, b_layout))
		return launch_gemm_skinny<float>(A, B, nullptr, nullptr, C, M, N, K, lda, ldb, ldc, b_layout, kEpiSoftcap, softcap, stream);
	if (b_layout == ANYGPU_B_COL_MAJOR)
		return launch_layout<ANYGPU_A_ROW_MAJOR, ANYGPU_B_COL_MAJOR, kEpiSoftcap>(A, B, nullptr, nullptr, C, M, N, K, lda, ldb, ldc,
		                                                                         0, 0, 0, 1, softcap, stream);
	return launch_layout<ANYGPU_A_ROW_MAJOR, ANYGPU_B_ROW_MAJOR, kEpiSoftcap>(A, B, nullptr, nullptr, C, M, N, K, lda, ldb, ldc,
	                                                                         0, 0, 0, 1, softcap, stream);
}

// C[m, n] = gelu_tanh(gate[m, n]) * up[m, n] from two [M, N] planes of sums; VEC: four columns per thread (N a multiple
// of 4, rows of C 16-byte aligned)
template <bool VEC>
__global__ __launch_bounds__(256) void gelu_mul_planes_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                              float* __restrict__ C, int64_t M, int64_t N, int64_t ldc)
{
	constexpr int kPer = VEC ? 4 : 1;
	const int64_t per_row = N / kPer;
	const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (item >= M * per_row) return;
	const int64_t m = item / per_row, n = (item % per_row) * kPer;
	if constexpr (VEC)
	{
		const float4_t g = *reinterpret_cast<const float4_t*>(gate + m * N + n);
		const float4_t u = *reinterpret_cast<const float4_t*>(up + m * N + n);
		float4_t out;
#pragma unroll
		for (int e = 0; e < 4; ++e) out[e] = finish_sum<kEpiGeluMul>(g[e], u[e], 0.0f, 0.0f);
		*reinterpret_cast<float4_t*>(C + m * ldc + n) = out;
	}
	else
		C[m * ldc + n] = finish_sum<kEpiGeluMul>(gate[m * N + n], up[m * N + n], 0.0f, 0.0f);
}

// rows from which the fused up-projection may run as two plain products and a pass that combines them (below, the band
// kernels stream both weight matrices in one launch)
constexpr int64_t kTwoProductsMinRows = 33;

hipError_t launch_gemm_f32_gelu_mul(const float* A, const float* B_gate, const float* B_up, float* C,
                                    int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                    int b_layout, hipStream_t stream)
{
	if (M == 0 || N == 0) return hipSuccess;
	// The plain product has more kernels to choose from (64-row tiles, cuts along K, divided products) than there are
	// forms with this epilogue, whose one four-wave kernel has 128-row tiles of 64 output columns: 40 rows of
	// 2304 -> 9216 took 133 us fused (144 blocks) and take 65 as two products into planes of the stream's workspace and a
	// pass over the planes that combines them; 300 rows 264 -> 217; 512 rows 393 -> 330 (2.25 rounds of blocks fused).
	// Where the fused kernel's blocks come out in whole rounds it stays ahead (384 rows: 261 against 278).  Priced with
	// the plans of the plain product.  Weights stored [K, N] have no four-wave form with this epilogue and run as two
	// products from the same row count on once they are large (1000 x 2304 -> 9216: 991 -> 695 us; 1024 -> 4096 stays).
	bool two_products = false;
	if (M >= kTwoProductsMinRows && K >= 256)
	{
		const bool fused_ring = b_layout == ANYGPU_B_COL_MAJOR && reinterpret_cast<uintptr_t>(B_up) % 16 == 0 &&
		                        gemm_f32_ring_applies(A, B_gate, M, N, K, lda, ldb, 0, 0, 1, 0, 64);
		if (M <= 200 || (!fused_ring && (double)K * (double)N >= 8.0e6)) two_products = true;
		else if (fused_ring)
		{
			const int64_t cus = chip_cus();
			const double slabs = (double)((K + kBK - 1) / kBK);
			const double fused_us = (double)((((M + 127) / 128) * ((N + 63) / 64) + cus - 1) / cus) * slabs * 0.9 + 6.0;
			const size_t ws_bytes = band::workspace_capacity(stream);
			const double plain_us = std::min(plan_tiles(128, M, N, K, 1, true, ws_bytes, true).cost, plan_tiles(64, M, N, K, 1, true, ws_bytes, true).cost) + 6.0;
			const double combine_us = 4.5 + 12.0 * (double)M * (double)N / 5.0e6;
			two_products = 2.0 * plain_us + combine_us < 0.97 * fused_us;
		}
	}
	if (two_products)
	{
		const size_t bytes = ((size_t)2 * M * N * sizeof(float) + 255) / 256 * 256;
		if (bytes <= band::workspace_copy_capacity(stream))
		{
			float* planes = nullptr;
			hipError_t err = band::workspace_acquire(stream, &planes, bytes);
			if (err != hipSuccess) return err;
			const band::WorkspaceReserve keep(bytes);
			float* up = planes + M * N;
			err = launch_gemm_f32(A, B_gate, nullptr, planes, M, N, K, lda, ldb, N, 0, 0, 0, 1, ANYGPU_A_ROW_MAJOR, b_layout, stream);
			if (err != hipSuccess) return err;
			err = launch_gemm_f32(A, B_up, nullptr, up, M, N, K, lda, ldb, N, 0, 0, 0, 1, ANYGPU_A_ROW_MAJOR, b_layout, stream);
			if (err != hipSuccess) return err;
			const bool vec = N % 4 == 0 && ldc % 4 == 0 && reinterpret_cast<uintptr_t>(C) % 16 == 0;
			const int64_t items = vec ? M * (N / 4) : M * N;
			const dim3 grid((unsigned)((items + 255) / 256));
			if (vec) gelu_mul_planes_kernel<true><<<grid, dim3(256), 0, stream>>>(planes, up, C, M, N, ldc);
			else gelu_mul_planes_kernel<false><<<grid, dim3(256), 0, stream>>>(planes, up, C, M, N, ldc);
			return hipGetLastError();
		}
	}
	if (gemm_band_applies<float>(A, B_gate, B_up, C, M, N, K, lda, ldb, ldc, b_layout))
		return launch_gemm_band<float>(A, B_gate, B_up, nullptr, C, M, N, K, lda, ldb, ldc, kEpiGeluMul, 0.0f, stream);
	if (b_layout == ANYGPU_B_ROW_MAJOR && gemm_band_ncontig_applies(A, B_gate, B_up, C, M, N, K, lda, ldb, ldc, true))
		return launch_gemm_band_ncontig(A, B_gate, B_up, nullptr, C, M, N, K, lda, ldb, ldc, kEpiGeluMul, 0.0f, stream);
	if (gemm_skinny_applies<float>(A, B_gate, B_up, M, N, K, lda, ldb, b_layout))
		return launch_gemm_skinny<float>(A, B_gate, B_up, nullptr, C, M, N, K, lda, ldb, ldc, b_layout, kEpiGeluMul, 0.0f, stream);
	// k-contiguous weights in whole slabs: the four-wave kernel with gate and up rows side by side in its B unit
	// (2048 x 2304 -> 9216: 1.40 -> 1.27 ms)
	if (b_layout == ANYGPU_B_COL_MAJOR && reinterpret_cast<uintptr_t>(B_up) % 16 == 0 &&
	    gemm_f32_ring_applies(A, B_gate, M, N, K, lda, ldb, 0, 0, 1, 0, 64))
		return launch_gemm_f32_ring<2, kEpiGeluMul>(A, B_gate, B_up, C, M, N, K, lda, ldb, ldc, 0, 0, 0, 1, 0.0f, 0, stream);
	if (b_layout == ANYGPU_B_COL_MAJOR)
		return launch_layout<ANYGPU_A_ROW_MAJOR, ANYGPU_B_COL_MAJOR, kEpiGeluMul>(A, B_gate, B_up, nullptr, C, M, N, K, lda, ldb, ldc,
		                                                                         0, 0, 0, 1, 0.0f, stream);
	return launch_layout<ANYGPU_A_ROW_MAJOR, ANYGPU_B_ROW_MAJOR, kEpiGeluMul>(A, B_gate, B_up, nullptr, C, M, N, K, lda, ldb, ldc,
	                                                                         0, 0, 0, 1, 0.0f, stream);
}

}  // namespace anygpu
