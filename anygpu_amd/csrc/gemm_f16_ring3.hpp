// 256 x 128 and 128 x 128 tiles of the fp16 GEMM (A [M, K], B [N, K], both k-contiguous) for whole 64-deep slabs: the
// four-wave scheme of gemm_f16_ring.hpp with smaller patches (128 x 64 or 64 x 64 per wave), for products that do not
// fill the chip with 256 x 256 tiles.  Three LDS stages of an A unit and a B unit each, a 64-deep slab per stage; the main
// loop is an assembly block with fixed registers (gemm_f16_ring_loop_8x4.inc, _4x4.inc, written by
// gen_gemm_f16_ring_loop.py, which explains the stage rotation and the schedule).
#pragma once

#include "anygpu_hip.h"
#include "gemm_f16_ring.hpp"

namespace anygpu {

// TM x TN MFMA tiles (16 x 16) per wave, 2 x 2 waves
template <int TM, int TN>
struct GemmRing3Cfg
{
	static_assert((TM == 8 && TN == 4) || (TM == 4 && TN == 4), "the loops that are generated");
	static constexpr int BM = 32 * TM, BN = 32 * TN, BK = 64, MI = 16;
	static constexpr int kThreads = 256, kWaves = 4;
	static constexpr int kStageBytes = (BM + BN) * 128;
	static constexpr int kTableBytes = 4 * 16 * 64 * 4;        // per wave 16 load offsets per lane
	static constexpr int kLdsBytes = 3 * kStageBytes + kTableBytes;
	static constexpr int kWaveM = 16 * TM, kWaveN = 16 * TN, kTilesM = TM, kTilesN = TN;
	static constexpr int WM = 2, WN = 2;
	static constexpr int kLoadsA = BM / 32, kLoadsB = BN / 32;  // per wave and slab: 8 rows of 128 bytes each
};

// blockIdx.y walks a batch of independent products that share the shape.  K a multiple of 64.  RAGGED: M and N need not
// be multiples of the tile and C may start and step at any element; operand rows past the end are read from the last
// valid row and the stores are guarded.
// SPLIT: blockIdx.y walks ranges of K (k_split deep, a multiple of 64; the strides step along K) of one product instead
// of a batch, and the raw fp32 sums of range y go to planes[y][M][N]; C is not touched.
// EPI: kEpiNone, kEpiBias (+ bias[n]) or kEpiSoftcap (ep_param * tanh(sum / ep_param)), applied to the fp32 sums (not SPLIT);
// or kEpiGeluMul: the tile is BN / 2 output columns wide and its B unit holds, for every wave column, gate rows (from B) in
// front of up rows (from `bias`, which then is the second weight matrix), as in gemm_f16_nt_ring_kernel.
// B_KN: B stored [K, N] (N a multiple of 8): a B unit of 64 k rows x BN n, filled four rows per load, fragments by
// transposing reads (gemm_f16_ring_loop_8x4kn.inc, _4x4kn.inc); not with kEpiGeluMul.
template <int TM, int TN, bool RAGGED, bool SPLIT, int EPI = kEpiNone, bool B_KN = false>
__global__ __launch_bounds__(256) void gemm_f16_nt_ring3_kernel(
	const half_t* __restrict__ A, const half_t* __restrict__ B, half_t* __restrict__ C,
	int K, int64_t lda, int64_t ldb, int64_t ldc, int tiles_m, int tiles_n,
	int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t M, int64_t N, float* __restrict__ planes, int k_split,
	const half_t* __restrict__ bias = nullptr, float ep_param = 0.0f)
{
	static_assert(!SPLIT || EPI == kEpiNone, "the planes hold raw sums");
	static_assert(!B_KN || EPI != kEpiGeluMul, "two weight matrices: k-contiguous only");
	static_assert(TN == 4, "a [K, N] unit row of 256 bytes: 16 chunks, four k rows per load");
	using Cfg = GemmRing3Cfg<TM, TN>;
	extern __shared__ __align__(1024) char lds[];
	if constexpr (SPLIT)
	{
		const int left = K - (int)blockIdx.y * k_split;
		K = left < k_split ? left : k_split;
	}

	A += (int64_t)blockIdx.y * stride_a;
	B += (int64_t)blockIdx.y * stride_b;
	C += (int64_t)blockIdx.y * stride_c;
	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wm = wave >> 1, wn = wave & 1;

	int tile_m, tile_n;
	tile_of_block<4>(blockIdx.x, tiles_m, tiles_n, tile_m, tile_n);
	const int64_t m0 = (int64_t)tile_m * Cfg::BM;
	constexpr bool DUAL = EPI == kEpiGeluMul;
	const int64_t n0 = (int64_t)tile_n * (DUAL ? Cfg::BN / 2 : Cfg::BN);
	// DUAL: the unit rows wave w loads are output columns (BN / 4) (w / 2) .. of the tile, from B (w even) or B2
	const half_t* const b_of_wave = DUAL && (wave & 1) ? bias : B;
	const int b_unit_row = DUAL ? 8 * Cfg::kLoadsB * (wave >> 1) : 8 * Cfg::kLoadsB * wave;

	// Direct loads.  A unit row is 64 halves = eight 16-byte chunks; chunk c of row r sits at position c ^ ((r >> 1) & 7).
	// One instruction fills 8 rows: lane -> row lane / 8, position lane % 8.  Instruction q of this wave covers rows
	// 8 (kLoads wave + q) .. + 7 of the unit.  The lane's byte offsets from the wave's first row go to the assembly block
	// through a table behind the stages: table[q][lane], q < 8 for A, 8 + q for B.
	const unsigned lds0 = (unsigned)(uintptr_t)(const __attribute__((address_space(3))) char*)lds;
	const int ld_row = lane >> 3, ld_pos = lane & 7;
	unsigned* const table = reinterpret_cast<unsigned*>(lds + 3 * Cfg::kStageBytes) + wave * (16 * 64) + lane;
	int64_t a_first = m0 + 8 * Cfg::kLoadsA * wave, b_first = n0 + b_unit_row;
	if constexpr (RAGGED)
	{
		a_first = a_first < M - 1 ? a_first : M - 1;
		b_first = b_first < N - 1 ? b_first : N - 1;
	}
#pragma unroll
	for (int q = 0; q < Cfg::kLoadsA; ++q)
	{
		const int row = 8 * (Cfg::kLoadsA * wave + q) + ld_row;
		int64_t a_row = m0 + row;
		if constexpr (RAGGED) a_row = a_row < M - 1 ? a_row : M - 1;
		table[64 * q] = (unsigned)(((a_row - a_first) * lda + ((ld_pos ^ ((row >> 1) & 7)) << 3)) * 2);
	}
#pragma unroll
	for (int q = 0; q < Cfg::kLoadsB; ++q)
	{
		const int row = 8 * (Cfg::kLoadsB * wave + q) + ld_row;                  // in the unit
		int64_t b_row = n0 + b_unit_row + 8 * q + ld_row;                        // in the matrix
		if constexpr (RAGGED) b_row = b_row < N - 1 ? b_row : N - 1;
		if constexpr (B_KN)
		{
			// one instruction fills 4 k rows of 256 bytes: lane -> row lane / 16, position lane % 16, and the chunk at
			// position p of row k is chunk p ^ kn_row_swizzle(k); instruction q covers rows 16 wave + 4 q .. + 3
			const int k_wave = 4 * q + (lane >> 4);
			int64_t col = (int64_t)(((lane & 15) ^ kn_row_swizzle(16 * wave + k_wave)) << 3);
			if constexpr (RAGGED)
				if (n0 + col + 8 > N) col = N - 8 - n0;
			table[64 * (8 + q)] = (unsigned)((k_wave * ldb + col) * 2);
		}
		else
			table[64 * (8 + q)] = (unsigned)(((b_row - b_first) * ldb + ((ld_pos ^ ((row >> 1) & 7)) << 3)) * 2);
	}
	const unsigned table_addr = lds0 + 3 * Cfg::kStageBytes + (wave * (16 * 64) + lane) * 4;
	const uintptr_t a_wave = reinterpret_cast<uintptr_t>(A + a_first * lda);
	const uintptr_t b_wave = reinterpret_cast<uintptr_t>(B_KN ? B + (int64_t)(16 * wave) * ldb + n0 : b_of_wave + b_first * ldb);
	const unsigned share_a = wave * (Cfg::kLoadsA * 1024);                       // the wave's rows inside a stage
	const unsigned share_b = Cfg::BM * 128 + wave * (Cfg::kLoadsB * 1024);
	const int slabs = K / 64;

	// Fragments: lane -> row lane % 16 of its MFMA tile, k group lane / 16 (8 halves) of the 32-deep step; addresses
	// inside a stage, the B unit behind the A unit.
	const unsigned frag_row = lane & 15;
	const unsigned frag_chunk = (lane >> 4) ^ ((frag_row >> 1) & 7);
	const unsigned a_addr = (wm * Cfg::kWaveM + frag_row) * 128 + frag_chunk * 16;
	// B stored [K, N]: lane r of a 16-lane group points a transposing read at k row 8 g + r / 4 (g: the lane's k group),
	// columns 4 (r % 4) .. + 3 of the MFMA tile; column tile j of wave column wn lies at chunk pair (4 wn + j) ^ (row
	// swizzle / 2), which the assembly block adds per tile from `b_swizzle`
	const unsigned kn_k = 8 * (lane >> 4) + (frag_row >> 2);
	const unsigned b_addr = B_KN ? Cfg::BM * 128 + kn_k * 256 + ((frag_row & 3) >> 1) * 16 + 8 * (frag_row & 1)
	                             : Cfg::BM * 128 + (wn * Cfg::kWaveN + frag_row) * 128 + frag_chunk * 16;
	[[maybe_unused]] const unsigned b_swizzle = (unsigned)((kn_row_swizzle((int)kn_k) >> 1) ^ (wn << 2)) << 5;
	[[maybe_unused]] const unsigned b_step = (unsigned)(128 * ldb);      // bytes from one [K, N] slab to the next

	// The accumulators leave the block as vectors of 32 registers pinned to a[0 : 4 TM TN): MFMA tile (i, j) in registers
	// 4 (TN i + j) .. + 3.
	constexpr int kVectors = TM * TN * 4 / 32;
	float32x_t r0, r1, r2 = {}, r3 = {};
#define ANYGPU_RING3_INPUTS \
	[vtab] "v"(table_addr), [aaddr] "v"(a_addr), [baddr] "v"(b_addr), \
	[abaselo] "s"((unsigned)a_wave), [abasehi] "s"((unsigned)(a_wave >> 32)), \
	[bbaselo] "s"((unsigned)b_wave), [bbasehi] "s"((unsigned)(b_wave >> 32)), \
	[lds0] "s"(lds0), [ldsa] "s"(share_a), [ldsb] "s"(share_b), [slabs] "s"(slabs)
#define ANYGPU_RING3_CLOBBERS \
	"v80", "v81", "v82", "v83", "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", "v94", "v95", \
	"v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109", \
	"v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123", \
	"v124", "v125", "v126", "v127", "v128", "v129", "v130", "v131", "v132", "v133", "v134", "v135", "v136", "v137", \
	"v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", "v147", "v148", "v149", "v150", "v151", \
	"v152", "v153", "v154", "v155", "v156", "v157", "v158", "v159", "v160", "v161", "v162", "v163", "v164", "v165", \
	"v166", "v167", "v168", "v169", "v170", "v171", "v172", "v173", "v174", "v175", "v176", "v177", "v178", "v179", \
	"v180", "v181", "v182", "v183", "v184", "v185", "v186", "v187", "v188", "v189", "v190", "v191", "v192", "v193", \
	"v194", "v195", "v196", "v197", "v198", "v199", "v200", "v201", "v202", "v203", "v204", "v205", "v206", "v207", \
	"v208", "v209", "v210", "v211", "v212", "v213", "v214", "v215", "v216", "v217", "v218", "v219", "v220", "v221", \
	"v222", "v223", "v224", "v225", "v226", "v227", "v228", "v229", "v230", "v231", "v232", "v233", "v234", "v235", \
	"v236", "v237", "v238", "v239", "v240", "v241", "v242", "v243", "v244", "v245", "v246", "v247", "v248", "v249", \
	"v250", "v251", "v252", "v253", "v254", "v255", "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", \
	"s69", "s70", "s71", "s72", "s73", "s74", "scc", "m0", "memory"
	if constexpr (TM == 8 && B_KN)
		asm volatile(
#include "gemm_f16_ring_loop_8x4kn.inc"
			: "={a[0:31]}"(r0), "={a[32:63]}"(r1), "={a[64:95]}"(r2), "={a[96:127]}"(r3)
			: ANYGPU_RING3_INPUTS, [bsx] "v"(b_swizzle), [bstep] "s"(b_step)
			: ANYGPU_RING3_CLOBBERS);
	else if constexpr (B_KN)
		asm volatile(
#include "gemm_f16_ring_loop_4x4kn.inc"
			: "={a[0:31]}"(r0), "={a[32:63]}"(r1)
			: ANYGPU_RING3_INPUTS, [bsx] "v"(b_swizzle), [bstep] "s"(b_step)
			: ANYGPU_RING3_CLOBBERS);
	else if constexpr (TM == 8)
		asm volatile(
#include "gemm_f16_ring_loop_8x4.inc"
			: "={a[0:31]}"(r0), "={a[32:63]}"(r1), "={a[64:95]}"(r2), "={a[96:127]}"(r3)
			: ANYGPU_RING3_INPUTS
			: ANYGPU_RING3_CLOBBERS);
	else
		asm volatile(
#include "gemm_f16_ring_loop_4x4.inc"
			: "={a[0:31]}"(r0), "={a[32:63]}"(r1)
			: ANYGPU_RING3_INPUTS
			: ANYGPU_RING3_CLOBBERS);
#undef ANYGPU_RING3_INPUTS
#undef ANYGPU_RING3_CLOBBERS

	float4_t acc[TM][TN];
	const float32x_t* vectors[4] = {&r0, &r1, &r2, &r3};
#pragma unroll
	for (int i = 0; i < TM; ++i)
#pragma unroll
		for (int j = 0; j < TN; ++j)
		{
			constexpr int kPerVector = 8;                            // MFMA tiles in a vector of 32 registers
			const int t = TN * i + j;
			const float32x_t& v = *vectors[(t / kPerVector) % kVectors];
			acc[i][j] = float4_t{v[4 * (t % kPerVector)], v[4 * (t % kPerVector) + 1], v[4 * (t % kPerVector) + 2], v[4 * (t % kPerVector) + 3]};
			if constexpr (SPLIT)
			{
				// (every sum into an ordinary register here, in straight-line code: taken out of the pinned vectors inside
				// the guarded stores below, the compiler produced a move it then rejected)
#pragma unroll
				for (int e = 0; e < 4; ++e)
				{
					float x = acc[i][j][e];
					asm volatile("" : "+v"(x));
					acc[i][j][e] = x;
				}
			}
		}
	if constexpr (SPLIT)
		store_patch_f32<Cfg>(acc, planes + (int64_t)blockIdx.y * M * N, m0 + wm * Cfg::kWaveM, n0 + wn * Cfg::kWaveN, lane, M, N);
	else
		store_patch_via_lds<Cfg, RAGGED, !RAGGED, EPI>(acc, lds, C, ldc, m0 + wm * Cfg::kWaveM, n0 + wn * (DUAL ? Cfg::kWaveN / 2 : Cfg::kWaveN),
		                                               wave, lane, M, N, bias, ep_param);
}

// planes != NULL: `batch` is the number of K ranges, k_split their depth, and the strides step along K.
template <int TM, int TN, int EPI = kEpiNone>
inline hipError_t launch_gemm_f16_ring3(const half_t* A, const half_t* B, half_t* C, int64_t M, int64_t N, int64_t K,
                                        int64_t lda, int64_t ldb, int64_t ldc,
                                        int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch, hipStream_t stream,
                                        float* planes = nullptr, int64_t k_split = 0, const half_t* bias = nullptr, float ep_param = 0.0f,
                                        int b_layout = ANYGPU_B_COL_MAJOR)
{
	using Cfg = GemmRing3Cfg<TM, TN>;
	const bool kn = b_layout == ANYGPU_B_ROW_MAJOR;
	const bool c_aligned = reinterpret_cast<uintptr_t>(C) % 16 == 0 && ldc % 8 == 0 && stride_c % 8 == 0;
	constexpr int kOutN = EPI == kEpiGeluMul ? Cfg::BN / 2 : Cfg::BN;       // output columns of a tile
	const bool ragged = M % Cfg::BM != 0 || N % kOutN != 0 || !c_aligned;
	const int which = planes != nullptr ? 2 : ragged ? 1 : 0;
	auto kernel = which == 1 ? gemm_f16_nt_ring3_kernel<TM, TN, true, false, EPI> : gemm_f16_nt_ring3_kernel<TM, TN, false, false, EPI>;
	if constexpr (EPI == kEpiNone)
	{
		if (which == 2) kernel = gemm_f16_nt_ring3_kernel<TM, TN, true, true, kEpiNone>;
		if (kn)
			kernel = which == 2 ? gemm_f16_nt_ring3_kernel<TM, TN, true, true, kEpiNone, true>
			       : which == 1 ? gemm_f16_nt_ring3_kernel<TM, TN, true, false, kEpiNone, true> : gemm_f16_nt_ring3_kernel<TM, TN, false, false, kEpiNone, true>;
	}
	else if (which == 2 || kn) return hipErrorInvalidValue;
	// More than 64 KB of dynamic LDS has to be granted per function and per device, once.
	static std::atomic<uint64_t> configured_devices[6];
	(void)hipGetLastError();
	int device = 0;
	hipError_t e = hipGetDevice(&device);
	if (e != hipSuccess) return e;
	const uint64_t bit = 1ull << (device & 63);
	const int slot = which + 3 * kn;
	if ((configured_devices[slot].load(std::memory_order_relaxed) & bit) == 0)
	{
		e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::kLdsBytes);
		if (e != hipSuccess) return e;
		configured_devices[slot].fetch_or(bit, std::memory_order_relaxed);
	}
	const int tiles_m = (int)((M + Cfg::BM - 1) / Cfg::BM), tiles_n = (int)((N + kOutN - 1) / kOutN);
	kernel<<<dim3((unsigned)(tiles_m * tiles_n), (unsigned)batch), dim3(256), Cfg::kLdsBytes, stream>>>(
		A, B, C, (int)K, lda, ldb, ldc, tiles_m, tiles_n, stride_a, stride_b, stride_c, M, N, planes, (int)k_split, bias, ep_param);
	return hipGetLastError();
}

}  // namespace anygpu
