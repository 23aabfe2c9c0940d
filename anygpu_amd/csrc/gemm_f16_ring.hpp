// 256 x 256 tile of the fp16 GEMM (A [M, K]; B [N, K], k-contiguous like A, or [K, N]) for whole 64-deep slabs: four
// waves, one per SIMD, each with a 128 x 128 patch of C in 256 accumulator registers, v_mfma_f32_16x16x32_f16.
//
// Against the eight-wave tile kernel (128 x 64 patches) a patch of 128 x 128 needs a third fewer LDS bytes per MFMA, and
// under this product the MI355X is power-limited: the bytes saved come back as clock.  One wave per SIMD has nobody to
// hide its stalls, so the main loop is one block of assembly with fixed registers (gemm_f16_ring_loop.inc, written by
// gen_gemm_f16_ring_loop.py, which also describes the register plan, the five-unit LDS ring and the schedule).  Measured
// in that loop at 4096^3: the matrix cores busy 94 - 95 % of the cycles at the 1.6 GHz the part sustains under it.
#pragma once

#include "anygpu_hip.h"
#include "gemm_f16_tile.hpp"

namespace anygpu {

typedef float float32x_t __attribute__((ext_vector_type(32)));

struct GemmRingCfg
{
	static constexpr int BM = 256, BN = 256, BK = 64, MI = 16;
	static constexpr int kThreads = 256, kWaves = 4;
	static constexpr int kUnitBytes = 256 * 128;          // one operand, one 64-deep slab
	static constexpr int kUnits = 5;
	static constexpr int kLdsBytes = kUnits * kUnitBytes;
	static constexpr int kWaveM = 128, kWaveN = 128, kTilesM = 8, kTilesN = 8;
	static constexpr int WM = 2, WN = 2;
};

// blockIdx.y walks a batch of independent products that share the shape.  K a multiple of 64.
// RAGGED: M and N need not be multiples of 256 and C may start and step at any element.  Operand rows past the end are
// read from the last valid row instead (they only feed results that are not stored) and the stores are guarded.
// probe (may be NULL; first product of a batch only): lane 0 of every block leaves the shader clock count (s_memtime) and
// the constant 100 MHz count (s_memrealtime) at entry and exit of its main loop in probe[4 block .. + 3], from which a
// caller gets the clock the part sustained under this kernel and the share of those cycles the matrix cores were busy.
// B_KN: B stored [K, N] (row k holds the n), staged as a [64 k][256 n] unit and read through transposing LDS reads; N is a
// multiple of 8 then, and column chunks past N are read from the last whole chunk of the row.
// EPI: kEpiNone, kEpiBias (+ bias[n]) or kEpiSoftcap (ep_param * tanh(sum / ep_param)), applied to the fp32 sums; or
// kEpiGeluMul (k-contiguous weights only): the tile is 128 output columns wide (N and tiles_n count those) and its B unit
// is put together from two matrices: of every wave column's 128 unit rows the first 64 come from B (the gate weights) and
// the second 64 from `bias`, which then is the second matrix B2 (the up weights, same pitch), both for the same 64 output
// columns, so that gate and up sums of an output element meet in one lane, A is read once for both products and
// gelu_tanh(gate) * up goes out.  The wave that loads a quarter of the unit loads it from one matrix.
template <bool RAGGED, bool B_KN, int EPI = kEpiNone>
__global__ __launch_bounds__(256) void gemm_f16_nt_ring_kernel(
	const half_t* __restrict__ A, const half_t* __restrict__ B, half_t* __restrict__ C,
	int K, int64_t lda, int64_t ldb, int64_t ldc, int tiles_m, int tiles_n,
	int64_t stride_a, int64_t stride_b, int64_t stride_c, unsigned long long* __restrict__ probe, int64_t M, int64_t N,
	const half_t* __restrict__ bias = nullptr, float ep_param = 0.0f)
{
	using Cfg = GemmRingCfg;
	extern __shared__ __align__(1024) char lds[];

	A += (int64_t)blockIdx.y * stride_a;
	B += (int64_t)blockIdx.y * stride_b;
	C += (int64_t)blockIdx.y * stride_c;
	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int wm = wave >> 1, wn = wave & 1;

	int tile_m, tile_n;
	tile_of_block<4>(blockIdx.x, tiles_m, tiles_n, tile_m, tile_n);
	const int64_t m0 = (int64_t)tile_m * 256;
	constexpr bool DUAL = EPI == kEpiGeluMul;
	static_assert(!DUAL || !B_KN, "two weight matrices: k-contiguous only");
	const int64_t n0 = (int64_t)tile_n * (DUAL ? 128 : 256);
	// DUAL: unit rows 64 w .. + 63 of wave w are output columns 64 (w / 2) .. + 63 of the tile, from B (w even) or B2
	const half_t* const b_of_wave = DUAL && (wave & 1) ? bias : B;
	const int b_unit_row = DUAL ? 64 * (wave >> 1) : 64 * wave;       // the wave's first row, as a column of the tile

	// Direct loads.  A unit row is 64 halves = 128 bytes = eight 16-byte chunks; chunk c of row r sits at position
	// c ^ ((r >> 1) & 7).  One instruction fills 8 rows: lane -> row lane / 8, position lane % 8.  Instruction q of this
	// wave covers rows 64 wave + 8 q .. + 7 of the operand's 256.  The lane's byte offset from the tile's first row for
	// each of its 16 loads of a slab goes to the assembly block through a table in LDS (the fifth unit, which the loop
	// fills last): table[q][lane] for this wave, q < 8 for A, the rest for B.
	const unsigned lds0 = (unsigned)(uintptr_t)(const __attribute__((address_space(3))) char*)lds;
	const int ld_row = lane >> 3, ld_pos = lane & 7;
	unsigned* const table = reinterpret_cast<unsigned*>(lds + 4 * Cfg::kUnitBytes) + wave * (16 * 64) + lane;
	// (offsets count from the first row of the wave's 64, which keeps them below 2^32 for the row pitches admitted)
	// A [K, N] unit of B has rows of 256 n = 512 bytes = 32 chunks; one instruction fills 2 k rows: lane -> row lane / 32,
	// position lane % 32, and the chunk at position p of row k is chunk p ^ kn_row_swizzle(k).  Instruction q of this wave
	// covers rows 16 wave + 2 q, + 1 of the slab's 64.
	int64_t a_first = m0 + 64 * wave, b_first = n0 + b_unit_row;
	if constexpr (RAGGED)
	{
		a_first = a_first < M - 1 ? a_first : M - 1;
		b_first = b_first < N - 1 ? b_first : N - 1;
	}
#pragma unroll
	for (int q = 0; q < 8; ++q)
	{
		const int row = 64 * wave + 8 * q + ld_row;
		const unsigned chunk = ld_pos ^ ((row >> 1) & 7);
		int64_t a_row = m0 + row, b_row = n0 + b_unit_row + 8 * q + ld_row;
		if constexpr (RAGGED)
		{
			a_row = a_row < M - 1 ? a_row : M - 1;
			b_row = b_row < N - 1 ? b_row : N - 1;
		}
		table[64 * q] = (unsigned)(((a_row - a_first) * lda + chunk * 8) * 2);
		if constexpr (B_KN)
		{
			const int k_wave = 2 * q + (lane >> 5);                // the k row, counted from the wave's first
			int64_t col = (int64_t)(((lane & 31) ^ kn_row_swizzle(16 * wave + k_wave)) << 3);
			if constexpr (RAGGED)
				if (n0 + col + 8 > N) col = N - 8 - n0;
			table[64 * (8 + q)] = (unsigned)((k_wave * ldb + col) * 2);
		}
		else
			table[64 * (8 + q)] = (unsigned)(((b_row - b_first) * ldb + chunk * 8) * 2);
	}
	const unsigned table_addr = lds0 + 4 * Cfg::kUnitBytes + (wave * (16 * 64) + lane) * 4;
	const uintptr_t a_wave = reinterpret_cast<uintptr_t>(A + a_first * lda);
	const uintptr_t b_wave = reinterpret_cast<uintptr_t>(B_KN ? B + (int64_t)(16 * wave) * ldb + n0 : b_of_wave + b_first * ldb);
	const unsigned wave_share = wave * 8192;               // the wave's 64 rows inside a unit
	const unsigned lds_wave = lds0 + wave_share;
	const int slabs = K / 64;

	// Fragments: lane -> row lane % 16 of its MFMA tile, k group lane / 16 (8 halves) of the 32-deep step.  Relative to
	// the unit offsets the loop keeps, which include the wave's share.
	const unsigned frag_row = lane & 15;
	const unsigned frag_chunk = (lane >> 4) ^ ((frag_row >> 1) & 7);
	const unsigned a_addr = (wm * 128 + frag_row) * 128 + frag_chunk * 16 - wave_share;
	// B stored [K, N]: lane r of a 16-lane group points a transposing read at k row 8 g + r / 4 (g: the lane's k group),
	// columns 4 (r % 4) .. + 3 of the MFMA tile; tile j of the patch lies at chunk pair j ^ (row swizzle / 2), a term the
	// assembly block adds per tile from `b_swizzle`.
	const unsigned kn_k = 8 * (lane >> 4) + (frag_row >> 2);
	const unsigned b_addr = B_KN ? kn_k * 512 + (wn * 16 + ((frag_row & 3) >> 1)) * 16 + 8 * (frag_row & 1) - wave_share
	                             : (wn * 128 + frag_row) * 128 + frag_chunk * 16 - wave_share;
	[[maybe_unused]] const unsigned b_swizzle = (unsigned)(kn_row_swizzle((int)kn_k) >> 1) << 5;
	[[maybe_unused]] const unsigned b_step = (unsigned)(128 * ldb);      // bytes from one [K, N] slab to the next

	// The accumulators leave the block as eight vectors of 32 registers pinned to a[0:255]: row i of the patch's MFMA
	// tiles in vector i.
	unsigned long long clock_in = 0, ticks_in = 0;
	if (probe != nullptr)
	{
		clock_in = __builtin_amdgcn_s_memtime();
		ticks_in = __builtin_amdgcn_s_memrealtime();
	}
	float32x_t r0, r1, r2, r3, r4, r5, r6, r7;
#define ANYGPU_RING_OUTPUTS \
	"={a[0:31]}"(r0), "={a[32:63]}"(r1), "={a[64:95]}"(r2), "={a[96:127]}"(r3), \
	"={a[128:159]}"(r4), "={a[160:191]}"(r5), "={a[192:223]}"(r6), "={a[224:255]}"(r7)
#define ANYGPU_RING_INPUTS \
	[vtab] "v"(table_addr), [aaddr] "v"(a_addr), [baddr] "v"(b_addr), \
	[abaselo] "s"((unsigned)a_wave), [abasehi] "s"((unsigned)(a_wave >> 32)), \
	[bbaselo] "s"((unsigned)b_wave), [bbasehi] "s"((unsigned)(b_wave >> 32)), \
	[ldsw] "s"(lds_wave), [slabs] "s"(slabs)
#define ANYGPU_RING_CLOBBERS \
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
	"s69", "s70", "s71", "s72", "s73", "scc", "m0", "memory"
	if constexpr (B_KN)
		asm volatile(
#include "gemm_f16_ring_loop_kn.inc"
			: ANYGPU_RING_OUTPUTS
			: ANYGPU_RING_INPUTS, [bsx] "v"(b_swizzle), [bstep] "s"(b_step)
			: ANYGPU_RING_CLOBBERS);
	else
		asm volatile(
#include "gemm_f16_ring_loop.inc"
			: ANYGPU_RING_OUTPUTS
			: ANYGPU_RING_INPUTS
			: ANYGPU_RING_CLOBBERS);
#undef ANYGPU_RING_OUTPUTS
#undef ANYGPU_RING_INPUTS
#undef ANYGPU_RING_CLOBBERS

	// (the lane number is derived again, from a thread number the compiler takes for a new value: the loop leaves it
	// no register to carry one through, and a spilled value would make the kernel a user of scratch memory)
	int tid_after = threadIdx.x;
	asm volatile("" : "+v"(tid_after));
	const int lane_after = tid_after & 63;
	if (probe != nullptr)
	{
		const unsigned long long clock_out = __builtin_amdgcn_s_memtime(), ticks_out = __builtin_amdgcn_s_memrealtime();
		if (tid_after == 0 && blockIdx.y == 0)
		{
			unsigned long long* slot = probe + 4 * (size_t)blockIdx.x;
			slot[0] = clock_in;
			slot[1] = clock_out;
			slot[2] = ticks_in;
			slot[3] = ticks_out;
		}
	}
	float4_t acc[8][8];
	const float32x_t* rows[8] = {&r0, &r1, &r2, &r3, &r4, &r5, &r6, &r7};
#pragma unroll
	for (int i = 0; i < 8; ++i)
#pragma unroll
		for (int j = 0; j < 8; ++j)
			acc[i][j] = float4_t{(*rows[i])[4 * j], (*rows[i])[4 * j + 1], (*rows[i])[4 * j + 2], (*rows[i])[4 * j + 3]};
	store_patch_via_lds<Cfg, RAGGED, !RAGGED, EPI>(acc, lds, C, ldc, m0 + wm * 128, n0 + wn * (DUAL ? 64 : 128), wave, lane_after, M, N, bias, ep_param);
}

// What the kernel assumes, checked on the host before every launch: whole slabs, 16-byte aligned operand rows, and
// operands small enough for the 32-bit lane offsets (a wave's 64 rows).
inline bool gemm_f16_ring_applies(const half_t* A, const half_t* B, int64_t M, int64_t N, int64_t K,
                                  int64_t lda, int64_t ldb, int64_t stride_a, int64_t stride_b, int64_t batch,
                                  int b_layout = ANYGPU_B_COL_MAJOR)
{
	if (b_layout == ANYGPU_B_ROW_MAJOR && N % 8 != 0) return false;
	const bool aligned = reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(B) % 16 == 0 &&
	                     lda % 8 == 0 && ldb % 8 == 0 && stride_a % 8 == 0 && stride_b % 8 == 0;
	return aligned && M > 0 && N > 0 && K >= 64 && K % 64 == 0 && lda < (1 << 24) && ldb < (1 << 24) &&
	       ((M + 255) / 256) * ((N + 255) / 256) <= 0x7FFFFFFFLL && batch >= 1 && batch <= 65535;
}

template <int EPI = kEpiNone>
inline hipError_t launch_gemm_f16_ring(const half_t* A, const half_t* B, half_t* C, int64_t M, int64_t N, int64_t K,
                                       int64_t lda, int64_t ldb, int64_t ldc,
                                       int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch, hipStream_t stream,
                                       unsigned long long* probe = nullptr, int b_layout = ANYGPU_B_COL_MAJOR,
                                       const half_t* bias = nullptr, float ep_param = 0.0f)
{
	const bool kn = b_layout == ANYGPU_B_ROW_MAJOR;
	// (whole tiles of an aligned C are streamed out in 16-byte vectors; anything else takes the guarded stores)
	const bool c_aligned = reinterpret_cast<uintptr_t>(C) % 16 == 0 && ldc % 8 == 0 && stride_c % 8 == 0;
	constexpr int kOutN = EPI == kEpiGeluMul ? 128 : 256;             // output columns of a tile
	const int ragged = (M % 256 != 0 || N % kOutN != 0 || !c_aligned) + 2 * kn;       // which instantiation
	auto kernel = (ragged & 1) == 0 ? gemm_f16_nt_ring_kernel<false, false, EPI> : gemm_f16_nt_ring_kernel<true, false, EPI>;
	if constexpr (EPI != kEpiGeluMul)
	{
		if (ragged == 2) kernel = gemm_f16_nt_ring_kernel<false, true, EPI>;
		if (ragged == 3) kernel = gemm_f16_nt_ring_kernel<true, true, EPI>;
	}
	else if (kn) return hipErrorInvalidValue;
	// More than 64 KB of dynamic LDS has to be granted per function and per device, once.
	static std::atomic<uint64_t> configured_devices[4];
	(void)hipGetLastError();
	int device = 0;
	hipError_t e = hipGetDevice(&device);
	if (e != hipSuccess) return e;
	const uint64_t bit = 1ull << (device & 63);
	if ((configured_devices[ragged].load(std::memory_order_relaxed) & bit) == 0)
	{
		e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, GemmRingCfg::kLdsBytes);
		if (e != hipSuccess) return e;
		configured_devices[ragged].fetch_or(bit, std::memory_order_relaxed);
	}
	const int tiles_m = (int)((M + 255) / 256), tiles_n = (int)((N + kOutN - 1) / kOutN);
	kernel<<<dim3((unsigned)(tiles_m * tiles_n), (unsigned)batch), dim3(256), GemmRingCfg::kLdsBytes, stream>>>(
		A, B, C, (int)K, lda, ldb, ldc, tiles_m, tiles_n, stride_a, stride_b, stride_c, probe, M, N, bias, ep_param);
	return hipGetLastError();
}

}  // namespace anygpu
