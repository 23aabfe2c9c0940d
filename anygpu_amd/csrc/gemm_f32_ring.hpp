// 128 x 128 and 64 x 64 tiles of the fp32 GEMM (A [M, K] and B [N, K], both k-contiguous) for whole 32-deep slabs: four
// waves, a 64 x 64 patch each as 2 x 2 tiles of v_mfma_f32_32x32x2_f32 (or a 32 x 32 patch as one tile), operands straight
// from global memory into three LDS stages, one barrier per slab.  The main loop is one block of assembly with fixed
// registers (gemm_f32_ring_loop.inc, gemm_f32_ring_loop_64.inc, written by gen_gemm_f32_ring_loop.py, which describes the
// register plan, the stages and the schedule).  The small tile is for products that do not fill the chip with big ones:
// an fp32 MFMA is slow enough that a quarter of the operand reuse still keeps the matrix cores fed.
#pragma once

#include <atomic>

#include "anygpu_hip.h"
#include "device_utils.hpp"
#include "gemm_epilogue.hpp"
#include "tile_walk.hpp"

namespace anygpu {

typedef float float32x_f32_t __attribute__((ext_vector_type(32)));

// T: MFMA tiles per wave and direction; the tile is 64 T x 64 T
template <int T>
struct GemmF32RingCfg
{
	static_assert(T == 1 || T == 2, "the loops that are generated");
	static constexpr int BM = 64 * T, BN = 64 * T, BK = 32;
	static constexpr int kStageBytes = (BM + BN) * 128;          // 128-byte rows: 32 floats
	static constexpr int kTableBytes = 4 * 16 * 64 * 4;          // per wave 16 load offsets per lane
	static constexpr int kLdsBytes = 3 * kStageBytes + kTableBytes;
	static constexpr int kLoads = 2 * T;                         // per wave, operand and slab: 8 rows of 128 bytes each
};

// blockIdx.y walks a batch of independent products that share the shape, or (k_split > 0) ranges of K of one product:
// the strides then step along K and C is the range's [M, N] plane of partial sums.  K (and k_split) multiples of 32,
// operand rows 16-byte aligned.  RAGGED: M and N need not be multiples of 128 and C may start and step at any element;
// operand rows past the end are read from the last valid row (they only feed results that are not stored), the stores
// are guarded.  EPI: kEpiBias (+ bias[n] when bias != NULL) or kEpiSoftcap, applied to the sums; or kEpiGeluMul (big tile,
// k-contiguous weights): the tile is 64 output columns wide (N counts those) and its B unit is put together from two
// matrices, of every wave column's 64 unit rows the first 32 from B (the gate weights) and the second 32 from `bias`,
// which then is the second matrix (the up weights, same pitch), both for the same 32 output columns: MFMA tile column 0
// of a wave holds the gate sums and column 1 the up sums of the same outputs, gelu_tanh(gate) * up goes out.  The wave
// that loads a quarter of the unit loads it from one matrix.
// B_KN: B stored [K, N] (N a multiple of 4): a B unit of 32 k rows x BN n, the chunks of rows 16 .. 31 stored with bit 3
// of their index flipped; a lane fetches its k one float at a time down its column.
template <int T, bool RAGGED, int EPI, bool B_KN = false>
__global__ __launch_bounds__(256) void gemm_f32_nt_ring_kernel(
	const float* __restrict__ A, const float* __restrict__ B, const float* __restrict__ bias, float* __restrict__ C,
	int64_t M, int64_t N, int K, int64_t lda, int64_t ldb, int64_t ldc,
	int64_t stride_a, int64_t stride_b, int64_t stride_c, float ep_param, int k_split, int operands_padded)
{
	using Cfg = GemmF32RingCfg<T>;
	constexpr bool DUAL = EPI == kEpiGeluMul;
	static_assert(!DUAL || (T == 2 && !B_KN), "two weight matrices: the big tile, k-contiguous");
	extern __shared__ __align__(1024) char lds[];
	if (k_split > 0)
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
	constexpr int kOutN = DUAL ? Cfg::BN / 2 : Cfg::BN;           // output columns of a tile
	tile_of_block<8>(blockIdx.x, (int)((M + Cfg::BM - 1) / Cfg::BM), (int)((N + kOutN - 1) / kOutN), tile_m, tile_n);
	const int64_t m0 = (int64_t)tile_m * Cfg::BM, n0 = (int64_t)tile_n * kOutN;
	// DUAL: the unit rows wave w loads are output columns 32 (w / 2) .. of the tile, from B (w even) or the second matrix
	const float* const b_of_wave = DUAL && (wave & 1) ? bias : B;
	const int b_unit_row = DUAL ? 8 * Cfg::kLoads * (wave >> 1) : 8 * Cfg::kLoads * wave;

	// Direct loads.  A unit row is 32 floats = eight 16-byte chunks; chunk c of row r sits at position c ^ ((r >> 1) & 7).
	// One instruction fills 8 rows: lane -> row lane / 8, position lane % 8; instruction q of this wave covers rows
	// 8 (kLoads wave + q) .. + 7 of the unit.  The lane's byte offsets from the wave's first row go to the assembly block
	// through a table behind the stages: table[q][lane], q < 4 for A, 8 + q for B.
	const unsigned lds0 = (unsigned)(uintptr_t)(const __attribute__((address_space(3))) char*)lds;
	const int ld_row = lane >> 3, ld_pos = lane & 7;
	unsigned* const table = reinterpret_cast<unsigned*>(lds + 3 * Cfg::kStageBytes) + wave * (16 * 64) + lane;
	int64_t a_first = m0 + 8 * Cfg::kLoads * wave, b_first = n0 + b_unit_row;
	// (operands_padded: the operands are copies that reach, filled with zeros, to the end of the last tile in every
	// direction; nothing to clamp then, and N need not be a multiple of 4 for B stored [K, N])
	const bool clamp = RAGGED && operands_padded == 0;
	if (clamp)
	{
		a_first = a_first < M - 1 ? a_first : M - 1;
		b_first = b_first < N - 1 ? b_first : N - 1;
	}
#pragma unroll
	for (int q = 0; q < Cfg::kLoads; ++q)
	{
		const int row = 8 * (Cfg::kLoads * wave + q) + ld_row;
		const unsigned chunk = ld_pos ^ ((row >> 1) & 7);
		int64_t a_row = m0 + row, b_row = n0 + b_unit_row + 8 * q + ld_row;
		if (clamp)
		{
			a_row = a_row < M - 1 ? a_row : M - 1;
			b_row = b_row < N - 1 ? b_row : N - 1;
		}
		table[64 * q] = (unsigned)(((a_row - a_first) * lda + chunk * 4) * 4);
		if constexpr (B_KN)
		{
			// one instruction fills 1024 / (4 BN) k rows: lane -> row lane / (BN / 4), position lane % (BN / 4); the wave's
			// instructions cover rows 8 wave .. 8 wave + 7 of the slab's 32
			constexpr int kLanesPerRow = Cfg::BN / 4, kRowsPerLoad = 64 / kLanesPerRow;
			const int k_wave = kRowsPerLoad * q + lane / kLanesPerRow;
			const int k = 8 * wave + k_wave;
			int64_t col = (int64_t)(((lane % kLanesPerRow) ^ (((k >> 4) & 1) << 3)) << 2);
			if (clamp && n0 + col + 4 > N) col = N - 4 - n0;
			table[64 * (8 + q)] = (unsigned)((k_wave * ldb + col) * 4);
		}
		else
			table[64 * (8 + q)] = (unsigned)(((b_row - b_first) * ldb + chunk * 4) * 4);
	}
	const unsigned table_addr = lds0 + 3 * Cfg::kStageBytes + (wave * (16 * 64) + lane) * 4;
	const uintptr_t a_wave = reinterpret_cast<uintptr_t>(A + a_first * lda);
	const uintptr_t b_wave = reinterpret_cast<uintptr_t>(B_KN ? B + (int64_t)(8 * wave) * ldb + n0 : b_of_wave + b_first * ldb);
	const unsigned share_a = wave * (Cfg::kLoads * 1024);
	const unsigned share_b = Cfg::BM * 128 + wave * (Cfg::kLoads * 1024);
	const int slabs = K / 32;

	// Fragments: lane -> row lane % 32 of its MFMA tile, half lane / 32: k = 16 half .. + 15 of the slab, i.e. chunks
	// 4 half .. + 3, two per 16-deep step; the assembly block derives the four addresses from the first by XOR.
	const unsigned frag_row = lane & 31;
	const unsigned first_pos = (4 * (lane >> 5)) ^ ((frag_row >> 1) & 7);
	const unsigned a_addr = (wm * 32 * T + frag_row) * 128 + first_pos * 16;
	// B stored [K, N]: the lane's column n = wn 32 T + 32 j + frag_row of the tile, its first k row 16 half; chunk index
	// bit 3 (byte bit 7) is j (T = 2) or wn (T = 1), flipped for the upper half of the lanes
	const unsigned half = lane >> 5;
	const unsigned b_addr = B_KN ? Cfg::BM * 128 + 16 * half * (Cfg::BN * 4) + (T == 2 ? wn * 256 : 0) + (frag_row >> 2) * 16 + (frag_row & 3) * 4
	                             : Cfg::BM * 128 + (wn * 32 * T + frag_row) * 128 + first_pos * 16;
	[[maybe_unused]] const unsigned b_flip = (T == 2 ? half : (half ^ (unsigned)wn)) << 7;
	[[maybe_unused]] const unsigned b_step = (unsigned)(128 * ldb);        // bytes from one [K, N] slab (32 rows) to the next

	// The accumulators leave the block as vectors pinned to a[0 : 16 T T): MFMA tile (i, j) in registers 16 (T i + j) .. + 15.
	float32x_f32_t r0 = {}, r1 = {};
	float16_t single = {};
#define ANYGPU_F32_RING_INPUTS \
	[vtab] "v"(table_addr), [aaddr] "v"(a_addr), [baddr] "v"(b_addr), \
	[abaselo] "s"((unsigned)a_wave), [abasehi] "s"((unsigned)(a_wave >> 32)), \
	[bbaselo] "s"((unsigned)b_wave), [bbasehi] "s"((unsigned)(b_wave >> 32)), \
	[lds0] "s"(lds0), [ldsa] "s"(share_a), [ldsb] "s"(share_b), [slabs] "s"(slabs)
#define ANYGPU_F32_RING_CLOBBERS \
		  "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109", \
		  "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123", \
		  "v124", "v125", "v126", "v127", "v128", "v129", "v130", "v131", "v132", "v133", "v134", "v135", "v136", "v137", \
		  "v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", "v147", "v148", "v149", "v150", "v151", \
		  "v152", "v153", "v154", "v155", "v156", "v157", "v158", "v159", "v160", "v161", "v162", "v163", "v164", "v165", \
		  "v166", "v167", "v168", "v169", "v170", "v171", "v172", "v173", "v174", "v175", "v176", "v177", "v178", "v179", \
		  "v180", "v181", "v182", "v183", "v184", "v185", "v186", "v187", "v188", "v189", "v190", "v191", \
		  "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", "s72", "s73", "s74", "scc", "m0", "memory"
	if constexpr (T == 2 && B_KN)
		asm volatile(
#include "gemm_f32_ring_loop_kn.inc"
			: "={a[0:31]}"(r0), "={a[32:63]}"(r1)
			: ANYGPU_F32_RING_INPUTS, [bsx] "v"(b_flip), [bstep] "s"(b_step)
			: ANYGPU_F32_RING_CLOBBERS);
	else if constexpr (B_KN)
		asm volatile(
#include "gemm_f32_ring_loop_64kn.inc"
			: "={a[0:15]}"(single)
			: ANYGPU_F32_RING_INPUTS, [bsx] "v"(b_flip), [bstep] "s"(b_step)
			: ANYGPU_F32_RING_CLOBBERS);
	else if constexpr (T == 2)
		asm volatile(
#include "gemm_f32_ring_loop.inc"
			: "={a[0:31]}"(r0), "={a[32:63]}"(r1)
			: ANYGPU_F32_RING_INPUTS
			: ANYGPU_F32_RING_CLOBBERS);
	else
		asm volatile(
#include "gemm_f32_ring_loop_64.inc"
			: "={a[0:15]}"(single)
			: ANYGPU_F32_RING_INPUTS
			: ANYGPU_F32_RING_CLOBBERS);
#undef ANYGPU_F32_RING_INPUTS
#undef ANYGPU_F32_RING_CLOBBERS

	// register r of lane l of a tile: C[m = l % 32][n = 8 (r / 4) + 4 (l / 32) + r % 4] of the 32 x 32 tile
	const unsigned misalign = RAGGED ? (unsigned)((reinterpret_cast<uintptr_t>(C) | (uintptr_t)(ldc * 4)) & 15) : 0u;
#pragma unroll
	for (int i = 0; i < T; ++i)
	{
		const int64_t m = m0 + wm * 32 * T + i * 32 + frag_row;
#pragma unroll
		for (int j = 0; j < (DUAL ? 1 : T); ++j)
		{
			const float32x_f32_t& v = i == 0 ? r0 : r1;
#pragma unroll
			for (int g = 0; g < 4; ++g)
			{
				const int64_t n = n0 + wn * (DUAL ? 32 : 32 * T) + j * 32 + 8 * g + 4 * (lane >> 5);
				float4_t out;
#pragma unroll
				for (int e = 0; e < 4; ++e)
				{
					if constexpr (DUAL) out[e] = finish_sum<EPI>(v[4 * g + e], v[16 + 4 * g + e], 0.0f, ep_param);
					else
					{
						const float bias_n = (EPI == kEpiBias && bias != nullptr && (!RAGGED || n + e < N)) ? bias[n + e] : 0.0f;
						out[e] = finish_sum<EPI>(T == 2 ? v[16 * j + 4 * g + e] : single[4 * g + e], 0.0f, bias_n, ep_param);
					}
				}
				if (!RAGGED || (m < M && n + 4 <= N))
				{
					typedef float4_t LooseVec __attribute__((aligned(4)));
					if (misalign == 0) *reinterpret_cast<float4_t*>(C + m * ldc + n) = out;
					else *reinterpret_cast<LooseVec*>(C + m * ldc + n) = out;
				}
				else if (m < M)
				{
#pragma unroll
					for (int e = 0; e < 4; ++e)
						if (n + e < N) C[m * ldc + n + e] = out[e];
				}
			}
		}
	}
}

// What the kernel assumes, checked on the host before every launch.
inline bool gemm_f32_ring_applies(const float* A, const float* B, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                  int64_t stride_a, int64_t stride_b, int64_t batch, int64_t k_split, int64_t tile = 128,
                                  int b_layout = ANYGPU_B_COL_MAJOR, bool operands_padded = false)
{
	if (b_layout == ANYGPU_B_ROW_MAJOR && N % 4 != 0 && !operands_padded) return false;
	const bool aligned = reinterpret_cast<uintptr_t>(A) % 16 == 0 && reinterpret_cast<uintptr_t>(B) % 16 == 0 &&
	                     lda % 4 == 0 && ldb % 4 == 0 && stride_a % 4 == 0 && stride_b % 4 == 0;
	return aligned && M > 0 && N > 0 && K >= 32 && K % 32 == 0 && k_split % 32 == 0 && K <= 0x7FFFFFFFLL &&
	       lda < (1 << 24) && ldb < (1 << 24) && ((M + tile - 1) / tile) * ((N + tile - 1) / tile) <= 0x7FFFFFFFLL && batch >= 1 && batch <= 65535;
}

template <int T, int EPI, bool B_KN = false>
inline hipError_t launch_gemm_f32_ring(const float* A, const float* B, const float* bias, float* C, int64_t M, int64_t N, int64_t K,
                                       int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                                       int64_t batch, float ep_param, int64_t k_split, hipStream_t stream, bool operands_padded = false)
{
	const bool c_aligned = reinterpret_cast<uintptr_t>(C) % 16 == 0 && ldc % 4 == 0 && stride_c % 4 == 0;
	using Cfg = GemmF32RingCfg<T>;
	constexpr int kOutN = EPI == kEpiGeluMul ? Cfg::BN / 2 : Cfg::BN;
	const bool ragged = M % Cfg::BM != 0 || N % kOutN != 0 || !c_aligned;
	auto kernel = ragged ? gemm_f32_nt_ring_kernel<T, true, EPI, B_KN> : gemm_f32_nt_ring_kernel<T, false, EPI, B_KN>;
	// More than 64 KB of dynamic LDS has to be granted per function and per device, once.
	static std::atomic<uint64_t> configured_devices[2];
	(void)hipGetLastError();
	int device = 0;
	hipError_t e = hipGetDevice(&device);
	if (e != hipSuccess) return e;
	const uint64_t bit = 1ull << (device & 63);
	if ((configured_devices[ragged].load(std::memory_order_relaxed) & bit) == 0)
	{
		e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::kLdsBytes);
		if (e != hipSuccess) return e;
		configured_devices[ragged].fetch_or(bit, std::memory_order_relaxed);
	}
	const int64_t tiles = ((M + Cfg::BM - 1) / Cfg::BM) * ((N + kOutN - 1) / kOutN);
	kernel<<<dim3((unsigned)tiles, (unsigned)batch), dim3(256), Cfg::kLdsBytes, stream>>>(
		A, B, bias, C, M, N, (int)K, lda, ldb, ldc, stride_a, stride_b, stride_c, ep_param, (int)k_split, operands_padded ? 1 : 0);
	return hipGetLastError();
}

}  // namespace anygpu
