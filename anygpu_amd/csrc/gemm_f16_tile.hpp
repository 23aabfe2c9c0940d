// Tile kernel of the fp16 GEMM ("NT": A [M,K] and B [N,K], both K-contiguous) for gfx950.
//
// A block owns a BM x BN tile of C.  Per 64-deep step it stages a BM x 64 slab of A and a
// BN x 64 slab of B in LDS (two stages, so the loads of slab t+1 are in flight while slab t
// is multiplied) and each wave accumulates a (BM/WM) x (BN/WN) patch on the matrix cores with
// fp32 accumulators, either with v_mfma_f32_32x32x16_f16 or with v_mfma_f32_16x16x32_f16
// (both take 8 halves per lane per operand and have the same peak rate).
//
// Global -> LDS goes through global_load_lds_dwordx4: every lane fetches 16 bytes and the
// hardware writes the 64 lanes of a wave to 1 KB of consecutive LDS, bypassing the VGPRs.
// An LDS slab row is 64 halves = 128 bytes = eight 16-byte chunks; chunk c of row r is stored
// at chunk position c ^ swz(r), so that the lanes which read the same logical chunk of
// consecutive rows for an MFMA operand (ds_read_b128) spread over all banks.  Because the
// LDS side of the direct load is fixed (lane i -> base + 16 i), the swizzle is applied on the
// global side: lane i of a load instruction fetches the chunk that belongs at position i.
//
// The products are formed transposed (the B slab is the first MFMA operand), which leaves
// every lane with 4 consecutive columns of one row of C; the epilogue parks row bands of the
// wave's patch in LDS and writes whole rows back, 16 bytes per lane.
//
// Under this kernel the MI355X is power-limited, not issue-limited: measured with
// s_memtime / s_memrealtime inside the main loop, the shader clock sits near 1.6 GHz (not 2.4)
// and schedules with fewer MFMA stalls simply run at a lower clock for the same wall time.
#pragma once

#include "device_utils.hpp"
#include "gemm_epilogue.hpp"

#include <atomic>
#include <type_traits>

#include "tile_walk.hpp"

namespace anygpu {

// SWZ selects which row bits permute the chunk position: 0 -> row & 7 (conflict free for 8
// lanes per LDS pass over 32 banks), 1 -> (row >> 1) & 7 (conflict free for 16 lanes per pass
// over 64 banks; measured conflict free on gfx950 with SQ_LDS_BANK_CONFLICT).
template <int SWZ>
__device__ __forceinline__ int swizzle_of_row(int row)
{
	return SWZ == 0 ? (row & 7) : ((row >> 1) & 7);
}

// The two MFMA shapes.  MI x MI output tile; a lane supplies row (lane % MI) of each operand
// and k group (lane / MI), 8 consecutive halves; one instruction is 512 / MI deep.
template <int MI> struct MfmaShape;

template <> struct MfmaShape<32>
{
	using Acc = float16_t;
	static constexpr int kAccRegs = 16;
	__device__ static __forceinline__ Acc mma(half8_t first, half8_t second, Acc c)
	{
		return __builtin_amdgcn_mfma_f32_32x32x16_f16(first, second, c, 0, 0, 0);
	}
	// register group g (4 registers) of lane l: row l % 32 of the second operand, 4 consecutive
	// rows of the first operand starting at:
	__device__ static __forceinline__ int first_row_of_group(int g, int lane) { return 8 * g + 4 * (lane >> 5); }
};

template <> struct MfmaShape<16>
{
	using Acc = float4_t;
	static constexpr int kAccRegs = 4;
	__device__ static __forceinline__ Acc mma(half8_t first, half8_t second, Acc c)
	{
		return __builtin_amdgcn_mfma_f32_16x16x32_f16(first, second, c, 0, 0, 0);
	}
	__device__ static __forceinline__ int first_row_of_group(int g, int lane) { (void)g; return 4 * (lane >> 4); }
};

template <int BM_, int BN_, int WM_, int WN_, int SWZ_, int ILV_ = 0, int GROUP_M_ = 4, int MI_ = 32, bool B_KN_ = false, int STAGES_ = 2, int KGROUPS_ = 1>
struct GemmTileCfg
{
	// B_KN = false: B stored [N, K] (k-contiguous, like A).  true: B stored [K, N] (the reference
	// layout): its slab is staged as [64 k][BN n] rows and the k-contiguous MFMA operand is formed by
	// the transposing LDS read ds_read_b64_tr_b16.
	static constexpr bool B_KN = B_KN_;
	static_assert(!B_KN_ || MI_ == 16, "the transposed-B path is written for the 16 x 16 x 32 MFMA");
	static constexpr int BM = BM_, BN = BN_, BK = 64, WM = WM_, WN = WN_, SWZ = SWZ_;
	static constexpr int ILV = ILV_;          // how LDS reads are spread between the MFMAs of one step
	static constexpr int GROUP_M = GROUP_M_;  // rows of tiles per column strip of the tile walk
	static constexpr int MI = MI_;            // MFMA tile edge: 32 (x16 deep) or 16 (x32 deep)
	static constexpr int kKGroups = kWaveSize / MI;       // k groups of 8 halves per instruction
	static constexpr int kSteps = 8 / kKGroups;           // MFMA steps per 64-deep slab
	// KGROUPS = 2: two groups of WM x WN waves share the tile; group g multiplies step g of the two 32-deep steps of
	// every slab and the groups' accumulators are added through LDS at the end.  Half the tile area of the plain form
	// with the same number of waves, the same wave patch and the same LDS bytes per MFMA.
	static constexpr int kKGroupsOfWaves = KGROUPS_;
	static_assert(KGROUPS_ == 1 || (KGROUPS_ == 2 && MI_ == 16 && STAGES_ == 2), "two k groups: one step of 32 each");
	static constexpr int kWaves = WM * WN * KGROUPS_;
	static constexpr int kThreads = kWaves * kWaveSize;
	static constexpr int kWaveM = BM / WM;
	static constexpr int kWaveN = BN / WN;
	static constexpr int kTilesM = kWaveM / MI;
	static constexpr int kTilesN = kWaveN / MI;
	static constexpr int kSlabABytes = BM * BK * 2;
	static constexpr int kSlabBBytes = BN * BK * 2;
	static constexpr int kStageBytes = kSlabABytes + kSlabBBytes;
	// LDS stages: slab t + STAGES - 1 is requested when slab t has been multiplied.  Two are enough where a slab takes
	// longer to multiply than to fetch (the big tiles); a 64 x 64 tile multiplies a slab in a tenth of the memory
	// latency and, alone on its CU, advanced one slab per latency with two stages.
	static constexpr int kStages = STAGES_;
	static_assert(STAGES_ >= 2, "double buffering at least");
	static constexpr int kLdsBytes = kStages * kStageBytes;
	// one direct load instruction of a wave moves 1 KB = 8 slab rows
	static constexpr int kLoadsA = BM / 8 / kWaves;
	static constexpr int kLoadsB = BN / 8 / kWaves;
	static_assert(MI == 32 || MI == 16, "unknown MFMA shape");
	static_assert(BM % (8 * kWaves) == 0 && BN % (8 * kWaves) == 0, "slab rows must divide over the waves");
	static_assert(kWaveM % MI == 0 && kWaveN % MI == 0, "wave patch must be whole MFMA tiles");
};

// vmcnt(0) with the other counters left alone (gfx9 encoding: vmcnt in [3:0] and [15:14],
// expcnt [6:4], lgkmcnt [11:8])
// global_load_lds_dwordx4 with the LDS base of the wave-wide 1 KB destination in M0 (wave-uniform)
__device__ __forceinline__ void direct_load_asm(const void* src, const char* lds_dst)
{
	const unsigned m0 = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)(const __attribute__((address_space(3))) char*)lds_dst);
	asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(m0) : "m0");
}

__device__ __forceinline__ void wait_vmem_all()
{
	__builtin_amdgcn_s_waitcnt(0x0F70);
}

// vmcnt(N): all but the N most recent vector memory operations of the wave have completed
template <int N>
__device__ __forceinline__ void wait_vmem_but()
{
	static_assert(N >= 0 && N < 64, "vmcnt has 6 bits");
	__builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// Swizzle of a [k][n] slab row (B stored [K, N]): 16-byte chunks move in pairs (a transposing read
// takes 32 contiguous bytes of a row), pair index ^ s(k).  The 16 lanes of a transposing read cover
// 4 consecutive k, the four lane groups of a wave sit 8 k apart: s(k) = (k & 3) | ((k >> 3) & 1) << 2
// gives the 8 rows that 32 lanes read together 8 different 32-byte bank slots.
__device__ __forceinline__ int kn_row_swizzle(int k)
{
	return 2 * ((k & 3) | (((k >> 3) & 1) << 2));
}

typedef short short4_t __attribute__((ext_vector_type(4)));

// ds_read_b64_tr_b16: within each group of 16 lanes, lane i receives element (i % 4) of the
// 4-element rows addressed by lanes i / 4, i / 4 + 4, i / 4 + 8, i / 4 + 12 of the group
// (lane mapping measured on gfx950).  With lane r of a group pointing at B[k0 + r / 4][n0 + 4 (r % 4) ...],
// lane i ends up with B[k0 .. k0 + 3][n0 + i]: four consecutive k of one column.
__device__ __forceinline__ half4_t lds_read_transposed_b64(const char* lds_addr)
{
	const short4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
		(__attribute__((address_space(3))) short4_t*)(lds_addr));
	return __builtin_bit_cast(half4_t, v);
}

// Epilogue through LDS.  With the B slab as the first MFMA operand, a group of 4 accumulator
// registers of a lane holds 4 consecutive columns of ONE row of C (row = lane % MI of the tile),
// so a direct store instruction would touch MI different rows with 8 bytes each.  Instead each
// wave parks one MI-row band of its patch (MI x kWaveN halves) in its own LDS scratch and reads
// it back row by row, 16 bytes per lane, so that the global stores cover whole rows of the band.
// The scratch row pitch is 16 bytes more than the row, which spreads the 8-byte writes of the
// rows over the banks.  The caller guarantees that nobody still reads or fills LDS.
// RAGGED: rows at or beyond M and columns at or beyond N are not stored (the 8-column chunk that crosses N goes out
// element by element).  Stores are made at element alignment: rows of C may start anywhere.
// STREAM: the whole vectors are stored with the non-temporal hint (C is 16-byte aligned then).  A launch that writes tens
// of megabytes otherwise ends with all of C dirty in the L2s and pays for the write-back when the kernel retires
// (4096^3: 93.5 -> 92.4 us); the same bytes written without the LDS pass, 64 contiguous bytes per row and instruction
// after a v_permlane16_swap between neighbouring tiles, were 1.5 us slower than whole rows through LDS.
typedef half8_t LooseHalf8Store __attribute__((aligned(2)));
typedef half4_t LooseHalf4Store __attribute__((aligned(8)));
typedef half2_t LooseHalf2Store __attribute__((aligned(4)));

// Eight halves to an address that is a multiple of 16 bytes plus `misalign` (the same for every store of a launch: rows
// of C start where its base and its pitch put them): in the widest pieces that alignment allows.
__device__ __forceinline__ void store_half8_at_alignment(half_t* dst, const half8_t& v, unsigned misalign)
{
	if (misalign == 0) *reinterpret_cast<half8_t*>(dst) = v;
	else if ((misalign & 7) == 0)
	{
		reinterpret_cast<LooseHalf4Store*>(dst)[0] = half4_t{v[0], v[1], v[2], v[3]};
		reinterpret_cast<LooseHalf4Store*>(dst)[1] = half4_t{v[4], v[5], v[6], v[7]};
	}
	else if ((misalign & 3) == 0)
	{
#pragma unroll
		for (int e = 0; e < 4; ++e) reinterpret_cast<LooseHalf2Store*>(dst)[e] = half2_t{v[2 * e], v[2 * e + 1]};
	}
	else *reinterpret_cast<LooseHalf8Store*>(dst) = v;
}

// EPI: what happens to a sum on its way out (gemm_epilogue.hpp).  kEpiBias adds bias[n] (fp16), kEpiSoftcap
// caps, and with kEpiGeluMul the patch holds two products side by side: MFMA column tiles 0 .. TN / 2 - 1 are A x B_gate
// and TN / 2 .. TN - 1 are A x B_up for the same kWaveN / 2 output columns (the kernel staged the B slab that way), and
// gelu_tanh(gate) * up goes out; n_base and N then count output columns.
constexpr int kEpiNone = -1;      // the sums go out as they are

template <typename Cfg, bool RAGGED, bool STREAM = false, int EPI = kEpiNone>
__device__ __forceinline__ void store_patch_via_lds(
	const typename MfmaShape<Cfg::MI>::Acc (&acc)[Cfg::kTilesM][Cfg::kTilesN], char* lds,
	half_t* __restrict__ C, int64_t ldc, int64_t m_base, int64_t n_base, int wave, int lane, int64_t M, int64_t N,
	const half_t* __restrict__ bias = nullptr, float ep_param = 0.0f)
{
	using Shape = MfmaShape<Cfg::MI>;
	constexpr int MI = Cfg::MI, TM = Cfg::kTilesM;
	constexpr int TN = EPI == kEpiGeluMul ? Cfg::kTilesN / 2 : Cfg::kTilesN;        // column tiles that are stored
	constexpr int kRowBytes = (EPI == kEpiGeluMul ? Cfg::kWaveN / 2 : Cfg::kWaveN) * 2;
	static_assert(EPI != kEpiGeluMul || Cfg::kTilesN % 2 == 0, "gate and up halves of the patch");
	constexpr int kPitch = kRowBytes + 16;
	constexpr int kLanesPerRow = kRowBytes / 16;
	constexpr int kRowsPerPass = kWaveSize / kLanesPerRow;
	static_assert(Cfg::kWaves * MI * kPitch <= Cfg::kLdsBytes, "epilogue scratch must fit in the staging LDS");
	char* scratch = lds + wave * (MI * kPitch);
	const int frag_row = lane % MI;
	// (n_base and the 8-column chunks are multiples of 16 bytes: a store is as aligned as C and its row pitch are)
	[[maybe_unused]] const unsigned misalign = (unsigned)((reinterpret_cast<uintptr_t>(C) | (uintptr_t)(ldc * 2)) & 15);
	// the bias of this lane's columns (the same for every row band)
	[[maybe_unused]] float bias_of[TN][Shape::kAccRegs / 4][4] = {};
	if constexpr (EPI == kEpiBias)
	{
#pragma unroll
		for (int j = 0; j < TN; ++j)
#pragma unroll
			for (int g = 0; g < Shape::kAccRegs / 4; ++g)
#pragma unroll
				for (int e = 0; e < 4; ++e)
				{
					const int64_t n = n_base + j * MI + Shape::first_row_of_group(g, lane) + e;
					bias_of[j][g][e] = (!RAGGED || n < N) ? (float)bias[n] : 0.0f;
				}
	}
#pragma unroll
	for (int i = 0; i < TM; ++i)
	{
#pragma unroll
		for (int j = 0; j < TN; ++j)
#pragma unroll
			for (int g = 0; g < Shape::kAccRegs / 4; ++g)
			{
				half4_t out;
#pragma unroll
				for (int e = 0; e < 4; ++e)
				{
					if constexpr (EPI == kEpiGeluMul)
						out[e] = (half_t)finish_sum<EPI, true>(acc[i][j][4 * g + e], acc[i][j + TN][4 * g + e], 0.0f, ep_param);
					else if constexpr (EPI == kEpiSoftcap)
						out[e] = (half_t)finish_sum<EPI, true>(acc[i][j][4 * g + e], 0.0f, 0.0f, ep_param);
					else if constexpr (EPI == kEpiBias)
						out[e] = (half_t)(acc[i][j][4 * g + e] + bias_of[j][g][e]);
					else
						out[e] = (half_t)acc[i][j][4 * g + e];
				}
				*reinterpret_cast<half4_t*>(scratch + frag_row * kPitch +
				                            (j * MI + Shape::first_row_of_group(g, lane)) * 2) = out;
			}
		constexpr int kPasses = (MI + kRowsPerPass - 1) / kRowsPerPass;
#pragma unroll
		for (int pass = 0; pass < kPasses; ++pass)
		{
			const int row = pass * kRowsPerPass + lane / kLanesPerRow;
			const int col16 = lane % kLanesPerRow;
			const bool inside = !RAGGED || (m_base + i * MI + row < M && n_base + col16 * 8 < N);
			if ((kRowsPerPass <= MI || row < MI) && inside)
			{
				const half8_t v = *reinterpret_cast<const half8_t*>(scratch + row * kPitch + col16 * 16);
				half_t* dst = C + (m_base + i * MI + row) * ldc + n_base + col16 * 8;
				if constexpr (STREAM && !RAGGED) __builtin_nontemporal_store(v, reinterpret_cast<half8_t*>(dst));
				else if (!RAGGED || n_base + col16 * 8 + 8 <= N) store_half8_at_alignment(dst, v, misalign);
				else
				{
#pragma unroll
					for (int e = 0; e < 8; ++e)
						if (n_base + col16 * 8 + e < N) dst[e] = v[e];
				}
			}
		}
	}
}

// The patch as raw fp32 sums into an [M, N] plane (ld = N, a multiple of 8): every lane stores its groups of four
// consecutive columns directly.  Rows at or beyond M and columns at or beyond N are not stored.
template <typename Cfg>
__device__ __forceinline__ void store_patch_f32(
	const typename MfmaShape<Cfg::MI>::Acc (&acc)[Cfg::kTilesM][Cfg::kTilesN],
	float* __restrict__ plane, int64_t m_base, int64_t n_base, int lane, int64_t M, int64_t N)
{
	using Shape = MfmaShape<Cfg::MI>;
	constexpr int MI = Cfg::MI;
#pragma unroll
	for (int i = 0; i < Cfg::kTilesM; ++i)
	{
		const int64_t m = m_base + i * MI + lane % MI;
#pragma unroll
		for (int j = 0; j < Cfg::kTilesN; ++j)
#pragma unroll
			for (int g = 0; g < Shape::kAccRegs / 4; ++g)
			{
				const int64_t n = n_base + j * MI + Shape::first_row_of_group(g, lane);
				if (m < M && n < N)
					*reinterpret_cast<float4_t*>(plane + m * N + n) =
						float4_t{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
			}
	}
}

// Scheduling-group masks of __builtin_amdgcn_sched_group_barrier
constexpr int kSchedMfma = 0x008;
constexpr int kSchedVmemRead = 0x020;
constexpr int kSchedDsRead = 0x100;

// The tile kernel, software pipelined.  Operand fragments are double-buffered in registers:
// while the MFMAs of one step run, the ds_read_b128 of the next step are issued in between
// them.  The barrier of a 64-deep slab sits in front of its LAST step, whose fragments are in
// registers by then: behind it the loads of slab t+2 go out (the stage they overwrite is no
// longer read by anybody) and the first fragments of slab t+1 are fetched, all under the
// shadow of the MFMAs of the last step of slab t.
// RAGGED: M and N need not be multiples of the tile (N a multiple of 8).  Operand rows past the
// end are read from the last valid row instead (they only feed results that are not stored).
// KTAIL: K need not be a multiple of the 64-deep slab (K >= 64, a multiple of 8).  The slabs cover
// the multiple; the remaining K % 64 columns are multiplied after the loop from fragments that
// every lane loads straight from global memory in the MFMA operand layout, zeros past K.
// SPLIT: blockIdx.y walks ranges of K (k_split deep, the strides step along K) of one product instead of a batch,
// and the raw fp32 sums of range y go to planes[y][M][N]; C is not touched.
// EPI: the epilogue (see store_patch_via_lds).  With kEpiGeluMul the tile is BN / 2 output columns wide (N and tiles_n
// count those) and its B slab is put together from two matrices: of every wave's kWaveN slab rows the first half comes
// from B (the gate weights) and the second half from B2 (the up weights), both for the same kWaveN / 2 output columns,
// so gate and up sums of an output element meet in one lane and A is read once for both products.
template <typename Cfg, bool RAGGED = false, bool KTAIL = false, bool SPLIT = false, int EPI = kEpiNone>
__global__ __launch_bounds__(Cfg::kThreads) void gemm_f16_nt_tile_kernel(
	const half_t* __restrict__ A, const half_t* __restrict__ B, half_t* __restrict__ C,
	int K, int64_t lda, int64_t ldb, int64_t ldc, int tiles_m, int tiles_n,
	int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t M, int64_t N,
	float* __restrict__ planes, int k_split,
	const half_t* __restrict__ B2 = nullptr, const half_t* __restrict__ bias = nullptr, float ep_param = 0.0f)
{
	using Shape = MfmaShape<Cfg::MI>;
	constexpr bool DUAL = EPI == kEpiGeluMul;
	static_assert(EPI == kEpiNone || (!SPLIT && Cfg::kKGroupsOfWaves == 1), "epilogues: the plain tile, uncut");
	constexpr int kOutN = DUAL ? Cfg::BN / 2 : Cfg::BN;           // output columns of a tile
	constexpr int kHalfWaveN = Cfg::kWaveN / 2;
	// DUAL: slab row (or column, for [K, N] weights) c of the tile -> which matrix, which output column of the tile
	const auto dual_col = [](int c, bool& second) {
		const int group = c / kHalfWaveN;
		second = (group & 1) != 0;
		return (group >> 1) * kHalfWaveN + c % kHalfWaveN;
	};
	if constexpr (SPLIT)
	{
		const int left = K - (int)blockIdx.y * k_split;
		K = left < k_split ? left : k_split;
	}
	// blockIdx.y walks a batch of independent products that share the shape
	A += (int64_t)blockIdx.y * stride_a;
	B += (int64_t)blockIdx.y * stride_b;
	C += (int64_t)blockIdx.y * stride_c;
	using Acc = typename Shape::Acc;
	constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, MI = Cfg::MI;
	constexpr int TM = Cfg::kTilesM, TN = Cfg::kTilesN;
	extern __shared__ __align__(1024) char lds[];
	typedef __attribute__((address_space(3))) void lds_void;
	typedef const __attribute__((address_space(1))) void global_void;

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: LDS targets of direct loads stay in SGPRs
	const int wk = wave / (Cfg::WM * Cfg::WN);                   // k group (0 unless the tile has two)
	const int wave_in_group = wave % (Cfg::WM * Cfg::WN);
	const int wm = wave_in_group / Cfg::WN;
	const int wn = wave_in_group % Cfg::WN;

	int tile_m, tile_n;
	tile_of_block<Cfg::GROUP_M>(blockIdx.x, tiles_m, tiles_n, tile_m, tile_n);
	const int64_t m0 = (int64_t)tile_m * BM;
	const int64_t n0 = (int64_t)tile_n * kOutN;

	// Direct loads.  Load instruction i of this wave fills slab rows [8 * (wave * kLoads + i), +8):
	// lane -> row offset lane / 8, chunk position lane % 8, i.e. logical chunk (lane % 8) ^ swz(row).
	const int ld_row = lane >> 3;
	const int ld_pos = lane & 7;
	const half_t* a_src[Cfg::kLoadsA];
	const half_t* b_src[Cfg::kLoadsB];
#pragma unroll
	for (int i = 0; i < Cfg::kLoadsA; ++i)
	{
		const int row = 8 * (wave * Cfg::kLoadsA + i) + ld_row;
		int64_t grow = m0 + row;
		if (RAGGED && grow > M - 1) grow = M - 1;
		a_src[i] = A + grow * lda + ((ld_pos ^ swizzle_of_row<Cfg::SWZ>(row)) << 3);
	}
	constexpr int kRowBytesKN = BN * 2;                 // [k][n] slab row
	constexpr int kRowsPerLoadKN = 1024 / kRowBytesKN;  // k rows one direct load instruction fills
	constexpr int kChunkMaskKN = BN / 8 - 1;            // narrow slabs have fewer chunk pairs to permute
#pragma unroll
	for (int i = 0; i < Cfg::kLoadsB; ++i)
	{
		if constexpr (Cfg::B_KN)
		{
			const int lanes_per_row = kWaveSize / kRowsPerLoadKN;
			const int k = kRowsPerLoadKN * (wave * Cfg::kLoadsB + i) + lane / lanes_per_row;
			const int pos = lane % lanes_per_row;
			int col = (pos ^ (kn_row_swizzle(k) & kChunkMaskKN)) << 3;
			bool second = false;
			if constexpr (DUAL) col = dual_col(col, second);
			int64_t gcol = n0 + col;
			if (RAGGED && gcol > N - 8) gcol = N - 8;
			b_src[i] = (second ? B2 : B) + (int64_t)k * ldb + gcol;
		}
		else
		{
			const int row = 8 * (wave * Cfg::kLoadsB + i) + ld_row;
			bool second = false;
			int64_t grow = n0 + (DUAL ? dual_col(row, second) : row);
			if (RAGGED && grow > N - 1) grow = N - 1;
			b_src[i] = (second ? B2 : B) + grow * ldb + ((ld_pos ^ swizzle_of_row<Cfg::SWZ>(row)) << 3);
		}
	}

	auto issue_loads = [&](int kt, int stage) {
		char* a_lds = lds + stage * Cfg::kStageBytes;
		char* b_lds = a_lds + Cfg::kSlabABytes;
		const int64_t koff = (int64_t)kt * BK;
		const int64_t koff_b = Cfg::B_KN ? koff * ldb : koff;
		if constexpr (Cfg::B_KN || Cfg::kStages > 2)
		{
			// Written as assembly for this layout: in front of a transposing LDS read the compiler waits for ALL of the
			// wave's outstanding direct loads (it cannot tell that they fill the other stage), which would put the
			// whole memory latency of the slab just requested in front of the first fragment read behind the barrier.
			// The waits these loads need are the explicit vmcnt in front of every slab barrier.  With more than two
			// stages the same holds for every layout: the compiler turns the vmcnt(n) that leaves the younger slabs in
			// flight into vmcnt(0) when it knows of direct loads.
#pragma unroll
			for (int i = 0; i < Cfg::kLoadsA; ++i)
				direct_load_asm(a_src[i] + koff, a_lds + 1024 * (wave * Cfg::kLoadsA + i));
#pragma unroll
			for (int i = 0; i < Cfg::kLoadsB; ++i)
				direct_load_asm(b_src[i] + koff_b, b_lds + 1024 * (wave * Cfg::kLoadsB + i));
		}
		else
		{
#pragma unroll
			for (int i = 0; i < Cfg::kLoadsA; ++i)
				__builtin_amdgcn_global_load_lds((global_void*)(a_src[i] + koff),
				                                 (lds_void*)(a_lds + 1024 * (wave * Cfg::kLoadsA + i)), 16, 0, 0);
#pragma unroll
			for (int i = 0; i < Cfg::kLoadsB; ++i)
				__builtin_amdgcn_global_load_lds((global_void*)(b_src[i] + koff_b),
				                                 (lds_void*)(b_lds + 1024 * (wave * Cfg::kLoadsB + i)), 16, 0, 0);
		}
	};

	Acc acc[TM][TN];
#pragma unroll
	for (int i = 0; i < TM; ++i)
#pragma unroll
		for (int j = 0; j < TN; ++j)
#pragma unroll
			for (int r = 0; r < Shape::kAccRegs; ++r) acc[i][j][r] = 0.0f;

	// operand fragments: lane -> slab row (lane % MI) of its MFMA tile, k group (lane / MI)
	const int frag_row = lane % MI;
	const int frag_kgroup = lane / MI;
	int a_off[TM], a_swz[TM], b_off[TN], b_swz[TN];
#pragma unroll
	for (int i = 0; i < TM; ++i)
	{
		const int row = wm * Cfg::kWaveM + i * MI + frag_row;
		a_off[i] = row * 128;
		a_swz[i] = swizzle_of_row<Cfg::SWZ>(row);
	}
	int b_off_kn[TN][2];   // transposed-B path: byte offsets of the two 4-deep transposing reads of a fragment
#pragma unroll
	for (int j = 0; j < TN; ++j)
	{
		const int row = wn * Cfg::kWaveN + j * MI + frag_row;
		b_off[j] = Cfg::kSlabABytes + row * 128;
		b_swz[j] = swizzle_of_row<Cfg::SWZ>(row);
		if constexpr (Cfg::B_KN)
		{
			// lane r of a 16-lane group addresses row k = 8 g + 4 h + r / 4, columns n .. n + 3
			const int n = wn * Cfg::kWaveN + j * MI + 4 * (frag_row & 3);
#pragma unroll
			for (int h = 0; h < 2; ++h)
			{
				const int k = 8 * frag_kgroup + 4 * h + (frag_row >> 2);
				b_off_kn[j][h] = Cfg::kSlabABytes + k * kRowBytesKN +
				                 (((n >> 3) ^ (kn_row_swizzle(k) & kChunkMaskKN)) << 4) + (n & 7) * 2;
			}
		}
	}

	half8_t af[2][TM], bf[2][TN];
	auto read_frags = [&](int buf, int stage, int step) {
		const char* base = lds + stage * Cfg::kStageBytes;
		const int chunk = step * Cfg::kKGroups + frag_kgroup;
#pragma unroll
		for (int i = 0; i < TM; ++i)
			af[buf][i] = *reinterpret_cast<const half8_t*>(base + a_off[i] + ((chunk ^ a_swz[i]) << 4));
#pragma unroll
		for (int j = 0; j < TN; ++j)
		{
			if constexpr (Cfg::B_KN)
			{
				// a step is 32 k deep; + 32 k rows leaves the row swizzle (bits 0, 1, 3 of k) unchanged
				const char* src = base + step * (32 * kRowBytesKN);
				const half4_t lo = lds_read_transposed_b64(src + b_off_kn[j][0]);
				const half4_t hi = lds_read_transposed_b64(src + b_off_kn[j][1]);
				bf[buf][j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
			}
			else
			{
				bf[buf][j] = *reinterpret_cast<const half8_t*>(base + b_off[j] + ((chunk ^ b_swz[j]) << 4));
			}
		}
	};
	auto multiply = [&](int buf) {
#pragma unroll
		for (int i = 0; i < TM; ++i)
#pragma unroll
			for (int j = 0; j < TN; ++j)
				acc[i][j] = Shape::mma(bf[buf][j], af[buf][i], acc[i][j]);
	};
	// where the LDS reads of the next step go between the TM * TN MFMAs of this one
	constexpr int kReads = TM + (Cfg::B_KN ? 2 * TN : TN);
	auto interleave_reads = [&]() {
		if constexpr (Cfg::ILV == 0)
		{
#pragma unroll
			for (int i = 0; i < kReads; ++i)
			{
				__builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
				__builtin_amdgcn_sched_group_barrier(kSchedDsRead, 1, 0);
			}
			__builtin_amdgcn_sched_group_barrier(kSchedMfma, TM * TN - kReads, 0);
		}
		else if constexpr (Cfg::ILV == 1)
		{
#pragma unroll
			for (int i = 0; i < kReads / 2; ++i)
			{
				__builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
				__builtin_amdgcn_sched_group_barrier(kSchedDsRead, 2, 0);
			}
			__builtin_amdgcn_sched_group_barrier(kSchedMfma, TM * TN - kReads / 2, 0);
		}
		// any other value: leave the placement to the compiler
	};

	const int ktiles = K / BK;

	// Loads past the last slab are clamped to the last slab: they land in a stage nobody reads
	// any more, which keeps the loop body free of branches.
	const int last = ktiles - 1;
	constexpr int S = Cfg::kStages;
	// loads of the S - 2 slabs that may stay in flight over a slab barrier
	constexpr int kInFlight = (S - 2) * (Cfg::kLoadsA + Cfg::kLoadsB);
#pragma unroll
	for (int i = 0; i < S - 1; ++i) issue_loads(min(i, last), i);
	wait_vmem_but<kInFlight>();
	__syncthreads();
	issue_loads(min(S - 1, last), S - 1);
	read_frags(0, 0, Cfg::kKGroupsOfWaves == 2 ? wk : 0);

	if constexpr (Cfg::kKGroupsOfWaves == 2)
	{
		// one step per wave and slab: the fragments of the next slab are read under the MFMAs of this one; two slabs
		// per trip so that the fragment buffers are compile-time
		auto slab = [&](int kt, auto buf) {
			constexpr int kBuf = decltype(buf)::value;
			const int stage_now = kt & 1;
			wait_vmem_but<kInFlight>();
			__syncthreads();
			issue_loads(min(kt + S, last), stage_now);
			read_frags(kBuf ^ 1, stage_now ^ 1, wk);
			multiply(kBuf);
			__builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
			__builtin_amdgcn_sched_group_barrier(kSchedVmemRead, Cfg::kLoadsA + Cfg::kLoadsB, 0);
			interleave_reads();
		};
		for (int kt = 0; kt < ktiles; kt += 2)
		{
			slab(kt, std::integral_constant<int, 0>());
			if (kt + 1 < ktiles) slab(kt + 1, std::integral_constant<int, 1>());
		}
	}
	else
	{
		int stage = 0;
		for (int kt = 0; kt < ktiles; ++kt)
		{
			if constexpr (S == 2) stage = kt & 1;               // (spelled this way the loop of the big tile is two scalar
			                                                     // instructions and a wait state shorter)
			const int next_stage = S == 2 ? (stage ^ 1) : (stage + 1 == S ? 0 : stage + 1);

	#pragma unroll
			for (int step = 0; step < Cfg::kSteps - 1; ++step)
			{
				read_frags((step + 1) & 1, stage, step + 1);
				multiply(step & 1);
				interleave_reads();
			}

			// slab t+1 has landed (own loads) and, behind the barrier, everybody's; stage `stage` is free
			wait_vmem_but<kInFlight>();
			__syncthreads();
			issue_loads(min(kt + S, last), stage);
			read_frags(0, next_stage, 0);
			multiply((Cfg::kSteps - 1) & 1);
			__builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
			__builtin_amdgcn_sched_group_barrier(kSchedVmemRead, Cfg::kLoadsA + Cfg::kLoadsB, 0);
			interleave_reads();
			if constexpr (S != 2) stage = next_stage;
		}
	}
	if constexpr (KTAIL)
	{
		constexpr int kStepDepth = 512 / MI;                 // k covered by one MFMA
		for (int k0 = ktiles * BK; k0 < K && wk == 0; k0 += kStepDepth)
		{
			const int kk = k0 + 8 * frag_kgroup;             // this lane's 8 consecutive k
			half8_t at[TM], bt[TN];
#pragma unroll
			for (int i = 0; i < TM; ++i)
			{
				int64_t grow = m0 + wm * Cfg::kWaveM + i * MI + frag_row;
				if (RAGGED && grow > M - 1) grow = M - 1;
				half8_t v = {};
				if (kk < K) v = *reinterpret_cast<const half8_t*>(A + grow * lda + kk);
				at[i] = v;
			}
#pragma unroll
			for (int j = 0; j < TN; ++j)
			{
				const int col = wn * Cfg::kWaveN + j * MI + frag_row;
				bool second = false;
				int64_t gcol = n0 + (DUAL ? dual_col(col, second) : col);
				if (RAGGED && gcol > N - 1) gcol = N - 1;
				const half_t* Bt = second ? B2 : B;
				half8_t v = {};
				if (kk < K)
				{
					if constexpr (Cfg::B_KN)
					{
#pragma unroll
						for (int e = 0; e < 8; ++e) v[e] = Bt[(int64_t)(kk + e) * ldb + gcol];
					}
					else
					{
						v = *reinterpret_cast<const half8_t*>(Bt + gcol * ldb + kk);
					}
				}
				bt[j] = v;
			}
#pragma unroll
			for (int i = 0; i < TM; ++i)
#pragma unroll
				for (int j = 0; j < TN; ++j) acc[i][j] = Shape::mma(bt[j], at[i], acc[i][j]);
		}
	}
	// no direct load may still be writing LDS when the scratch is reused or the block retires
	wait_vmem_all();
	__syncthreads();
	if constexpr (Cfg::kKGroupsOfWaves == 2)
	{
		// the second group's accumulators reach the first through LDS, half of them at a time (a wave's half is
		// 16 KB: [register][lane] floats), and only the first group stores
		static_assert(Cfg::WM * Cfg::WN * (TM * TN / 2) * Shape::kAccRegs * kWaveSize * 4 <= Cfg::kLdsBytes, "half the accumulators fit in LDS");
		float* red = reinterpret_cast<float*>(lds) + wave_in_group * ((TM * TN / 2) * Shape::kAccRegs * kWaveSize) + lane;
#pragma unroll
		for (int half = 0; half < 2; ++half)
		{
			if (wk == 1)
			{
#pragma unroll
				for (int t = 0; t < TM * TN / 2; ++t)
#pragma unroll
					for (int r = 0; r < Shape::kAccRegs; ++r)
						red[(t * Shape::kAccRegs + r) * kWaveSize] = acc[(half * (TM * TN / 2) + t) / TN][(half * (TM * TN / 2) + t) % TN][r];
			}
			__syncthreads();
			if (wk == 0)
			{
#pragma unroll
				for (int t = 0; t < TM * TN / 2; ++t)
#pragma unroll
					for (int r = 0; r < Shape::kAccRegs; ++r)
						acc[(half * (TM * TN / 2) + t) / TN][(half * (TM * TN / 2) + t) % TN][r] += red[(t * Shape::kAccRegs + r) * kWaveSize];
			}
			__syncthreads();
		}
		if (wk == 1) return;
	}
	if constexpr (SPLIT)
		store_patch_f32<Cfg>(acc, planes + (int64_t)blockIdx.y * M * N, m0 + wm * Cfg::kWaveM, n0 + wn * Cfg::kWaveN, lane, M, N);
	else
		store_patch_via_lds<Cfg, RAGGED, false, EPI>(acc, lds, C, ldc, m0 + wm * Cfg::kWaveM, n0 + wn * (DUAL ? kHalfWaveN : Cfg::kWaveN),
		                                             wave_in_group, lane, M, N, bias, ep_param);
}

// planes != NULL (SPLIT): `batch` is the number of K ranges, k_split their depth.
template <typename Cfg, bool RAGGED = false, bool KTAIL = false, bool SPLIT = false, int EPI = kEpiNone>
hipError_t launch_gemm_f16_tile(const half_t* A, const half_t* B, half_t* C, int64_t M, int64_t N, int64_t K,
                                int64_t lda, int64_t ldb, int64_t ldc,
                                int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch, hipStream_t stream,
                                float* planes = nullptr, int64_t k_split = 0,
                                const half_t* B2 = nullptr, const half_t* bias = nullptr, float ep_param = 0.0f)
{
	auto kernel = gemm_f16_nt_tile_kernel<Cfg, RAGGED, KTAIL, SPLIT, EPI>;
	constexpr int kOutN = EPI == kEpiGeluMul ? Cfg::BN / 2 : Cfg::BN;
	// More than 64 KB of dynamic LDS has to be granted per function and per device, once.
	static std::atomic<uint64_t> configured_devices{0};
	(void)hipGetLastError();
	int device = 0;
	hipError_t e = hipGetDevice(&device);
	if (e != hipSuccess) return e;
	const uint64_t bit = 1ull << (device & 63);
	if ((configured_devices.load(std::memory_order_relaxed) & bit) == 0)
	{
		e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
		                        hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::kLdsBytes);
		if (e != hipSuccess) return e;
		configured_devices.fetch_or(bit, std::memory_order_relaxed);
	}
	const int tiles_m = (int)((M + Cfg::BM - 1) / Cfg::BM), tiles_n = (int)((N + kOutN - 1) / kOutN);
	kernel<<<dim3((unsigned)(tiles_m * tiles_n), (unsigned)batch), dim3(Cfg::kThreads), Cfg::kLdsBytes, stream>>>(
		A, B, C, (int)K, lda, ldb, ldc, tiles_m, tiles_n, stride_a, stride_b, stride_c, M, N, planes, (int)k_split,
		B2, bias, ep_param);
	return hipGetLastError();
}

}  // namespace anygpu
