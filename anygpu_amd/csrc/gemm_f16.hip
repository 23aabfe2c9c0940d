// fp16 x fp16 -> fp32-accumulate -> fp16 GEMM for gfx950 on the MFMA units: the launchers, their plans, the merge and
// edge kernels.
//
// Four-wave kernels (gemm_f16_ring.hpp: 256 x 256 tiles; gemm_f16_ring3.hpp: 256 x 128 and 128 x 128): one wave per SIMD,
// main loops in generated assembly, whole 64-deep slabs, any M and N, B either [N, K] (k-contiguous like A) or [K, N]
// (the reference layout, transposed on the way out of LDS); the smaller two also cut along K.
// Eight-wave and 64 x 64 tile kernels (gemm_f16_tile.hpp): everything the above do not take (a K tail, few rows).
// Operands the 16-byte chunk loads cannot fetch are copied aligned into the stream's workspace first (gemm_repack.hip);
// where that is not possible or not worth it, the edge kernel: 64 x 64 tiles, guarded scalar loads and stores, either
// B layout, any shape, stride and alignment.
#include <algorithm>

#include "device_utils.hpp"
#include "gemm_f16_tile.hpp"
#include "gemm_f16_ring.hpp"
#include "gemm_f16_ring3.hpp"
#include "launch.hpp"
#include "gemm_band.hpp"
#include "anygpu_hip.h"

namespace anygpu {

// ---------------------------------------------------------------------------------------------
// Edge kernel for operands the tile kernels cannot take (N or K no multiple of 8, rows or pointers that are not
// 16-byte aligned): 128 x 128 tile, 4 waves with a 64 x 64 patch each (2 x 2 MFMA tiles of 32 x 32 x 16), 32-deep
// slabs through registers into LDS.  A vector of 8 halves that lies inside its row is fetched with one 16-byte
// load at element alignment, the ends of rows element by element, everything outside the operand is zero in LDS.
// [K, N] weights are transposed on their way into LDS (the MFMA operand is k-contiguous).
// ---------------------------------------------------------------------------------------------
// Launches of at most two 64 x 64 tiles per CU run the form with four LDS stages: alone on its CU a
// block multiplies a slab in a tenth of the memory latency, and with two stages it advanced one slab per latency
// (256 x 4096 . 4096 x 4096: 29.9 -> 16.0 us, vendor 19.1).  Denser launches keep two stages: 16 KB per stage, five
// blocks per CU cover the latency with occupancy (1024 x 2048 . 2048 x 2304: 19.3 us against 21.9 with four stages).
constexpr int kEdgeTile = 128;
constexpr int kEdgeDepth = 32;
constexpr int kEdgePitch = kEdgeDepth + 8;      // halves per LDS row: 80 bytes, keeps 16-byte alignment

typedef half8_t LooseHalf8 __attribute__((aligned(2)));
typedef half4_t LooseHalf4 __attribute__((aligned(2)));

// 8 consecutive elements of a row of `len` valid elements starting at `pos`; zeros past the end
__device__ __forceinline__ half8_t edge_fetch(const half_t* row, int64_t pos, int64_t len, bool row_ok)
{
	half8_t v = {};
	if (!row_ok || pos >= len) return v;
	if (pos + 8 <= len) return *reinterpret_cast<const LooseHalf8*>(row + pos);
#pragma unroll
	for (int e = 0; e < 8; ++e)
		if (pos + e < len) v[e] = row[pos + e];
	return v;
}

template <int B_LAYOUT>
__global__ __launch_bounds__(256) void gemm_f16_edge_kernel(
	const half_t* __restrict__ A, const half_t* __restrict__ B, half_t* __restrict__ C,
	int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
	int64_t stride_a, int64_t stride_b, int64_t stride_c)
{
	__shared__ __align__(16) half_t a_lds[kEdgeTile * kEdgePitch];
	__shared__ __align__(16) half_t b_lds[kEdgeTile * kEdgePitch];
	A += (int64_t)blockIdx.z * stride_a;
	B += (int64_t)blockIdx.z * stride_b;
	C += (int64_t)blockIdx.z * stride_c;

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = tid >> 6;
	const int64_t m0 = (int64_t)blockIdx.y * kEdgeTile;
	const int64_t n0 = (int64_t)blockIdx.x * kEdgeTile;
	const int wm = wave >> 1, wn = wave & 1;

	float16_t acc[2][2];
#pragma unroll
	for (int i = 0; i < 2; ++i)
#pragma unroll
		for (int j = 0; j < 2; ++j)
#pragma unroll
			for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

	// a slab is 128 rows x 4 vectors (k-contiguous operands) or 32 k rows x 16 vectors ([K, N] weights): 2 per thread
	half8_t ar[2], br[2];
	auto fetch = [&](int64_t k0) {
#pragma unroll
		for (int i = 0; i < 2; ++i)
		{
			const int q = tid + 256 * i;
			{
				const int r = q >> 2, c = (q & 3) * 8;
				ar[i] = edge_fetch(A + (m0 + r) * lda, k0 + c, K, m0 + r < M);
			}
			if (B_LAYOUT == ANYGPU_B_COL_MAJOR)
			{
				const int r = q >> 2, c = (q & 3) * 8;
				br[i] = edge_fetch(B + (n0 + r) * ldb, k0 + c, K, n0 + r < N);
			}
			else
			{
				const int kr = q & 31, c = (q >> 5) * 8;    // a wave's lanes on consecutive k: conflict-free LDS rows below
				br[i] = edge_fetch(B + (k0 + kr) * ldb, n0 + c, N, k0 + kr < K);
			}
		}
	};
	auto stage = [&]() {
#pragma unroll
		for (int i = 0; i < 2; ++i)
		{
			const int q = tid + 256 * i;
			*reinterpret_cast<half8_t*>(&a_lds[(q >> 2) * kEdgePitch + (q & 3) * 8]) = ar[i];
			if (B_LAYOUT == ANYGPU_B_COL_MAJOR)
			{
				*reinterpret_cast<half8_t*>(&b_lds[(q >> 2) * kEdgePitch + (q & 3) * 8]) = br[i];
			}
			else
			{
				const int kr = q & 31, c = (q >> 5) * 8;
#pragma unroll
				for (int e = 0; e < 8; ++e) b_lds[(c + e) * kEdgePitch + kr] = br[i][e];
			}
		}
	};

	const int frag_row = lane & 31;
	const int kb = (lane >> 5) * 8;
	fetch(0);
	for (int64_t k0 = 0; k0 < K; k0 += kEdgeDepth)
	{
		__syncthreads();                        // the previous slab has been read
		stage();
		__syncthreads();
		if (k0 + kEdgeDepth < K) fetch(k0 + kEdgeDepth);
#pragma unroll
		for (int st = 0; st < kEdgeDepth / 16; ++st)
		{
			half8_t af[2], bf[2];
#pragma unroll
			for (int i = 0; i < 2; ++i)
			{
				af[i] = *reinterpret_cast<const half8_t*>(&a_lds[(wm * 64 + i * 32 + frag_row) * kEdgePitch + 16 * st + kb]);
				bf[i] = *reinterpret_cast<const half8_t*>(&b_lds[(wn * 64 + i * 32 + frag_row) * kEdgePitch + 16 * st + kb]);
			}
#pragma unroll
			for (int i = 0; i < 2; ++i)
#pragma unroll
				for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
		}
	}

	// register 4 g + e of a lane: row lane % 32 of the A tile, column 8 g + 4 (lane / 32) + e of the B tile
#pragma unroll
	for (int i = 0; i < 2; ++i)
	{
		const int64_t m = m0 + wm * 64 + i * 32 + frag_row;
		if (m >= M) continue;
#pragma unroll
		for (int j = 0; j < 2; ++j)
#pragma unroll
			for (int g = 0; g < 4; ++g)
			{
				const int64_t n = n0 + wn * 64 + j * 32 + 8 * g + 4 * (lane >> 5);
				half_t* dst = C + m * ldc + n;
				if (n + 4 <= N)
				{
					*reinterpret_cast<LooseHalf4*>(dst) = half4_t{(half_t)acc[i][j][4 * g], (half_t)acc[i][j][4 * g + 1],
					                                              (half_t)acc[i][j][4 * g + 2], (half_t)acc[i][j][4 * g + 3]};
				}
				else
				{
#pragma unroll
					for (int e = 0; e < 4; ++e)
						if (n + e < N) dst[e] = (half_t)acc[i][j][4 * g + e];
				}
			}
	}
}

// What the launcher knows about the cost of its kernels: microseconds per 64-deep slab, measured on one MI355X.  It
// only ever compares sums of these with each other (and with the two absolute terms of a cut along K), so what decides
// is their ratios; the boxes of the pool differ by up to 7 % in the clock they sustain, which moves all of them alike.
// The number of CUs is the device's, not a constant.
struct TilePrices
{
	static constexpr double kBig = 1.56;          // 256 x 256, eight waves: per round of blocks (4096^3: 256 blocks, 64 slabs, 100 us)
	static constexpr double kBigWhole = 1.45;     // 256 x 256, four waves (whole tiles of k-contiguous operands): 4096^3 93 us
	static constexpr double kRect = 0.93;         // 256 x 128 in two k groups: per round of blocks
	static constexpr double kMid = 0.75;          // 128 x 128: per block and CU (144 blocks 0.75 - 1.0, 288 1.0, 576 1.7 - 2.0)
	static constexpr double kSmallAlone = 0.22;   // 64 x 64 with four stages, a CU per block
	static constexpr double kSmallPair = 0.42;    //   ... where some CUs hold two (they decide when the launch ends)
	static constexpr double kSmallDense = 0.27;   // 64 x 64 with two stages in dense launches: per block and CU
	static constexpr double kMergeLaunchUs = 4.5; // the merge launch of a cut along K
	static constexpr double kPlaneBytesPerUs = 5.0e6;   // its planes, written and read back at 5 TB/s
	static constexpr double kSplitSetupSlabs = 3.0;     // prologue and epilogue of a block, in slabs
};

// Time per 64-deep slab of `nblocks` blocks of tile edge t spread over `cus` CUs.  The smaller tiles, of which a CU holds
// several, follow the average number of blocks per CU with a floor where a lone block waits on latency.
static double slab_us(int64_t t, int64_t nblocks, int64_t cus, bool whole_tiles = false)
{
	const double rounds = (double)((nblocks + cus - 1) / cus);
	const double share = nblocks > cus ? (double)nblocks / (double)cus : 1.0;
	if (t == 256) return (whole_tiles ? TilePrices::kBigWhole : TilePrices::kBig) * rounds;
	if (t == 128) return TilePrices::kMid * share;
	if (nblocks <= 2 * cus) return nblocks <= cus ? TilePrices::kSmallAlone : TilePrices::kSmallPair;
	return TilePrices::kSmallDense * share;
}

// The four-wave kernels (one block per CU; k-contiguous operands, whole 64-deep slabs): 256 x 256, 256 x 128 and
// 128 x 128 tiles, the two smaller ones also cut along K into planes.  Microseconds per slab and round of blocks with the
// chip full and half full (fewer blocks share the L2s and the power budget), and per launch, from sweeps over K with
// uniform random operands (operands of small integers run up to a fifth faster: the clock follows the power drawn).
// 256 x 256: 4096 x 4096 x K 53.7 / 189.3 us at K = 2048 / 8192, 2048 x 4096 x K (half full) 43.8 / 139.2;
// 256 x 128: 2048 x 4096 x K 30.0 / 103.5, 2048 x 2048 x K 24.7 / 79.8;  128 x 128: 2048 x 2048 x K 17.8 / 62.6,
// 1024 x 2048 x K 14.5 / 49.6 (the vendor library on 2048 x 2048 x K: 24 / 73).
struct FourWavePrices
{
	static constexpr double kSlabFull[3] = {1.41, 0.77, 0.465};
	static constexpr double kSlabHalf[3] = {1.0, 0.575, 0.36};
	static constexpr double kLaunch[3] = {8.5, 5.5, 3.0};
	static constexpr double kOperandBytesPerUs = 5.5e6;      // what HBM gives a launch that reads its operands once
};

struct FourWavePlan
{
	int kind = -1;         // 0: 256 x 256, 1: 256 x 128, 2: 128 x 128
	int64_t splits = 1;
	double us = 1e30;
};

// dual: two products side by side in a tile (GELU(gate) * up), which then covers half the output columns
static FourWavePlan plan_four_wave(int64_t M, int64_t N, int64_t K, int64_t batch, int64_t cus, int64_t plane_room, bool dual = false)
{
	FourWavePlan best;
	const int64_t slabs = K / 64;
	for (int kind = 0; kind < 3; ++kind)
	{
		const int64_t bm = kind == 2 ? 128 : 256, bn = (kind == 0 ? 256 : 128) / (dual ? 2 : 1);
		const int64_t blocks = ((M + bm - 1) / bm) * ((N + bn - 1) / bn) * batch;
		if (blocks / batch > 0x7FFFFFFFLL) continue;
		const int64_t max_splits = (kind == 0 || batch != 1) ? 1 : std::min<int64_t>({16, K / 512, plane_room});
		for (int64_t sp = 1; sp <= std::max<int64_t>(1, max_splits); ++sp)
		{
			const int64_t nb = blocks * sp;
			if (sp > 1 && nb > 2 * cus) break;
			const int64_t rounds = (nb + cus - 1) / cus;
			const double fill = nb >= cus ? 1.0 : (double)nb / (double)cus;
			const double t = fill <= 0.5 ? 0.0 : (fill - 0.5) / 0.5;
			const double per_slab = FourWavePrices::kSlabHalf[kind] + t * (FourWavePrices::kSlabFull[kind] - FourWavePrices::kSlabHalf[kind]);
			const int64_t depth = (slabs + sp - 1) / sp;
			double us = (double)rounds * (double)depth * per_slab;
			// (few rows against a large weight matrix: the launch cannot end before the operands have come in once)
			const double stream_us = 2.0 * ((double)M + (double)N) * (double)K * (double)batch / FourWavePrices::kOperandBytesPerUs;
			if (us < stream_us) us = stream_us;
			us += FourWavePrices::kLaunch[kind];
			if (sp > 1) us += TilePrices::kMergeLaunchUs + 8.0 * (double)sp * (double)M * (double)N / TilePrices::kPlaneBytesPerUs;
			if (us < best.us)
			{
				best.kind = kind;
				best.splits = sp;
				best.us = us;
			}
		}
	}
	return best;
}

// What the launcher expects one uncut product to take with the best of its tile kernels, from the prices above (for
// comparing a product with the same product divided by rows; microseconds).
// `plane_bytes`: what the stream's workspace offers the planes of a cut along K (0: none).
static double estimate_tiles_us(int64_t M, int64_t N, int64_t K, int64_t cus, bool whole_tiles, size_t plane_bytes)
{
	const double slabs = (double)((K + 63) / 64);
	const auto blocks = [&](int64_t t) { return ((M + t - 1) / t) * ((N + t - 1) / t); };
	double per_slab = std::min({slab_us(256, blocks(256), cus, whole_tiles), slab_us(128, blocks(128), cus), slab_us(64, blocks(64), cus)});
	const int64_t blocks_rect = ((M + 255) / 256) * ((N + 127) / 128);
	per_slab = std::min(per_slab, TilePrices::kRect * (double)((blocks_rect + cus - 1) / cus));
	double us = per_slab * slabs + 6.0;
	const int64_t plane_room = (K >= 1024 && N % 8 == 0) ? (int64_t)(plane_bytes / ((size_t)M * N * sizeof(float))) : 0;
	if (whole_tiles) us = std::min(us, plan_four_wave(M, N, K, 1, cus, plane_room).us);
	// no launch ends before its operands have come in once (few rows: at what the bandwidth-shaped kernels reach)
	const double stream_us = 2.0 * ((double)M + (double)N) * (double)K / 6.2e6 + 3.0;
	return std::max(us, stream_us);
}

// C[m, n] = half(finish(sum over splits of planes[split][m][n])), one thread per eight columns (N a multiple of 8), the
// planes added in order.  EPI: kEpiBias (+ bias[n] when bias != NULL) or kEpiSoftcap.
template <int EPI>
__global__ __launch_bounds__(256) void gemm_f16_split_merge_kernel(
	const float* __restrict__ planes, half_t* __restrict__ C, int64_t M, int64_t N, int64_t ldc, int splits,
	const half_t* __restrict__ bias, float ep_param)
{
	const int64_t chunks = N / 8;
	const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
	const int64_t m = item / chunks;
	const int64_t n = (item % chunks) * 8;
	if (m >= M) return;
	const int64_t plane = M * N;
	const float* src = planes + m * N + n;
	float4_t lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = {0.0f, 0.0f, 0.0f, 0.0f};
	int sp = 0;
	for (; sp + 4 <= splits; sp += 4)
	{
		float4_t v[4][2];
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			v[i][0] = *reinterpret_cast<const float4_t*>(src + (sp + i) * plane);
			v[i][1] = *reinterpret_cast<const float4_t*>(src + (sp + i) * plane + 4);
		}
#pragma unroll
		for (int i = 0; i < 4; ++i)
		{
			lo += v[i][0];
			hi += v[i][1];
		}
	}
	for (; sp < splits; ++sp)
	{
		lo += *reinterpret_cast<const float4_t*>(src + sp * plane);
		hi += *reinterpret_cast<const float4_t*>(src + sp * plane + 4);
	}
	half8_t out;
#pragma unroll
	for (int e = 0; e < 4; ++e)
	{
		const float bias_lo = (EPI == kEpiBias && bias) ? (float)bias[n + e] : 0.0f;
		const float bias_hi = (EPI == kEpiBias && bias) ? (float)bias[n + 4 + e] : 0.0f;
		out[e] = (half_t)finish_sum<EPI, true>(lo[e], 0.0f, bias_lo, ep_param);
		out[4 + e] = (half_t)finish_sum<EPI, true>(hi[e], 0.0f, bias_hi, ep_param);
	}
	*reinterpret_cast<LooseHalf8*>(C + m * ldc + n) = out;      // rows of C may start at any element
}

static hipError_t launch_split_merge(const float* planes, half_t* c, int64_t M, int64_t N, int64_t ldc, int splits,
                                     const GemmF16Finish* finish, hipStream_t stream)
{
	const int64_t items = M * (N / 8);
	const dim3 grid((unsigned)((items + 255) / 256));
	if (finish && finish->epilogue == kEpiSoftcap)
		gemm_f16_split_merge_kernel<kEpiSoftcap><<<grid, dim3(256), 0, stream>>>(planes, c, M, N, ldc, splits, nullptr, finish->ep_param);
	else
		gemm_f16_split_merge_kernel<kEpiBias><<<grid, dim3(256), 0, stream>>>(
			planes, c, M, N, ldc, splits, finish ? static_cast<const half_t*>(finish->bias) : nullptr, 0.0f);
	return hipGetLastError();
}

bool gemm_f16_probe_applies(const void* A, const void* B, const void* C, int64_t M, int64_t N, int64_t K,
                            int64_t lda, int64_t ldb, int64_t ldc, int b_layout)
{
	return b_layout == ANYGPU_B_COL_MAJOR && reinterpret_cast<uintptr_t>(C) % 16 == 0 && ldc % 8 == 0 &&
	       gemm_f16_ring_applies(static_cast<const half_t*>(A), static_cast<const half_t*>(B), M, N, K, lda, ldb, 0, 0, 1);
}

hipError_t launch_gemm_f16_probe(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                                 int64_t lda, int64_t ldb, int64_t ldc, unsigned long long* probe, hipStream_t stream)
{
	return launch_gemm_f16_ring(static_cast<const half_t*>(A), static_cast<const half_t*>(B), static_cast<half_t*>(C), M, N, K,
	                            lda, ldb, ldc, 0, 0, 0, 1, stream, probe);
}

// rows up to which the wide band kernel takes fp16 output heads with k-contiguous weights
constexpr int64_t kWideMaxRowsF16 = 64;

hipError_t launch_gemm_f16(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                           int64_t lda, int64_t ldb, int64_t ldc,
                           int64_t stride_a, int64_t stride_b, int64_t stride_c, int64_t batch,
                           int b_layout, hipStream_t stream, GemmF16Finish* finish)
{
	if (finish) finish->handled = false;
	if (M == 0 || N == 0 || batch == 0) return hipSuccess;
	if (finish && batch != 1) return hipErrorInvalidValue;
	// (with `finish`: a part of a divided product, with whichever kernel takes it and the epilogue)
	const auto launch_part = [&](const half_t* a_part, const half_t* b_part, half_t* c_part, int64_t m, int64_t n, int64_t n_first) -> hipError_t
	{
		if (!finish) return launch_gemm_f16(a_part, b_part, c_part, m, n, K, lda, ldb, ldc, 0, 0, 0, 1, b_layout, stream);
		const half_t* bias_part = finish->bias ? static_cast<const half_t*>(finish->bias) + n_first : nullptr;
		bool supported = false;
		const hipError_t err = launch_gemm_f16_epilogue(a_part, b_part, nullptr, bias_part, c_part, m, n, K, lda, ldb, ldc, b_layout,
		                                                finish->epilogue, finish->ep_param, stream, &supported);
		return err != hipSuccess ? err : supported ? hipSuccess : hipErrorInvalidValue;
	};
	const int fin_epi = finish ? finish->epilogue : (int)kEpiBias;
	const half_t* fin_bias = finish ? static_cast<const half_t*>(finish->bias) : nullptr;
	const float fin_param = finish ? finish->ep_param : 0.0f;
	const half_t* a = static_cast<const half_t*>(A);
	const half_t* b = static_cast<const half_t*>(B);
	half_t* c = static_cast<half_t*>(C);

	// The tile kernels fetch 16-byte chunks of the operands along K (along N for [K, N] weights), which have to be
	// aligned; C is stored at element alignment, so with k-contiguous weights N, ldc and the start of C are free.
	const bool aligned = (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(B) % 16 == 0) &&
	                     (lda % 8 == 0) && (ldb % 8 == 0) && (stride_a % 8 == 0) && (stride_b % 8 == 0);
	const bool tiles_ok = aligned && K >= 64 && K % 8 == 0 && (b_layout == ANYGPU_B_COL_MAJOR || N % 8 == 0);
	// (the cut along K writes fp32 planes with rows of N: 16-byte stores there)
	const bool planes_ok = N % 8 == 0;
	// Few rows.  With four LDS stages and the cut along K the 64 x 64 tiles stream weights as fast as the kernels
	// written for few rows or faster, although most of their MFMA rows are padding: k-contiguous weights from three
	// rows on (4 x 14336 . 14336 x 4096: skinny 45 us, tiles 21 us; 8 rows of the same: band 25 us, tiles 21 us;
	// 32 x 2304 . 2304 x 32003: band 32 us, tiles 23 us; 64 x 4096 . 4096 x 14336: band 30 us, tiles 20 us), and
	// n-contiguous weights at every row count (9216 x 2304 weights, 4 rows: 17 us against 51 us; 2304 x 256000: 214 us
	// against 247 us).  One and two rows of k-contiguous weights stay with the skinny kernels (1 x 2304 . 2304 x 256000:
	// 166 us against 198 us; small weights 9 us against 13 us), and whatever the tile kernels cannot take goes to the
	// band kernels (5 .. 64 rows) or the skinny ones.
	const bool tiles_first = tiles_ok && (b_layout == ANYGPU_B_ROW_MAJOR || M >= 3);
	// Operands the tile kernels cannot fetch (an odd start or row pitch, K no multiple of 8, [K, N] weights with such an
	// N) are copied into the stream's workspace as aligned k-contiguous rows, zeros up to the next multiple of 64 behind
	// K, and the product runs on the copies: 4096 x 4100 . [4096, 4100] weights 270 -> 117 us (vendor 105 - 110).  From
	// 64 rows on (below that the weights are streamed once anyway and a copy would triple that), for products worth
	// two more launches, where the workspace holds the copies; otherwise the element-wise kernel at the bottom.
	// (fewer rows as well where none of the kernels for few rows takes the operands as they lie and the element-wise
	// kernel would be left: 16 x 4095 -> 4096 87 us that way, [K, N] weights with 4095 columns 287; the vendor 20 - 22)
	bool few_rows_copy = false;
	if (!tiles_ok && !finish && batch == 1 && M < 64 && (double)N * (double)K >= (double)(1 << 20))
	{
		const bool taken = (b_layout == ANYGPU_B_ROW_MAJOR && gemm_band_kn_f16_applies(A, B, C, M, N, K, lda, ldb, ldc)) ||
		                   (b_layout == ANYGPU_B_COL_MAJOR && M >= 3 && gemm_band_kc_wide_applies<half_t>(a, b, c, M, N, K, lda, ldb, ldc, kWideMaxRowsF16)) ||
		                   gemm_band_applies<half_t>(a, b, nullptr, c, M, N, K, lda, ldb, ldc, b_layout) ||
		                   gemm_skinny_applies<half_t>(a, b, nullptr, M, N, K, lda, ldb, b_layout);
		few_rows_copy = !taken;
	}
	if (!tiles_ok && !finish && batch == 1 && ((M >= 64 && (double)M * (double)N * (double)K >= (double)(1 << 27)) || few_rows_copy))
	{
		const bool k_odd = K % 8 != 0;
		const bool copy_a = k_odd || reinterpret_cast<uintptr_t>(A) % 16 != 0 || lda % 8 != 0;
		const bool copy_b = k_odd || reinterpret_cast<uintptr_t>(B) % 16 != 0 || ldb % 8 != 0 || (b_layout == ANYGPU_B_ROW_MAJOR && N % 8 != 0);
		const int64_t k_pad = (K + 63) / 64 * 64;
		const size_t bytes_b = copy_b ? ((size_t)N * k_pad * 2 + 255) / 256 * 256 : 0;
		const size_t room = band::workspace_copy_capacity(stream);
		// (a copy of A that does not fit beside the one of B is made and used in bands of rows, one after the other)
		int64_t band_rows = M;
		if (copy_a && bytes_b < room && (size_t)M * k_pad * 2 > room - bytes_b)
			band_rows = (int64_t)((room - bytes_b) / ((size_t)k_pad * 2)) / 256 * 256;
		const size_t bytes_a = copy_a ? ((size_t)band_rows * k_pad * 2 + 255) / 256 * 256 : 0;
		if ((copy_a || copy_b) && (band_rows == M || band_rows >= 256) && bytes_a + bytes_b <= room)
		{
			float* front = nullptr;
			hipError_t err = band::workspace_acquire(stream, &front, bytes_a + bytes_b);
			if (err != hipSuccess) return err;
			half_t* b_copy = reinterpret_cast<half_t*>(front);
			half_t* a_copy = reinterpret_cast<half_t*>(reinterpret_cast<char*>(front) + bytes_b);
			if (copy_b)
			{
				err = b_layout == ANYGPU_B_COL_MAJOR ? launch_repack_rows(b, ldb, N, K, b_copy, k_pad, 2, stream)
				                                     : launch_repack_transposed(b, ldb, K, N, b_copy, k_pad, 2, stream);
				if (err != hipSuccess) return err;
			}
			// (both copied: the zeros behind K make whole slabs of it; one copied: K stays, the copy just has its own pitch)
			const int64_t k_used = copy_a && copy_b ? k_pad : K;
			const band::WorkspaceReserve keep(bytes_a + bytes_b);
			for (int64_t m0 = 0; m0 < M; m0 += band_rows)
			{
				const int64_t rows = std::min(band_rows, M - m0);
				if (copy_a)
				{
					err = launch_repack_rows(a + m0 * lda, lda, rows, K, a_copy, k_pad, 2, stream);
					if (err != hipSuccess) return err;
				}
				err = launch_gemm_f16(copy_a ? a_copy : a + m0 * lda, copy_b ? b_copy : b, c + m0 * ldc, rows, N, k_used,
				                      copy_a ? k_pad : lda, copy_b ? k_pad : ldb, ldc, 0, 0, 0, 1, copy_b ? ANYGPU_B_COL_MAJOR : b_layout, stream);
				if (err != hipSuccess) return err;
			}
			return hipSuccess;
		}
	}
	// few rows against n-contiguous weights with so many columns that they alone fill the chip (the output head): the
	// band kernel that transposes 8 x 8 blocks of the weights in its registers (2304 x 256000, 16 - 64 rows: the tile kernels
	// take 234 - 282 us, the vendor library 215 - 230)
	// (the kernels for few rows and the merges below take the caller's epilogue; that band kernel has no bias form)
	const auto done = [&](hipError_t err) { if (finish) finish->handled = true; return err; };
	if (batch == 1 && b_layout == ANYGPU_B_ROW_MAJOR && !(fin_epi == kEpiBias && fin_bias) && gemm_band_kn_f16_applies(A, B, C, M, N, K, lda, ldb, ldc))
		return done(launch_gemm_band_kn_f16(A, B, C, M, N, K, lda, ldb, ldc, fin_epi, fin_param, stream));
	// the same for k-contiguous weights, from three rows on (one and two rows: the skinny kernels): whole 128-byte lines
	// per weight row and load instruction, an exchange between lane pairs in front of the MFMAs
	if (batch == 1 && b_layout == ANYGPU_B_COL_MAJOR && M >= 3 && gemm_band_kc_wide_applies<half_t>(a, b, c, M, N, K, lda, ldb, ldc, kWideMaxRowsF16))
		return done(launch_gemm_band_kc_wide<half_t>(a, b, fin_bias, c, M, N, K, lda, ldb, ldc, fin_epi, fin_param, stream));
	if (batch == 1 && !tiles_first && gemm_band_applies<half_t>(a, b, nullptr, c, M, N, K, lda, ldb, ldc, b_layout))
		return done(launch_gemm_band<half_t>(a, b, nullptr, fin_bias, c, M, N, K, lda, ldb, ldc, fin_epi, fin_param, stream));
	if (batch == 1 && !tiles_first && gemm_skinny_applies<half_t>(a, b, nullptr, M, N, K, lda, ldb, b_layout))
		return done(launch_gemm_skinny<half_t>(a, b, nullptr, fin_bias, c, M, N, K, lda, ldb, ldc, b_layout, fin_epi, fin_param, stream));

	if (tiles_ok)
	{
		// Tile kernels.  Big: 8 waves, 128 x 64 patch per wave, 64-bank swizzle, one LDS read behind each of the
		// first MFMAs, 16 x 16 x 32 MFMA (both MFMA shapes have the same peak rate, but under this kernel the chip
		// is power-limited and the 16 x 16 x 32 form measured 13 % faster at 4096^3: 99 us against 114 us for
		// 32 x 32 x 16 with the same tiling).  Small: 4 waves, 64 x 64 patch per wave, two blocks fit a CU.
		// Tiny: 4 waves, 32 x 32 patch per wave, the granularity the reference's own fp16 kernels require.
		// The KN forms take the reference layout, B stored [K, N], through transposing LDS reads.
		// The largest tile that still gives the chip enough blocks is taken; shapes that are not multiples of
		// it run the same kernels with clamped operand rows and guarded stores; a K that is not a multiple of the
		// 64-deep slab adds a tail multiplied from registers.
		const auto blocks = [&](int64_t tile) { return ((M + tile - 1) / tile) * ((N + tile - 1) / tile) * batch; };
		const int64_t cus = device_cu_count();
		// 256 x 256 tiles of whole 64-deep slabs take the four-wave kernel, which is cheaper per slab
		const bool whole_tiles = gemm_f16_ring_applies(a, b, M, N, K, lda, ldb, stride_a, stride_b, batch, b_layout);
		const auto slab_us = [cus, whole_tiles](int64_t t, int64_t nblocks) { return anygpu::slab_us(t, nblocks, cus, whole_tiles); };
		// Rows that end a little past a multiple of 256 make a whole further row of tiles (520 rows: three of 256, the
		// last one with 8 rows) and often a worse choice of tile for all of them: where the prices say so, the product
		// is divided into the whole multiples and the rest, which is launched as a product of its own with its own
		// kernel (520 x 4096 -> 14336: 84 us whole, 50 + 19 divided; vendor 66).
		// (a rest of more than 128 rows fills half of its tiles and more: 900 x 3584 -> 18944 got slower divided)
		if (batch == 1 && M > 256 && M % 256 != 0 && M % 256 <= 128)
		{
			const int64_t m_body = M / 256 * 256, m_tail = M - m_body;
			const size_t plane_bytes = band::workspace_capacity(stream);
			const double whole_us = estimate_tiles_us(M, N, K, cus, whole_tiles, plane_bytes);
			const double divided_us = estimate_tiles_us(m_body, N, K, cus, whole_tiles, plane_bytes) + estimate_tiles_us(m_tail, N, K, cus, whole_tiles, plane_bytes);
			if (divided_us < 0.97 * whole_us)
			{
				const hipError_t err = launch_part(a, b, c, m_body, N, 0);
				if (err != hipSuccess) return err;
				return done(launch_part(a + m_body * lda, b, c + m_body * ldc, m_tail, N, 0));
			}
		}
		const double cost256 = slab_us(256, blocks(256)), cost128 = slab_us(128, blocks(128)), cost64 = slab_us(64, blocks(64));
		int64_t tile = (cost256 <= cost128 && cost256 <= cost64) ? 256 : cost128 <= cost64 ? 128 : 64;

		// A product of 256 x 256 tiles that fills whole rounds of blocks and a bit (320 tiles pay two rounds) is divided
		// by columns into the whole rounds and the rest, which is launched as a product of its own with its own tile.
		if (tile == 256 && batch == 1)
		{
			const int64_t tiles_m = (M + 255) / 256, tiles_n = (N + 255) / 256;
			const int64_t whole = tiles_m * tiles_n / cus * cus;
			const int64_t head_cols = whole / tiles_m;
			if (whole > 0 && head_cols > 0 && head_cols < tiles_n)
			{
				const int64_t n_head = head_cols * 256, n_tail = N - n_head;
				const auto tail_blocks = [&](int64_t t) { return ((M + t - 1) / t) * ((n_tail + t - 1) / t); };
				double tail_cost = slab_us(256, tail_blocks(256));
				if (slab_us(128, tail_blocks(128)) < tail_cost) tail_cost = slab_us(128, tail_blocks(128));
				if (slab_us(64, tail_blocks(64)) < tail_cost) tail_cost = slab_us(64, tail_blocks(64));
				const double slabs = (double)((K + 63) / 64);
				const double divided = (slab_us(256, head_cols * tiles_m) + tail_cost) * slabs + TilePrices::kSplitSetupSlabs;
				if (divided < 0.93 * cost256 * slabs)
				{
					const hipError_t err = launch_part(a, b, c, M, n_head, 0);
					if (err != hipSuccess) return err;
					const half_t* b_tail = (b_layout == ANYGPU_B_COL_MAJOR) ? b + n_head * ldb : b + n_head;
					return done(launch_part(a, b_tail, c + n_head, M, n_tail, n_head));
				}
			}
		}
		// 256 x 128 tiles: eight waves in two groups that split every slab between them (one block per CU).  Per flop
		// they cost a fifth more than the 256 x 256 tiles and a third less than the 128 x 128 ones, and they are taken
		// where their number suits the 256 CUs better (2048 x 4096 . 4096 x 4096: 76 -> 62 us, vendor 62;
		// 1024 x 4096 . 4096 x 6144: 70 -> 55 us, vendor 51).
		const int64_t blocks_rect = ((M + 255) / 256) * ((N + 127) / 128) * batch;
		const double cost_rect = TilePrices::kRect * (double)((blocks_rect + cus - 1) / cus);
		const double cost_square = tile == 256 ? cost256 : tile == 128 ? cost128 : cost64;
		// (against several rounds of 256 x 256 tiles the margin is wider: their later rounds run faster than priced,
		// 4096 x 4096 . 4096 x 6144, 384 tiles: 176 us where two full rounds would take 200)
		const bool rect = K >= 512 && cost_rect < (tile == 256 ? 0.85 : 0.95) * cost_square;
		// A single product with fewer blocks than CUs and a deep K is cut along K: every range is a launch "batch"
		// writing raw fp32 sums to its own [M, N] plane of the stream's workspace, and a merge kernel adds the planes
		// in order and rounds once.  Priced with the same slab times plus the merge launch (4.5 us) and the traffic of
		// the planes (written under the product, read back by the merge: 8 bytes per sum at 5 TB/s), for every tile
		// size that leaves CUs idle: a bigger tile cut along K often beats the smaller tile that fills the chip
		// unsplit (256 x 14336 . 14336 x 4096: 128 x 128 tiles in 4 ranges, 98 -> 50 us, vendor 53;
		// 1024 x 9216 . 9216 x 2304: 73 -> 60 us, vendor 58 - 64).
		int64_t splits = 1;
		const int64_t tile_unsplit = tile;
		const double kLaunchUs = 6.0;             // prologue, epilogue and the gap between launches, for comparing plans
		double plan_us = (double)((K + 63) / 64) * (rect ? cost_rect : cost_square) + kLaunchUs;
		int64_t plane_room = 0;
		if (batch == 1 && planes_ok && K >= 1024)
		{
			const double slabs = (double)(K / 64);
			double best = slabs * (rect ? cost_rect : cost_square);
			// (as many planes as the stream's workspace holds: the caller's, or the library's own for eager launches; a
			// stream under capture without a caller's workspace has none and runs uncut)
			const int64_t room = (int64_t)(band::workspace_capacity(stream) / ((size_t)M * N * sizeof(float)));
			plane_room = room;
			for (const int64_t t : {(int64_t)256, (int64_t)128, (int64_t)64})
			{
				if (blocks(t) >= cus) continue;
				for (int64_t sp = 2; sp <= 16 && sp <= K / 512 && sp <= room; ++sp)
				{
					const double cost = (slabs / (double)sp + TilePrices::kSplitSetupSlabs) * anygpu::slab_us(t, blocks(t) * sp, cus) + TilePrices::kMergeLaunchUs +
					                    8.0 * (double)sp * (double)M * (double)N / TilePrices::kPlaneBytesPerUs;
					if (cost < 0.9 * best)
					{
						best = cost;
						splits = sp;
						tile = t;
					}
				}
			}
			if (splits > 1) plan_us = best + kLaunchUs;
		}
		// The four-wave kernels where they apply and come out cheaper than the plan so far: their smaller tiles cost
		// about half per slab of what the eight-wave tiles of the same size do (2048^3: 26 -> 16 us, vendor 22;
		// 2048 x 4096 x 4096: 60 -> 44 us, vendor 55 - 60; 512 x 6144 x 4096: 43 -> 24 us, vendor 29 - 32).
		if (whole_tiles)
		{
			const FourWavePlan four = plan_four_wave(M, N, K, batch, cus, planes_ok ? plane_room : 0);
			if (four.kind >= 0 && four.us < plan_us)
			{
				if (four.kind == 0)
				{
					if (finish) return hipSuccess;
					return launch_gemm_f16_ring(a, b, c, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, batch, stream, nullptr, b_layout);
				}
				float* planes = nullptr;
				int64_t ranges = four.splits, k_split = 0;
				if (ranges > 1)
				{
					k_split = ((K / 64 + ranges - 1) / ranges) * 64;
					ranges = (K + k_split - 1) / k_split;
				}
				if (finish && ranges <= 1) return hipSuccess;
				if (ranges > 1)
				{
					const hipError_t ws_err = band::workspace_acquire(stream, &planes);
					if (ws_err != hipSuccess) return ws_err;
				}
				const int64_t sa = ranges > 1 ? k_split : stride_a;
				const int64_t sb = ranges > 1 ? (b_layout == ANYGPU_B_COL_MAJOR ? k_split : k_split * ldb) : stride_b;
				const int64_t count = ranges > 1 ? ranges : batch;
				const hipError_t err = four.kind == 1
					? launch_gemm_f16_ring3<8, 4>(a, b, c, M, N, K, lda, ldb, ldc, sa, sb, stride_c, count, stream, planes, k_split, nullptr, 0.0f, b_layout)
					: launch_gemm_f16_ring3<4, 4>(a, b, c, M, N, K, lda, ldb, ldc, sa, sb, stride_c, count, stream, planes, k_split, nullptr, 0.0f, b_layout);
				if (err != hipSuccess || ranges <= 1) return err;
				return done(launch_split_merge(planes, c, M, N, ldc, (int)ranges, finish, stream));
			}
		}
		if (splits > 1)
		{
			int64_t k_split = 0;
			while (splits > 1)
			{
				k_split = ((K + splits - 1) / splits + 63) / 64 * 64;
				const int64_t ranges = (K + k_split - 1) / k_split;
				if (ranges == splits && K - (splits - 1) * k_split >= 64) break;     // every range holds at least a slab
				splits = ranges == splits ? splits - 1 : ranges;
			}
			if (splits > 1)
			{
				float* planes = nullptr;
				const hipError_t ws_err = band::workspace_acquire(stream, &planes);
				if (ws_err != hipSuccess) return ws_err;
				const int64_t step_b = (b_layout == ANYGPU_B_COL_MAJOR) ? k_split : k_split * ldb;
				const bool deep_stages = blocks(64) * splits <= 2 * cus;
				hipError_t err;
#define ANYGPU_F16_SPLIT(BT, WM, WN, KN, STG, KG) \
				err = launch_gemm_f16_tile<GemmTileCfg<BT, BT, WM, WN, 1, 0, 4, 16, KN, STG, KG>, true, true, true>( \
					a, b, c, M, N, K, lda, ldb, ldc, k_split, step_b, 0, splits, stream, planes, k_split)
				if (b_layout == ANYGPU_B_COL_MAJOR)
				{
					if (tile == 256) ANYGPU_F16_SPLIT(256, 2, 4, false, 2, 1);
					else if (tile == 128) ANYGPU_F16_SPLIT(128, 2, 2, false, 2, 1);
					else if (deep_stages) ANYGPU_F16_SPLIT(64, 2, 2, false, 4, 1);
					else ANYGPU_F16_SPLIT(64, 2, 2, false, 2, 1);
				}
				else
				{
					if (tile == 256) ANYGPU_F16_SPLIT(256, 2, 4, true, 2, 1);
					else if (tile == 128) ANYGPU_F16_SPLIT(128, 2, 2, true, 2, 1);
					else if (deep_stages) ANYGPU_F16_SPLIT(64, 2, 2, true, 4, 1);
					else ANYGPU_F16_SPLIT(64, 2, 2, true, 2, 1);
				}
#undef ANYGPU_F16_SPLIT
				if (err != hipSuccess) return err;
				return done(launch_split_merge(planes, c, M, N, ldc, (int)splits, finish, stream));
			}
		}
		// unsplit (also where the stream has no workspace to cut into, as under capture): the tile priced for that.
		// One "general" instantiation serves ragged M / N and a K tail alike.
		if (finish) return hipSuccess;
		tile = tile_unsplit;
		if (rect && blocks_rect / batch <= 0x7FFFFFFFLL)
		{
			const bool ragged_rect = (M % 256 != 0) || (N % 128 != 0) || (K % 64 != 0);
#define ANYGPU_F16_RECT(KN) \
			return ragged_rect ? launch_gemm_f16_tile<GemmTileCfg<256, 128, 2, 2, 1, 0, 4, 16, KN, 2, 2>, true, true>(a, b, c, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, batch, stream) \
			                   : launch_gemm_f16_tile<GemmTileCfg<256, 128, 2, 2, 1, 0, 4, 16, KN, 2, 2>, false, false>(a, b, c, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, batch, stream)
			if (b_layout == ANYGPU_B_COL_MAJOR) ANYGPU_F16_RECT(false);
			ANYGPU_F16_RECT(true);
#undef ANYGPU_F16_RECT
		}
		const bool ragged = (M % tile != 0) || (N % tile != 0) || (K % 64 != 0);
		const bool fits = ((M + tile - 1) / tile) * ((N + tile - 1) / tile) <= 0x7FFFFFFFLL;
		const bool deep_stages = blocks(64) <= 2 * cus;
#define ANYGPU_F16_TILE(BT, WM, WN, KN, STG, KG) \
		return ragged ? launch_gemm_f16_tile<GemmTileCfg<BT, BT, WM, WN, 1, 0, 4, 16, KN, STG, KG>, true, true>(a, b, c, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, batch, stream) \
		              : launch_gemm_f16_tile<GemmTileCfg<BT, BT, WM, WN, 1, 0, 4, 16, KN, STG, KG>, false, false>(a, b, c, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, batch, stream)
		if (fits && b_layout == ANYGPU_B_COL_MAJOR)
		{
			// whole 256 x 256 tiles of k-contiguous operands: the four-wave kernel with 128 x 128 patches (4096^3: 93 us
			// against 99 us for the eight-wave tile on the same box, vendor library 93 us)
			// (up to 128 rows half of a 256 x 256 tile is empty and the product waits for its weights: the 128 x 128
			// four-wave tiles, of which a CU holds more loads in flight, stream them faster once they fill the chip,
			// 128 x 8192 -> 131072: 449 -> 383 us, 65 x 2304 -> 256000: 308 -> 253, vendor 391 / 236)
			if (tile == 256 && whole_tiles && M <= 128 && batch == 1 && blocks(128) >= cus)
				return launch_gemm_f16_ring3<4, 4>(a, b, c, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, batch, stream, nullptr, 0, nullptr, 0.0f, b_layout);
			if (tile == 256 && whole_tiles)
				return launch_gemm_f16_ring(a, b, c, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, batch, stream);
			if (tile == 256) ANYGPU_F16_TILE(256, 2, 4, false, 2, 1);
			if (tile == 128) ANYGPU_F16_TILE(128, 2, 2, false, 2, 1);
			if (deep_stages) ANYGPU_F16_TILE(64, 2, 2, false, 4, 1);
			ANYGPU_F16_TILE(64, 2, 2, false, 2, 1);
		}
		if (fits && b_layout == ANYGPU_B_ROW_MAJOR)
		{
			if (tile == 256 && whole_tiles && M <= 128 && batch == 1 && blocks(128) >= cus)        // (as above; [K, N]: 451 -> 395 us)
				return launch_gemm_f16_ring3<4, 4>(a, b, c, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, batch, stream, nullptr, 0, nullptr, 0.0f, b_layout);
			if (tile == 256 && whole_tiles)
				return launch_gemm_f16_ring(a, b, c, M, N, K, lda, ldb, ldc, stride_a, stride_b, stride_c, batch, stream, nullptr, b_layout);
			if (tile == 256) ANYGPU_F16_TILE(256, 2, 4, true, 2, 1);
			if (tile == 128) ANYGPU_F16_TILE(128, 2, 2, true, 2, 1);
			if (deep_stages) ANYGPU_F16_TILE(64, 2, 2, true, 4, 1);
			ANYGPU_F16_TILE(64, 2, 2, true, 2, 1);
		}
#undef ANYGPU_F16_TILE
	}
	if (finish) return hipSuccess;

	const dim3 grid((unsigned)((N + kEdgeTile - 1) / kEdgeTile), (unsigned)((M + kEdgeTile - 1) / kEdgeTile), (unsigned)batch);
	discard_stale_error();
	if (b_layout == ANYGPU_B_COL_MAJOR)
		gemm_f16_edge_kernel<ANYGPU_B_COL_MAJOR><<<grid, dim3(256), 0, stream>>>(a, b, c, M, N, K, lda, ldb, ldc,
		                                                                 stride_a, stride_b, stride_c);
	else
		gemm_f16_edge_kernel<ANYGPU_B_ROW_MAJOR><<<grid, dim3(256), 0, stream>>>(a, b, c, M, N, K, lda, ldb, ldc,
		                                                                 stride_a, stride_b, stride_c);
	return hipGetLastError();
}

// bias / softcap applied in place to a finished product (the shapes only the edge kernel takes)
template <int EPI>
__global__ __launch_bounds__(256) void gemm_f16_finish_kernel(half_t* __restrict__ C, const half_t* __restrict__ bias,
                                                              int64_t M, int64_t N, int64_t ldc, float ep_param)
{
	const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (item >= M * N) return;
	const int64_t m = item / N, n = item % N;
	half_t* p = C + m * ldc + n;
	*p = (half_t)finish_sum<EPI>((float)*p, 0.0f, EPI == kEpiBias ? (float)bias[n] : 0.0f, ep_param);
}

// The fp16 product with an epilogue: kEpiBias (+ bias[n], fp16), kEpiSoftcap (cap * tanh(sum / cap)) or kEpiGeluMul
// (gelu_tanh(A B) * (A B2)), applied to the fp32 sums before the one rounding to fp16.  Few rows against k-contiguous
// weights take the band kernels; everything else the plain tile kernels (256 / 128 / 64, priced like the unfused
// product, uncut), whose epilogue does the work.
hipError_t launch_gemm_f16_epilogue(const void* A, const void* B, const void* B2, const void* bias, void* C,
                                    int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                    int b_layout, int epilogue, float ep_param, hipStream_t stream, bool* supported)
{
	*supported = true;
	if (M == 0 || N == 0) return hipSuccess;
	const half_t* a = static_cast<const half_t*>(A);
	const half_t* b = static_cast<const half_t*>(B);
	const half_t* b2 = static_cast<const half_t*>(B2);
	const half_t* bs = static_cast<const half_t*>(bias);
	half_t* c = static_cast<half_t*>(C);
	const bool dual = epilogue == kEpiGeluMul;
	const bool aligned = (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(B) % 16 == 0) &&
	                     (!dual || reinterpret_cast<uintptr_t>(B2) % 16 == 0) && (lda % 8 == 0) && (ldb % 8 == 0);
	const bool tiles_ok = aligned && K >= 64 && K % 8 == 0 && (b_layout == ANYGPU_B_COL_MAJOR || N % 8 == 0);
	// one product: the few-row kernels and the plans cut along K of the plain product, which take the epilogue along
	// (8 x 9216 -> 2304 with a bias: 64 us through an uncut tile kernel, the plain product takes 14)
	if (!dual)
	{
		GemmF16Finish finish = {epilogue, bias, ep_param, false};
		const hipError_t err = launch_gemm_f16(A, B, C, M, N, K, lda, ldb, ldc, 0, 0, 0, 1, b_layout, stream, &finish);
		if (err != hipSuccess || finish.handled) return err;
	}
	if (dual && gemm_band_applies<half_t>(a, b, b2, c, M, N, K, lda, ldb, ldc, b_layout))
		return launch_gemm_band<half_t>(a, b, b2, nullptr, c, M, N, K, lda, ldb, ldc, epilogue, ep_param, stream);
	if (!tiles_ok)
	{
		if (dual)
		{
			*supported = false;
			return hipSuccess;
		}
		const hipError_t err = launch_gemm_f16(A, B, C, M, N, K, lda, ldb, ldc, 0, 0, 0, 1, b_layout, stream);
		if (err != hipSuccess) return err;
		const dim3 grid((unsigned)((M * N + 255) / 256));
		if (epilogue == kEpiBias) gemm_f16_finish_kernel<kEpiBias><<<grid, dim3(256), 0, stream>>>(c, bs, M, N, ldc, ep_param);
		else gemm_f16_finish_kernel<kEpiSoftcap><<<grid, dim3(256), 0, stream>>>(c, bs, M, N, ldc, ep_param);
		return hipGetLastError();
	}
	const int64_t cus = device_cu_count();
	// one product, k-contiguous weights, whole slabs: the four-wave kernels, priced like the unfused product, uncut
	if (b_layout == ANYGPU_B_COL_MAJOR && gemm_f16_ring_applies(a, b, M, N, K, lda, ldb, 0, 0, 1, b_layout) &&
	    (!dual || reinterpret_cast<uintptr_t>(B2) % 16 == 0))
	{
		const FourWavePlan four = plan_four_wave(M, N, K, 1, cus, 0, dual);
		const auto small_blocks = [&](int64_t t) { return ((M + t - 1) / t) * ((N + (dual ? t / 2 : t) - 1) / (dual ? t / 2 : t)); };
		const double small_us = (double)(K / 64) * slab_us(64, small_blocks(64), cus) + 6.0;
		if (four.kind >= 0 && four.us < small_us)
		{
#define ANYGPU_F16_EPI_FOUR(EPI) \
			do { \
				if (four.kind == 0) return launch_gemm_f16_ring<EPI>(a, b, c, M, N, K, lda, ldb, ldc, 0, 0, 0, 1, stream, nullptr, b_layout, bs, ep_param); \
				if (four.kind == 1) return launch_gemm_f16_ring3<8, 4, EPI>(a, b, c, M, N, K, lda, ldb, ldc, 0, 0, 0, 1, stream, nullptr, 0, bs, ep_param); \
				return launch_gemm_f16_ring3<4, 4, EPI>(a, b, c, M, N, K, lda, ldb, ldc, 0, 0, 0, 1, stream, nullptr, 0, bs, ep_param); \
			} while (0)
			if (epilogue == kEpiSoftcap) ANYGPU_F16_EPI_FOUR(kEpiSoftcap);
			if (epilogue == kEpiBias) ANYGPU_F16_EPI_FOUR(kEpiBias);
			// (the second weight matrix travels in the bias argument)
			if (four.kind == 0) return launch_gemm_f16_ring<kEpiGeluMul>(a, b, c, M, N, K, lda, ldb, ldc, 0, 0, 0, 1, stream, nullptr, b_layout, b2, 0.0f);
			if (four.kind == 1) return launch_gemm_f16_ring3<8, 4, kEpiGeluMul>(a, b, c, M, N, K, lda, ldb, ldc, 0, 0, 0, 1, stream, nullptr, 0, b2, 0.0f);
			return launch_gemm_f16_ring3<4, 4, kEpiGeluMul>(a, b, c, M, N, K, lda, ldb, ldc, 0, 0, 0, 1, stream, nullptr, 0, b2, 0.0f);
#undef ANYGPU_F16_EPI_FOUR
		}
	}
	// a tile of edge t covers t (t / 2 with two products) output columns
	const auto blocks = [&](int64_t t) { return ((M + t - 1) / t) * ((N + (dual ? t / 2 : t) - 1) / (dual ? t / 2 : t)); };
	const double cost256 = slab_us(256, blocks(256), cus), cost128 = slab_us(128, blocks(128), cus), cost64 = slab_us(64, blocks(64), cus);
	const int64_t tile = (cost256 <= cost128 && cost256 <= cost64) ? 256 : cost128 <= cost64 ? 128 : 64;
	if (blocks(tile) > 0x7FFFFFFFLL)
	{
		*supported = false;
		return hipSuccess;
	}
#define ANYGPU_F16_EPI_TILE(BT, WM, WN, KN, EPI) \
	return launch_gemm_f16_tile<GemmTileCfg<BT, BT, WM, WN, 1, 0, 4, 16, KN, 2, 1>, true, true, false, EPI>( \
		a, b, c, M, N, K, lda, ldb, ldc, 0, 0, 0, 1, stream, nullptr, 0, b2, bs, ep_param)
#define ANYGPU_F16_EPI_LAYOUT(KN, EPI) \
	do { \
		if (tile == 256) ANYGPU_F16_EPI_TILE(256, 2, 4, KN, EPI); \
		if (tile == 128) ANYGPU_F16_EPI_TILE(128, 2, 2, KN, EPI); \
		ANYGPU_F16_EPI_TILE(64, 2, 2, KN, EPI); \
	} while (0)
#define ANYGPU_F16_EPI(EPI) \
	do { \
		if (b_layout == ANYGPU_B_COL_MAJOR) ANYGPU_F16_EPI_LAYOUT(false, EPI); \
		ANYGPU_F16_EPI_LAYOUT(true, EPI); \
	} while (0)
	if (epilogue == kEpiSoftcap) ANYGPU_F16_EPI(kEpiSoftcap);
	if (epilogue == kEpiGeluMul) ANYGPU_F16_EPI(kEpiGeluMul);
	ANYGPU_F16_EPI(kEpiBias);
#undef ANYGPU_F16_EPI
#undef ANYGPU_F16_EPI_LAYOUT
#undef ANYGPU_F16_EPI_TILE
}

}  // namespace anygpu
