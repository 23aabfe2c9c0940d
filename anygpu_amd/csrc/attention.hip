// Fused scaled-dot-product attention, forward, fp16 in / fp16 out, for gfx950:
//     y = softmax(mask(softcap(alpha * q k^T))) v        per (batch, head)
// in ONE kernel.  The score matrix never reaches HBM: for 8 heads x 8192 x 8192 keys the
// three-launch form (q k^T, row softmax, p v) writes and reads 1 GiB of scores twice; this kernel
// reads q, k, v and writes y.
//
// A block of 8 waves owns 128 consecutive queries of one head, 16 per wave (256 and 32 at head
// dimension 128), so that two waves share a SIMD.  It walks the visible key range in tiles of 64 keys.  Per tile:
//   * K and V rows go global -> LDS directly into two stages; the loads of the next tile are in flight while
//     this one is being used;
//   * S^T = K Q^T with v_mfma_f32_16x16x32_f16: the K fragment is the first operand, the Q
//     fragment (kept in registers for the whole kernel) the second, so a lane ends up holding,
//     for ONE query (lane % 16), the scores of keys 4 (lane / 16) + r of each 16-key block.
//     Row maxima and sums are therefore in-lane loops plus two cross-row steps (row swaps in the VALU);
//   * scale / softcap / mask in fp32, online max / sum in the log2 domain, p = exp2(z - m)
//     rounded to fp16;
//   * O^T += V^T P^T: first operand V^T, read out of the row-major V tile with transposing LDS
//     loads (ds_read_b64_tr_b16: four consecutive keys of one column per lane), second operand the
//     p values exactly as they sit in the lane.  The result again has the query in lane % 16, so the
//     running rescale exp2(m_old - m_new) is an in-lane multiply.
// The summation index of the second product is "key slot" (lane group, j): both operands use
// slot j <-> key 16 * (2 t + j / 4) + 4 * (lane / 16) + j % 4 of the tile, so no shuffle is needed
// between the two products.
//
// At head dimension 256 a second kernel of the same layout (sdp_attention_fwd_f16_skew_kernel) computes
// the scores of tile t + 1 beside the softmax of tile t, so that the matrix and the vector instructions of a wave
// do not depend on each other.
//
// Masks are index rules (causal with the diagonal at n_k - n_q, sliding window); tiles without a
// visible key are skipped.  A query without any visible key gets zeros.
#include "device_utils.hpp"
#include "attention_walk.hpp"
#include "attention_split.hpp"
#include "attention_tile_map.hpp"
#include "gemm_band.hpp"
#include "launch.hpp"

#include <algorithm>
#include <atomic>
#include <optional>
#include <type_traits>
#include <utility>

namespace anygpu {

namespace {

constexpr int kAttnKeysPerTile = 64;

typedef short short4_t __attribute__((ext_vector_type(4)));

// ds_read_b64_tr_b16: within each group of 16 lanes, lane i receives element (i % 4) of the
// 4-element rows addressed by lanes i / 4, i / 4 + 4, i / 4 + 8, i / 4 + 12 of the group.  With lane
// r of a group pointing at V[k0 + r / 4][d0 + 4 (r % 4) ...], lane i ends up with V[k0 .. k0 + 3][d0 + i].
__device__ __forceinline__ half4_t lds_read_tr_b64(const char* lds_addr)
{
	const short4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(lds_addr));
	return __builtin_bit_cast(half4_t, v);
}

struct AttnArgs
{
	const half_t* q;
	const half_t* k;
	const half_t* v;
	half_t* y;
	int n_q, n_k;
	int q_per_kv;          // query heads that share one k / v head
	int diag;              // key j is causally visible to query i iff j <= i + diag
	int causal;
	int window;            // 0: off; else key j is visible iff j > i + diag - window
	float k_in, k_cap;     // logit transform constants (see logit2)
	float* partials;       // key-split blocks leave their partial results here: [head][split slot][part][query][D + 2]
	const half_t* mask;    // MASK kernels: additive mask [n_q, n_k] shared by all heads (added behind scale and softcap)
	int64_t mask_stride;   // halves between its rows
	const unsigned long long* tile_map;   // MASK kernels: visible-tile words [query block][map_words] (attention_tile_map.hpp), or nullptr
	int map_words;
};

// log2(e) * softcap(alpha * s); without softcap k_in = alpha log2(e); with it
// cap log2(e) tanh(alpha s / cap) = k_cap - 2 k_cap / (1 + exp2(s k_in)), k_in = 2 log2(e) alpha / cap
template <bool SOFTCAP>
__device__ __forceinline__ float logit2(float s, float k_in, float k_cap)
{
	if constexpr (SOFTCAP)
	{
		const float t = fast_exp2(s * k_in);
		return fmaf(fast_rcp(1.0f + t), -2.0f * k_cap, k_cap);
	}
	return s * k_in;
}

template <int D>
struct AttnLds
{
	// Row pitches in bytes.  Measured over pads of 16 / 32 / 48 bytes for K and 16 / 32 / 64 for V: 32 and 32 is
	// the fastest pair at every head dimension (8 - 10 % over 16 and 32).
	static constexpr int kPitchK = 2 * D + 32;
	static constexpr int kPitchV = 2 * D + 32;
	static constexpr int kBytes = kAttnKeysPerTile * (kPitchK + kPitchV);
};

// QB: 16-query blocks per wave, WAVES: waves per block; a block owns 16 * QB * WAVES consecutive queries.
// MASK: an additive mask tensor instead of the index rules (the launcher passes none): the four mask values of a lane's four scores
// of a key block are consecutive in memory; they are requested a tile ahead and added behind scale and softcap; a tile
// that the mask hides from every query of a wave costs the wave no products (it still issues its share of the next
// tile's loads); a tile that the visible-tile map of the mask (attention_tile_map.hpp) has not set for the block is
// neither loaded nor waited for.
template <int D, bool SOFTCAP, int QB, int WAVES, bool MASK = false>
__global__ __launch_bounds__(64 * WAVES) void sdp_attention_fwd_f16_kernel(const AttnArgs a, const AttnWalk walk)
{
	constexpr int kAttnQueriesPerBlock = 16 * QB * WAVES;
	extern __shared__ __align__(16) char lds[];
	using L = AttnLds<D>;
	// (these follow the stage of the tile in use)
	const char* k_lds = lds;
	const char* v_lds = lds + kAttnKeysPerTile * L::kPitchK;
	constexpr int KS = D / 32;                      // MFMA steps along the head dimension (q k^T)
	constexpr int DC = D / 16;                      // 16-wide column blocks of the output

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = tid >> 6;
	const int n = lane & 15;                        // query inside a 16-block (second MFMA operand index)
	const int g = lane >> 4;                        // lane group: k slots 8 g .. 8 g + 7 of an MFMA
	int bh, q_block, part, parts, split_slot;
	if (!attn_walk_locate_part(walk, blockIdx.x, bh, q_block, part, parts, split_slot)) return;       // the whole block
	const int q0 = q_block * kAttnQueriesPerBlock;
	const half_t* qp = a.q + (int64_t)bh * a.n_q * D;
	const half_t* kp = a.k + (int64_t)(bh / a.q_per_kv) * a.n_k * D;
	const half_t* vp = a.v + (int64_t)(bh / a.q_per_kv) * a.n_k * D;
	half_t* yp = a.y + (int64_t)bh * a.n_q * D;

	// visible key range of the whole block: from the first key of its first query to the last of its last
	const int q_last = (q0 + kAttnQueriesPerBlock - 1 < a.n_q ? q0 + kAttnQueriesPerBlock - 1 : a.n_q - 1);
	int key_hi = a.n_k - 1;
	if (a.causal && q_last + a.diag < key_hi) key_hi = q_last + a.diag;
	int key_lo = 0;
	if (a.window > 0 && q0 + a.diag - a.window + 1 > 0) key_lo = q0 + a.diag - a.window + 1;
	int t_first = key_lo / kAttnKeysPerTile;
	int t_last = key_hi >= 0 ? key_hi / kAttnKeysPerTile : -1;
	// MASK: the visible-tile map of the mask, where the launcher has made one: the words of this query block
	const unsigned long long* map_row = nullptr;
	if constexpr (MASK)
	{
		if (a.tile_map != nullptr) map_row = a.tile_map + (int64_t)q_block * a.map_words;
	}
	if (parts > 1)
	{
		// one part of the block's key tiles; the other parts are other blocks', a merge kernel combines them.  With a
		// map the parts divide the VISIBLE tiles among them, else the range
		if (MASK && map_row != nullptr) attention_visible_share(map_row, part, parts, t_first, t_last);
		else
		{
			const int per = (t_last - t_first + parts) / parts;
			t_first += part * per;
			if (t_first + per - 1 < t_last) t_last = t_first + per - 1;
		}
	}

	// this wave's queries as second operands: lane (n, g) holds q[row][32 s + 8 g .. + 7]
	int q_row[QB];
	half8_t qf[QB][KS];
#pragma unroll
	for (int b = 0; b < QB; ++b)
	{
		q_row[b] = q0 + 16 * QB * wave + 16 * b + n;
#pragma unroll
		for (int s = 0; s < KS; ++s)
		{
			half8_t val = {};
			if (q_row[b] < a.n_q) val = *reinterpret_cast<const half8_t*>(qp + (int64_t)q_row[b] * D + 32 * s + 8 * g);
			qf[b][s] = val;
		}
	}
	// visible keys of each of the two queries this lane serves: lo <= key <= hi
	int vis_lo[QB], vis_hi[QB];
#pragma unroll
	for (int b = 0; b < QB; ++b)
	{
		vis_hi[b] = a.causal ? q_row[b] + a.diag : a.n_k - 1;
		if (vis_hi[b] > a.n_k - 1) vis_hi[b] = a.n_k - 1;
		vis_lo[b] = a.window > 0 ? q_row[b] + a.diag - a.window + 1 : 0;
	}

	float m_run[QB], l_run[QB];                    // l_run: this lane's share of the row sum
	float4_t o[QB][DC];
#pragma unroll
	for (int b = 0; b < QB; ++b)
	{
		m_run[b] = -INFINITY;
		l_run[b] = 0.0f;
#pragma unroll
		for (int c = 0; c < DC; ++c) o[b][c] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
	}
	// keys visible to every query of this wave need no per-element test: [all_lo, all_hi]
	const int wq0 = q0 + 16 * QB * wave, wq1 = wq0 + 16 * QB - 1;
	const int all_hi = a.causal ? (wq0 + a.diag < a.n_k - 1 ? wq0 + a.diag : a.n_k - 1) : a.n_k - 1;
	const int all_lo = a.window > 0 ? wq1 + a.diag - a.window + 1 : 0;

	// Tiles go global -> LDS without staging registers, into two stages.  A load instruction fills 1 KB of
	// consecutive LDS; with padded tile rows a few of its lanes land in the padding and fetch a valid chunk nobody
	// reads.  Load i = wave + WAVES j of a tile: this lane's 16 bytes are the chunk at byte slot_src[j] from the
	// tile's first key.  Rows past the last key are replaced by the last one (their scores are masked, their p is
	// 0).  Written as assembly: the compiler would make every transposing LDS read wait for all outstanding
	// direct loads of the wave; the waits they need are the explicit ones in front of the tile barrier.
	constexpr int kStageBytes = L::kBytes;
	constexpr int kLoadsPerTile = kAttnKeysPerTile * L::kPitchK / 1024;
	constexpr int kSlots = (kLoadsPerTile + WAVES - 1) / WAVES;
	static_assert(L::kPitchK == L::kPitchV && kAttnKeysPerTile * L::kPitchK % 1024 == 0, "whole load instructions");
	int slot_src[kSlots];
	const int wave_s = __builtin_amdgcn_readfirstlane(wave);
#pragma unroll
	for (int j = 0; j < kSlots; ++j)
	{
		const int byte = (wave_s + WAVES * j) * 1024 + lane * 16;
		const int row = (byte / L::kPitchK) % kAttnKeysPerTile;      // (an instruction past the tile is never issued)
		const int off = byte % L::kPitchK;
		slot_src[j] = row * (2 * D) + (off < 2 * D ? off : 0);
	}
	const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
	auto issue_slot = [&](int t, int stage, int j) {
		const int i = wave_s + WAVES * j;
		if (WAVES * j + WAVES - 1 < kLoadsPerTile || i < kLoadsPerTile)
		{
			int rel = slot_src[j];
			if ((t + 1) * kAttnKeysPerTile > a.n_k)                       // block-uniform: the ragged last tile
			{
				const int row = rel / (2 * D);
				const int last = a.n_k - 1 - t * kAttnKeysPerTile;
				if (row > last) rel -= (row - last) * (2 * D);
			}
			const int64_t tile_off = (int64_t)t * (kAttnKeysPerTile * 2 * D);
			const char* ksrc = (const char*)kp + tile_off;
			const char* vsrc = (const char*)vp + tile_off;
			const unsigned m0k = lds_base + stage * kStageBytes + i * 1024;
			const unsigned m0v = m0k + kAttnKeysPerTile * L::kPitchK;
			asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(rel), "s"(ksrc), "s"(m0k) : "memory", "m0");
			asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(rel), "s"(vsrc), "s"(m0v) : "memory", "m0");
		}
	};

	// MASK: the mask values of tile t.  A lane's four scores of key block kb belong to keys 16 kb + 4 g .. + 3: fetched as
	// they are needed, the four lanes of a query would take 32 bytes of its mask row per instruction, sixteen quarter
	// lines.  Instead lane (n, g) fetches the sixteen values of key block g of its query (32 consecutive bytes at any
	// alignment: a whole 128-byte line per query and pair of instructions), and when the tile's turn comes the lane
	// groups exchange 8-byte pieces by row swaps in the VALU (a 4 x 4 transposition over g).  Keys past the end and
	// rows past the last query count as hidden.
	half4_t mk_next[MASK ? QB : 1][4];
	auto load_mask = [&](int t) {
		typedef half8_t LooseHalf8 __attribute__((aligned(2)));
#pragma unroll
		for (int b = 0; b < (MASK ? QB : 0); ++b)
		{
			const int key = t * kAttnKeysPerTile + 16 * g;
			const half_t hidden = (half_t)(-INFINITY);
			half8_t lo = {hidden, hidden, hidden, hidden, hidden, hidden, hidden, hidden}, hi = lo;
			if (q_row[b] < a.n_q)
			{
				const half_t* src = a.mask + (int64_t)q_row[b] * a.mask_stride + key;
				if (key + 15 < a.n_k)
				{
					lo = *reinterpret_cast<const LooseHalf8*>(src);
					hi = *reinterpret_cast<const LooseHalf8*>(src + 8);
				}
				else
				{
#pragma unroll
					for (int r = 0; r < 8; ++r)
					{
						if (key + r < a.n_k) lo[r] = src[r];
						if (key + 8 + r < a.n_k) hi[r] = src[8 + r];
					}
				}
			}
			mk_next[b][0] = __builtin_shufflevector(lo, lo, 0, 1, 2, 3);
			mk_next[b][1] = __builtin_shufflevector(lo, lo, 4, 5, 6, 7);
			mk_next[b][2] = __builtin_shufflevector(hi, hi, 0, 1, 2, 3);
			mk_next[b][3] = __builtin_shufflevector(hi, hi, 4, 5, 6, 7);
		}
	};
	// piece j of lane group g <-> piece g of lane group j, for every lane % 16: v_permlane32_swap exchanges the upper half
	// of its first operand with the lower half of its second, v_permlane16_swap the odd rows of the first with the even
	// rows of the second (all lanes of the wave are active here)
	auto exchange_mask_pieces = [&](half4_t (&piece)[4]) {
		typedef unsigned int uint2_t __attribute__((ext_vector_type(2)));
		uint2_t w[4];
#pragma unroll
		for (int j = 0; j < 4; ++j) w[j] = __builtin_bit_cast(uint2_t, piece[j]);
#pragma unroll
		for (int d = 0; d < 2; ++d)
		{
			unsigned int r0 = w[0][d], r1 = w[1][d], r2 = w[2][d], r3 = w[3][d];
			asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(r0), "+v"(r2));
			asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(r1), "+v"(r3));
			asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(r0), "+v"(r1));
			asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(r2), "+v"(r3));
			w[0][d] = r0;
			w[1][d] = r1;
			w[2][d] = r2;
			w[3][d] = r3;
		}
#pragma unroll
		for (int j = 0; j < 4; ++j) piece[j] = __builtin_bit_cast(half4_t, w[j]);
	};
	// MASK: the walk visits the tiles that the map has set (all of them without a map); t_next is the tile after t on
	// that walk, the stages alternate along it
	if constexpr (MASK) t_first = attention_next_visible_tile(map_row, t_first, t_last);
	if (t_first <= t_last)
	{
		if constexpr (MASK) load_mask(t_first);
#pragma unroll
		for (int j = 0; j < kSlots; ++j) issue_slot(t_first, 0, j);
	}
	int t_next = 0, stage_m = 0;
	for (int t = t_first; t <= t_last; t = MASK ? t_next : t + 1, stage_m ^= 1)
	{
		// own loads of tile t have landed; behind the barrier everybody's have, and everybody is done with the
		// stage of the tile before, which the loads of the next tile overwrite
		__builtin_amdgcn_s_waitcnt(0x0F70);            // vmcnt(0)
		__syncthreads();
		const int stage = MASK ? stage_m : (t - t_first) & 1;
		if constexpr (MASK) t_next = attention_next_visible_tile(map_row, t + 1, t_last);
		else t_next = t + 1;
		k_lds = lds + stage * kStageBytes;
		v_lds = k_lds + kAttnKeysPerTile * L::kPitchK;
		const bool more = t_next <= t_last;
		// the mask values of this tile move out of the way of the next tile's, which go out now; they stay halves until
		// the scores meet them (the float form would not fit the registers at head_dim 256)
		half4_t mk[MASK ? QB : 1][4];
		if constexpr (MASK)
		{
			bool any_visible = false;
#pragma unroll
			for (int b = 0; b < QB; ++b)
			{
#pragma unroll
				for (int kb = 0; kb < 4; ++kb) mk[b][kb] = mk_next[b][kb];
				exchange_mask_pieces(mk[b]);
#pragma unroll
				for (int kb = 0; kb < 4; ++kb)
#pragma unroll
					for (int r = 0; r < 4; ++r) any_visible |= mk[b][kb][r] > (half_t)(-INFINITY);
			}
			if (more) load_mask(t_next);
			if (__builtin_amdgcn_ballot_w64(any_visible) == 0)
			{
				if (more)
				{
#pragma unroll
					for (int j = 0; j < kSlots; ++j) issue_slot(t_next, stage ^ 1, j);
				}
				continue;
			}
		}

		// ---- S^T = K Q^T: s[b][kb] = scores of query block b against key block kb ----
		float4_t s[QB][4];
#pragma unroll
		for (int b = 0; b < QB; ++b)
#pragma unroll
			for (int kb = 0; kb < 4; ++kb) s[b][kb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
		for (int kb = 0; kb < 4; ++kb)
#pragma unroll
			for (int st = 0; st < KS; ++st)
			{
				const half8_t kf = *reinterpret_cast<const half8_t*>(k_lds + (16 * kb + n) * L::kPitchK + (32 * st + 8 * g) * 2);
#pragma unroll
				for (int b = 0; b < QB; ++b)
					s[b][kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[b][st], s[b][kb], 0, 0, 0);
				// the next tile's loads, spread behind the key blocks of this product: a wave that issues them in one
				// burst is held until the CU's vector memory path (64 bytes per clock) has taken them
				if (st == KS - 1 && more)
				{
#pragma unroll
					for (int j = kb; j < kSlots; j += 4) issue_slot(t_next, stage ^ 1, j);
				}
			}

		// ---- online softmax; p as the second operand of the next product ----
		half8_t pf[QB][2];
		const int tile_key0 = t * kAttnKeysPerTile;
		const bool interior = tile_key0 >= all_lo && tile_key0 + kAttnKeysPerTile - 1 <= all_hi;   // wave-uniform
#pragma unroll
		for (int b = 0; b < QB; ++b)
		{
			float z[4][4];
			float mt = -INFINITY;
			if (interior && !MASK)
			{
#pragma unroll
				for (int kb = 0; kb < 4; ++kb)
#pragma unroll
					for (int r = 0; r < 4; ++r)
					{
						z[kb][r] = logit2<SOFTCAP>(s[b][kb][r], a.k_in, a.k_cap);
						mt = fmaxf(mt, z[kb][r]);
					}
			}
			else
			{
#pragma unroll
				for (int kb = 0; kb < 4; ++kb)
#pragma unroll
					for (int r = 0; r < 4; ++r)
					{
						const int key = tile_key0 + 16 * kb + 4 * g + r;
						const float zz = logit2<SOFTCAP>(s[b][kb][r], a.k_in, a.k_cap) + (MASK ? (float)mk[MASK ? b : 0][kb][r] * kLog2e : 0.0f);
						z[kb][r] = (MASK || (key >= vis_lo[b] && key <= vis_hi[b])) ? zz : -INFINITY;
						mt = fmaxf(mt, z[kb][r]);
					}
			}
			mt = max_over_lane_rows(mt);
			const float m_new = fmaxf(m_run[b], mt);
			const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;   // nothing visible so far: every term is exp2(-inf) = 0
			float psum = 0.0f;
			float p[4][4];
#pragma unroll
			for (int kb = 0; kb < 4; ++kb)
#pragma unroll
				for (int r = 0; r < 4; ++r)
				{
					p[kb][r] = fast_exp2(z[kb][r] - m_safe);
					psum += p[kb][r];
				}
			// the running maximum settles after a few tiles; when no query of the wave raised it, the
			// rescale factor is 1 everywhere and the pass over the accumulators is skipped
			if (__builtin_amdgcn_ballot_w64(m_new > m_run[b]) != 0)
			{
				const float corr = fast_exp2(m_run[b] - m_safe);
				l_run[b] *= corr;
#pragma unroll
				for (int c = 0; c < DC; ++c) o[b][c] *= corr;
			}
			l_run[b] += psum;
			m_run[b] = m_new;
#pragma unroll
			for (int tt = 0; tt < 2; ++tt)
#pragma unroll
				for (int j = 0; j < 8; ++j) pf[b][tt][j] = (half_t)p[2 * tt + j / 4][j % 4];
		}

		// ---- O^T += V^T P^T ----
#pragma unroll
		for (int tt = 0; tt < 2; ++tt)
#pragma unroll
			for (int c = 0; c < DC; ++c)
			{
				const char* src = v_lds + (32 * tt + 4 * g + (n >> 2)) * L::kPitchV + (16 * c + 4 * (n & 3)) * 2;
				const half4_t lo = lds_read_tr_b64(src);
				const half4_t hi = lds_read_tr_b64(src + 16 * L::kPitchV);
				const half8_t vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
				for (int b = 0; b < QB; ++b)
					o[b][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf[b][tt], o[b][c], 0, 0, 0);
			}
	}

	// ---- normalise and store: lane (n, g) holds y[row][16 c + 4 g .. + 3] ----
#pragma unroll
	for (int b = 0; b < QB; ++b)
	{
		float l = l_run[b];
		l += __shfl_xor(l, 16);
		l += __shfl_xor(l, 32);
		if (parts > 1)
		{
			// unnormalised accumulators, running maximum and sum of this half of the keys
			if (q_row[b] < a.n_q)
			{
				float* dst = a.partials + ((((int64_t)bh * walk.n_split + split_slot) * parts + part) * kAttnQueriesPerBlock + (q_row[b] - q0)) * (D + 2);
#pragma unroll
				for (int c = 0; c < DC; ++c) *reinterpret_cast<WsFloat4*>(dst + 16 * c + 4 * g) = o[b][c];
				if (g == 0)
				{
					dst[D] = m_run[b];
					dst[D + 1] = l;
				}
			}
			continue;
		}
		const float inv = l > 0.0f ? 1.0f / l : 0.0f;
		if (q_row[b] < a.n_q)
		{
#pragma unroll
			for (int c = 0; c < DC; ++c)
			{
				half4_t out;
#pragma unroll
				for (int r = 0; r < 4; ++r) out[r] = (half_t)(o[b][c][r] * inv);
				*reinterpret_cast<half4_t*>(yp + (int64_t)q_row[b] * D + 16 * c + 4 * g) = out;
			}
		}
	}
}

// The same product with the two halves of a tile's work taken from DIFFERENT tiles, so that matrix and vector
// instructions of one wave have no dependence on each other and can issue side by side:
//     step A of tile t:  S(t + 1) = K(t + 1) Q^T  (MFMA + LDS reads)   beside   max, exp2, sum, fp16 of z(t)  (VALU)
//     step B of tile t:  O += V(t)^T P(t)^T        (MFMA + LDS reads)   beside   z(t + 1) = mask(softcap(S(t + 1)))  (VALU)
// In the kernel above every wave of the block multiplies, then exponentiates, then multiplies (the barriers of a
// tile keep the eight waves in step), so the matrix cores idle while the VALU works and the other way round.  The
// LDS holds K of tile t + 1 next to V of tile t (two stages of each, filled global -> LDS directly).  QB is 1 in
// every launch: with two 16-query blocks per wave the kernel measured slower at every head dimension.
template <int D, bool SOFTCAP, int QB, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void sdp_attention_fwd_f16_skew_kernel(const AttnArgs a, const AttnWalk walk)
{
	constexpr int kAttnQueriesPerBlock = 16 * QB * WAVES;
	extern __shared__ __align__(16) char lds[];
	using L = AttnLds<D>;
	constexpr int KS = D / 32;
	constexpr int DC = D / 16;

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
	const int n = lane & 15;
	const int g = lane >> 4;
	int bh, q_block, part, parts, split_slot;
	if (!attn_walk_locate_part(walk, blockIdx.x, bh, q_block, part, parts, split_slot)) return;
	const int q0 = q_block * kAttnQueriesPerBlock;
	const half_t* qp = a.q + (int64_t)bh * a.n_q * D;
	const half_t* kp = a.k + (int64_t)(bh / a.q_per_kv) * a.n_k * D;
	const half_t* vp = a.v + (int64_t)(bh / a.q_per_kv) * a.n_k * D;
	half_t* yp = a.y + (int64_t)bh * a.n_q * D;

	const int q_last = (q0 + kAttnQueriesPerBlock - 1 < a.n_q ? q0 + kAttnQueriesPerBlock - 1 : a.n_q - 1);
	int key_hi = a.n_k - 1;
	if (a.causal && q_last + a.diag < key_hi) key_hi = q_last + a.diag;
	int key_lo = 0;
	if (a.window > 0 && q0 + a.diag - a.window + 1 > 0) key_lo = q0 + a.diag - a.window + 1;
	int t_first = key_lo / kAttnKeysPerTile;
	int t_last = key_hi >= 0 ? key_hi / kAttnKeysPerTile : -1;
	if (parts > 1)
	{
		// one part of the block's key tiles; the other parts are other blocks', a merge kernel combines them
		const int per = (t_last - t_first + parts) / parts;
		t_first += part * per;
		if (t_first + per - 1 < t_last) t_last = t_first + per - 1;
	}

	// this wave's queries as second operands: lane (n, g) holds q[row][32 s + 8 g .. + 7]
	int q_row[QB], vis_lo[QB], vis_hi[QB];
	half8_t qf[QB][KS];
#pragma unroll
	for (int b = 0; b < QB; ++b)
	{
		q_row[b] = q0 + 16 * QB * wave + 16 * b + n;
#pragma unroll
		for (int s = 0; s < KS; ++s)
		{
			half8_t val = {};
			if (q_row[b] < a.n_q) val = *reinterpret_cast<const half8_t*>(qp + (int64_t)q_row[b] * D + 32 * s + 8 * g);
			qf[b][s] = val;
		}
		vis_hi[b] = a.causal ? q_row[b] + a.diag : a.n_k - 1;
		if (vis_hi[b] > a.n_k - 1) vis_hi[b] = a.n_k - 1;
		vis_lo[b] = a.window > 0 ? q_row[b] + a.diag - a.window + 1 : 0;
	}
	// keys visible to every query of this wave need no per-element test: [all_lo, all_hi]
	const int wq0 = q0 + 16 * QB * wave, wq1 = wq0 + 16 * QB - 1;
	const int all_hi = a.causal ? (wq0 + a.diag < a.n_k - 1 ? wq0 + a.diag : a.n_k - 1) : a.n_k - 1;
	const int all_lo = a.window > 0 ? wq1 + a.diag - a.window + 1 : 0;

	float m_run[QB], m_new[QB], l_run[QB];         // l_run: this lane's share of the row sum
	float4_t o[QB][DC];
#pragma unroll
	for (int b = 0; b < QB; ++b)
	{
		m_run[b] = -INFINITY;
		l_run[b] = 0.0f;
#pragma unroll
		for (int c = 0; c < DC; ++c) o[b][c] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
	}

	// Tiles go global -> LDS without staging registers, K and V in two stages each.  A load instruction fills 1 KB
	// of consecutive LDS; with padded tile rows a few of its lanes land in the padding and fetch a valid chunk
	// nobody reads.  Load i = wave + WAVES j of a tile: this lane's 16 bytes are the chunk at byte slot_src[j]
	// from the tile's first key.  Rows past the last key are replaced by the last one (their scores are masked,
	// their p is 0).  Written as assembly: the compiler would make every transposing LDS read wait for all
	// outstanding direct loads of the wave; the waits they need are the explicit ones in front of the barrier.
	constexpr int kStageBytes = L::kBytes;
	constexpr int kLoadsPerTile = kAttnKeysPerTile * L::kPitchK / 1024;
	constexpr int kSlots = (kLoadsPerTile + WAVES - 1) / WAVES;
	static_assert(L::kPitchK == L::kPitchV && kAttnKeysPerTile * L::kPitchK % 1024 == 0, "whole load instructions");
	// (slot_ragged: the same for the tile that holds the last key when it is not a whole tile)
	int slot_src[kSlots], slot_ragged[kSlots];
	const int t_ragged = a.n_k % kAttnKeysPerTile != 0 ? a.n_k / kAttnKeysPerTile : -1;
#pragma unroll
	for (int j = 0; j < kSlots; ++j)
	{
		const int byte = (wave + WAVES * j) * 1024 + lane * 16;
		const int row = (byte / L::kPitchK) % kAttnKeysPerTile;      // (an instruction past the tile is never issued)
		const int off = byte % L::kPitchK;
		slot_src[j] = row * (2 * D) + (off < 2 * D ? off : 0);
		const int last = a.n_k - 1 - t_ragged * kAttnKeysPerTile;
		slot_ragged[j] = slot_src[j] - (row > last ? (row - last) * (2 * D) : 0);
	}
	const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
	// slot j of tile t of matrix `src` into the K (which = 0) or V (which = 1) part of a stage.  The waves that have
	// no load in the last slot skip it inside the statement, so that the code around it stays one scheduling region.
	// The statements claim no memory effect (LDS reads may be scheduled across them: they fill the stage that is
	// not being read); what keeps them between the barrier of their tile and the wait of the next is the token they
	// hand from one to the next.
	int token = 0;
	auto issue_slot = [&](const half_t* src, int which, int t, int stage, int j) {
		const int i = wave + WAVES * j;
		const int rel = t == t_ragged ? slot_ragged[j] : slot_src[j];
		const char* base = (const char*)src + (int64_t)t * (kAttnKeysPerTile * 2 * D);
		const unsigned m0v = lds_base + stage * kStageBytes + which * (kAttnKeysPerTile * L::kPitchK) + i * 1024;
		if (WAVES * j + WAVES - 1 < kLoadsPerTile)
			asm("s_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : "+s"(token) : "v"(rel), "s"(base), "s"(m0v) : "m0");
		else
			asm("s_cmp_lt_u32 %4, %5\n\ts_cbranch_scc0 1f\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n1:"
			    : "+s"(token) : "v"(rel), "s"(base), "s"(m0v), "s"(i), "n"(kLoadsPerTile) : "m0", "scc");
	};
	// own loads have landed; behind the barrier everybody's have, and everybody is done with what the loads issued
	// after it overwrite
	auto tile_barrier = [&]() {
		asm volatile("s_waitcnt vmcnt(0)" : : "s"(token) : "memory");
		__syncthreads();
		asm volatile("" : "=s"(token));
	};
	// z of score e = 4 kb + r of query block b against tile t: scale / softcap in the log2 domain, masked keys at -inf
	auto logit_of_score = [&](auto interior_tag, float sv, int t, int b, int e, int g) {
		const float zz = logit2<SOFTCAP>(sv, a.k_in, a.k_cap);
		if constexpr (decltype(interior_tag)::value) return zz;
		else
		{
			// (a sum, so that the transform is not made conditional on the mask; the bounds pass through an empty
			// statement, so that the compiler does not keep sixteen pre-combined pairs of them in registers over the
			// whole kernel)
			int lo = vis_lo[b], hi = vis_hi[b];
			asm volatile("" : "+v"(lo), "+v"(hi));
			const int key = t * kAttnKeysPerTile + 16 * (e / 4) + 4 * g + e % 4;
			return zz + ((key >= lo && key <= hi) ? 0.0f : -INFINITY);
		}
	};
	// the same in three pieces, for steps that must not contain an operation together with the one that needs its
	// result: begin -> middle -> finish (without softcap the first is all there is)
	auto logit_begin = [&](float sv) {
		if constexpr (SOFTCAP) return fast_exp2(sv * a.k_in);
		else return sv * a.k_in;
	};
	auto logit_middle = [&](float tv) {
		if constexpr (SOFTCAP) return fast_rcp(1.0f + tv);
		else return tv;
	};
	auto logit_finish = [&](auto interior_tag, float rv, int t, int b, int e, int g) {
		float zz = rv;
		if constexpr (SOFTCAP) zz = fmaf(rv, -2.0f * a.k_cap, a.k_cap);
		if constexpr (decltype(interior_tag)::value) return zz;
		else
		{
			int lo = vis_lo[b], hi = vis_hi[b];
			asm volatile("" : "+v"(lo), "+v"(hi));
			const int key = t * kAttnKeysPerTile + 16 * (e / 4) + 4 * g + e % 4;
			return zz + ((key >= lo && key <= hi) ? 0.0f : -INFINITY);
		}
	};
	auto is_interior = [&](int t) {
		const int key0 = t * kAttnKeysPerTile;
		return key0 >= all_lo && key0 + kAttnKeysPerTile - 1 <= all_hi;
	};

	float z[QB][16];
	// running maximum including tile t (m_run: through tile t - 1); known one tile ahead, like z
	auto row_max = [&](int b) {
		float mt = -INFINITY;
#pragma unroll
		for (int e = 0; e < 16; ++e) mt = fmaxf(mt, z[b][e]);
		return fmaxf(m_run[b], max_over_lane_rows(mt));
	};
	if (t_first <= t_last)
	{
#pragma unroll
		for (int j = 0; j < kSlots; ++j)
		{
			issue_slot(kp, 0, t_first, 0, j);
			issue_slot(vp, 1, t_first, 0, j);
		}
		tile_barrier();
		if (t_first < t_last)
		{
#pragma unroll
			for (int j = 0; j < kSlots; ++j) issue_slot(kp, 0, t_first + 1, 1, j);
		}
#pragma unroll
		for (int kb = 0; kb < 4; ++kb)
		{
			float4_t acc[QB];
#pragma unroll
			for (int b = 0; b < QB; ++b) acc[b] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
			for (int st = 0; st < KS; ++st)
			{
				const half8_t kf = *reinterpret_cast<const half8_t*>(lds + (16 * kb + n) * L::kPitchK + (32 * st + 8 * g) * 2);
#pragma unroll
				for (int b = 0; b < QB; ++b) acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[b][st], acc[b], 0, 0, 0);
			}
#pragma unroll
			for (int b = 0; b < QB; ++b)
#pragma unroll
				for (int r = 0; r < 4; ++r) z[b][4 * kb + r] = logit_of_score(std::false_type{}, acc[b][r], t_first, b, 4 * kb + r, g);
		}
	}
#pragma unroll
	for (int b = 0; b < QB; ++b) m_new[b] = t_first <= t_last ? row_max(b) : -INFINITY;

	// One tile.  MORE: tile t + 1 exists (its K is on its way into the other stage); INTERIOR: every key of tile
	// t + 1 is visible to every query of the wave.  Apart from the rescale at its top the tile is one stretch of
	// code without branches.
	auto tile = [&](auto more_tag, auto interior_tag, int t) {
		constexpr bool MORE = decltype(more_tag)::value;
		// the running maximum settles after a few tiles; when no query of the wave raised it, the rescale factor
		// is 1 everywhere and the pass over the accumulators is skipped
		float m_safe[QB];
#pragma unroll
		for (int b = 0; b < QB; ++b)
		{
			m_safe[b] = (m_new[b] == -INFINITY) ? 0.0f : m_new[b];   // nothing visible so far: every term is exp2(-inf) = 0
			if (__builtin_amdgcn_ballot_w64(m_new[b] > m_run[b]) != 0)
			{
				const float corr = fast_exp2(m_run[b] - m_safe[b]);
				l_run[b] *= corr;
#pragma unroll
				for (int c = 0; c < DC; ++c) o[b][c] *= corr;
			}
			m_run[b] = m_new[b];
		}
		// K(t + 1) and V(t) have landed; K(t) and V(t - 1) are free for the loads issued below
		tile_barrier();
		// (the lane's coordinates derived again from a thread number the compiler takes for a new value: a handful of
		// instructions per tile, and the registers they and the addresses made of them would occupy over the whole
		// kernel are free)
		int tid_again = threadIdx.x;
		asm volatile("" : "+v"(tid_again));
		const int n = tid_again & 15, g = (tid_again & (kWaveSize - 1)) >> 4;
		const int stage = (t - t_first) & 1;
		const char* k_next = lds + (stage ^ 1) * kStageBytes;
		const char* v_lds = lds + stage * kStageBytes + kAttnKeysPerTile * L::kPitchK;
		const int t_k = t + 2 <= t_last ? t + 2 : t_last;       // (past the end: the last tile once more, into the free stage)

		// The tile as steps of one operand out of LDS and the QB MFMAs that use it (64 at head dimension 256): those of
		// S(t + 1) = K(t + 1) Q^T, the four key blocks in turn so that consecutive MFMAs do not wait for each other's
		// result, then those of O^T += V(t)^T P(t)^T.  Behind its MFMAs a step issues the LDS reads of the operand
		// kAhead steps later and does its share of the vector work: in the first half p(t) = exp2(z(t) - m), the 16
		// scores of a query block spread evenly over the steps, in the second z(t + 1) likewise; one load of the next
		// tiles goes out every kLoadSpacing steps.  The scheduler may reorder inside a step, not across steps.
		// (2 to 5 steps ahead measure alike, 6 and 8 slower; the boundary tiles, with their masks, have registers for 2)
		constexpr int kAhead = decltype(interior_tag)::value ? 4 : 2;
		constexpr int kLoadSpacing = 6 < (4 * KS + 2 * DC) / (2 * kSlots) ? 6 : (4 * KS + 2 * DC) / (2 * kSlots);
		constexpr int kStepsA = MORE ? 4 * KS : 0, kSteps = kStepsA + 2 * DC;
		half8_t frag[kAhead];
		auto read_operand = [&](int i) {
			if (i < kStepsA)
			{
				const int st = i / 4, kb = i % 4;
				return *reinterpret_cast<const half8_t*>(k_next + (16 * kb + n) * L::kPitchK + (32 * st + 8 * g) * 2);
			}
			const int tt = (i - kStepsA) / DC, c = (i - kStepsA) % DC;
			const char* src = v_lds + (32 * tt + 4 * g + (n >> 2)) * L::kPitchV + (16 * c + 4 * (n & 3)) * 2;
			const half4_t lo = lds_read_tr_b64(src);
			const half4_t hi = lds_read_tr_b64(src + 16 * L::kPitchV);
			return (half8_t)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
		};
		float4_t s_next[QB][4];
		float psum[QB], z_max[QB];
		half8_t pf[QB][2];
#pragma unroll
		for (int b = 0; b < QB; ++b)
		{
			psum[b] = 0.0f;
#pragma unroll
			for (int kb = 0; kb < 4; ++kb) s_next[b][kb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
		}
		auto p_of_score = [&](int b, int e) {
			const float pv = fast_exp2(z[b][e] - m_safe[b]);
			psum[b] += pv;
			pf[b][e / 8][e % 8] = (half_t)pv;
		};
		// stage of score e that belongs to step i, if any (see the table at its call)
		float xa[QB][16], tb[QB][16];
		auto vector_stage = [&](auto tag, int b, int e, int i) {
			constexpr int kStepsB = 2 * DC;
			const int a0 = e * kStepsA / 16, b0 = kStepsA + e * kStepsB / 16;
			if (i == a0) xa[b][e] = fast_exp2(z[b][e] - m_safe[b]);
			if (i == a0 + 1)
			{
				psum[b] += xa[b][e];
				pf[b][e / 8][e % 8] = (half_t)xa[b][e];
			}
			if (i == b0) tb[b][e] = logit_begin(s_next[b][e / 4][e % 4]);
			if (i == b0 + 1) tb[b][e] = logit_middle(tb[b][e]);
			if (i == b0 + 2)
			{
				z[b][e] = logit_finish(tag, tb[b][e], t + 1, b, e, g);
				z_max[b] = e == 0 ? z[b][0] : fmaxf(z_max[b], z[b][e]);
			}
		};
#pragma unroll
		for (int i = 0; i < kAhead; ++i) frag[i] = read_operand(i);
		if constexpr (!MORE)
		{
#pragma unroll
			for (int b = 0; b < QB; ++b)
#pragma unroll
				for (int e = 0; e < 16; ++e) p_of_score(b, e);
		}
		__builtin_amdgcn_sched_barrier(0);
		// (the step number as a type: every index below is a constant, whatever the optimiser makes of the loop)
		auto step = [&](auto step_tag) {
			constexpr int i = decltype(step_tag)::value;
			// The two waves of a SIMD (w and w + 4) take turns at the higher issue priority, one over the steps of the
			// first product, the other over those of the second: with equal priorities they reach every phase of a
			// tile together and compete for the same unit (Gemma2 block: 285 -> 279 us in one process; the same wave
			// always ahead: slower; turns of 16 steps or fewer: the extra branches cost registers, slower).
			if constexpr (MORE && (i == 0 || i == kStepsA))
			{
				if (((wave >> 2) & 1) == (i == 0 ? 0 : 1)) __builtin_amdgcn_s_setprio(2);
				else __builtin_amdgcn_s_setprio(0);
			}
#pragma unroll
			for (int b = 0; b < QB; ++b)
			{
				if (i < kStepsA) s_next[b][i % 4] = __builtin_amdgcn_mfma_f32_16x16x32_f16(frag[i % kAhead], qf[b][i / 4], s_next[b][i % 4], 0, 0, 0);
				else o[b][(i - kStepsA) % DC] = __builtin_amdgcn_mfma_f32_16x16x32_f16(frag[i % kAhead], pf[b][(i - kStepsA) / DC], o[b][(i - kStepsA) % DC], 0, 0, 0);
			}
			if (i + kAhead < kSteps) frag[i % kAhead] = read_operand(i + kAhead);
			if constexpr (MORE)
			{
				// the next tiles' loads, one every kLoadSpacing steps: a burst holds the wave at each load until the
				// CU's vector memory path (64 bytes per clock) has taken the ones in front of it
				if (i % kLoadSpacing == 1 && i / kLoadSpacing < 2 * kSlots)
				{
					const int m = i / kLoadSpacing;
					if (m % 2 == 0) issue_slot(vp, 1, t + 1, stage ^ 1, m / 2);
					else issue_slot(kp, 0, t_k, stage, m / 2);
				}
				// The 16 scores of a query block spread evenly over the steps of each half, every score's operations in
				// stages one step apart, so that none sits in a step with the one that needs its result (a
				// transcendental's result is not there for the next instruction, and a wave issues in order):
				//   first half, score e from step e kStepsA / 16:   x = exp2(z - m)  |  sum += x, p = fp16(x)
				//   second half, score e from step kStepsA + e kStepsB / 16:   t = exp2(s k_in)  |  r = 1 / (1 + t)  |
				//                                                              z = k_cap - 2 k_cap r, masked; tile maximum
				// (stages that fall behind the last step run behind it; p of the second half of the keys is needed from
				// step kStepsA + DC on, so the last scores' second stage may sit in the second half)
#pragma unroll
				for (int e = 0; e < 16; ++e)
#pragma unroll
					for (int b = 0; b < QB; ++b) vector_stage(interior_tag, b, e, i);
				// (p is first used behind the branch that follows the first half: without a use here the compiler moves
				// the whole half's vector work there)
				if constexpr (i == kStepsA - 1)
				{
#pragma unroll
					for (int b = 0; b < QB; ++b) asm volatile("" : "+v"(pf[b][0]), "+v"(psum[b]));
				}
			}
			__builtin_amdgcn_sched_barrier(0);
		};
		[&]<int... I>(std::integer_sequence<int, I...>) { (step(std::integral_constant<int, I>{}), ...); }(std::make_integer_sequence<int, kSteps>{});
		if constexpr (MORE)
		{
			// the stages behind the last step, in order
#pragma unroll
			for (int late = kSteps; late < kSteps + 2; ++late)
#pragma unroll
				for (int e = 0; e < 16; ++e)
#pragma unroll
					for (int b = 0; b < QB; ++b) vector_stage(interior_tag, b, e, late);
		}
#pragma unroll
		for (int b = 0; b < QB; ++b)
		{
			l_run[b] += psum[b];
			if constexpr (MORE) m_new[b] = fmaxf(m_run[b], max_over_lane_rows(z_max[b]));
		}
	};
	for (int t = t_first; t < t_last; ++t)
	{
		if (is_interior(t + 1)) tile(std::true_type{}, std::true_type{}, t);
		else tile(std::true_type{}, std::false_type{}, t);
	}
	__builtin_amdgcn_s_setprio(0);
	if (t_first <= t_last) tile(std::false_type{}, std::true_type{}, t_last);

	// ---- normalise and store: lane (n, g) holds y[row][16 c + 4 g .. + 3] ----
	// (the lane's coordinates are derived again, from a thread number the compiler takes for a new value, so that
	// nothing of them has to stay in registers over the tiles, where none is free)
	int tid_again = threadIdx.x;
	asm volatile("" : "+v"(tid_again));
	const int n_out = tid_again & 15, g_out = (tid_again & (kWaveSize - 1)) >> 4;
#pragma unroll
	for (int b = 0; b < QB; ++b)
	{
		const int row_out = q0 + 16 * QB * wave + 16 * b + n_out;
		float l = l_run[b];
		l += __shfl_xor(l, 16);
		l += __shfl_xor(l, 32);
		if (parts > 1)
		{
			// unnormalised accumulators, running maximum and sum of this half of the keys
			if (row_out < a.n_q)
			{
				float* dst = a.partials + ((((int64_t)bh * walk.n_split + split_slot) * parts + part) * kAttnQueriesPerBlock + (row_out - q0)) * (D + 2);
#pragma unroll
				for (int c = 0; c < DC; ++c) *reinterpret_cast<WsFloat4*>(dst + 16 * c + 4 * g_out) = o[b][c];
				if (g_out == 0)
				{
					dst[D] = m_run[b];
					dst[D + 1] = l;
				}
			}
			continue;
		}
		const float inv = l > 0.0f ? 1.0f / l : 0.0f;
		if (row_out < a.n_q)
		{
#pragma unroll
			for (int c = 0; c < DC; ++c)
			{
				half4_t out;
#pragma unroll
				for (int r = 0; r < 4; ++r) out[r] = (half_t)(o[b][c][r] * inv);
				*reinterpret_cast<half4_t*>(yp + (int64_t)row_out * D + 16 * c + 4 * g_out) = out;
			}
		}
	}
}

// SKEW: the kernel that takes the two halves of a tile's work from different tiles
template <int D, bool SOFTCAP, int QB, bool SKEW = false, bool MASK = false>
hipError_t launch_variant(const AttnArgs& args_in, int64_t batch_heads, hipStream_t stream)
{
	constexpr int WAVES = 8;
	static_assert(!(SKEW && MASK), "the mask tensor goes through the plain kernel");
	auto kernel = [] {
		if constexpr (SKEW) return sdp_attention_fwd_f16_skew_kernel<D, SOFTCAP, QB, WAVES>;
		else return sdp_attention_fwd_f16_kernel<D, SOFTCAP, QB, WAVES, MASK>;
	}();
	constexpr int kLdsBytes = 2 * AttnLds<D>::kBytes;           // two stages
	constexpr int kQueriesPerBlock = 16 * QB * WAVES;
	(void)hipGetLastError();
	if (kLdsBytes > 64 * 1024)
	{
		// more than 64 KB of dynamic LDS has to be granted per function and per device, once
		static std::atomic<uint64_t> configured_devices{0};
		int device = 0;
		hipError_t e = hipGetDevice(&device);
		if (e != hipSuccess) return e;
		const uint64_t bit = 1ull << (device & 63);
		if ((configured_devices.load(std::memory_order_relaxed) & bit) == 0)
		{
			e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
			if (e != hipSuccess) return e;
			configured_devices.fetch_or(bit, std::memory_order_relaxed);
		}
	}
	AttnArgs args = args_in;
	const int64_t q_blocks = (args.n_q + kQueriesPerBlock - 1) / kQueriesPerBlock;
	const AttnSplitPlan plan = plan_attention_split(args.n_q, args.n_k, args.causal, args.diag, args.window, batch_heads,
	                                                kQueriesPerBlock, kAttnKeysPerTile, D, band::workspace_capacity(stream));
	// (or, with too few query blocks for the chip, every block in several parts of its key range)
	const int64_t parts_all = plan.n_split > 0 ? 1 : plan_attention_parts(args.n_q, args.n_k, args.causal, args.diag, batch_heads, kQueriesPerBlock,
	                                                                    kAttnKeysPerTile, D, band::workspace_capacity(stream));
	args.partials = nullptr;
	if (plan.n_split > 0 || parts_all > 1)
	{
		const hipError_t ws_err = band::workspace_acquire(stream, &args.partials);
		if (ws_err != hipSuccess) return ws_err;
	}
	const AttnWalk walk = make_attn_walk(q_blocks, batch_heads, args.q_per_kv, plan.n_split, plan.n_big, parts_all);
	if (attn_walk_blocks(walk) > 0x7FFFFFFFLL) return hipErrorInvalidValue;
	kernel<<<dim3((unsigned)attn_walk_blocks(walk)), dim3(64 * WAVES), kLdsBytes, stream>>>(args, walk);
	hipError_t err = hipGetLastError();
	if (err != hipSuccess || walk.n_split == 0) return err;
	const int64_t items = batch_heads * walk.n_split * kQueriesPerBlock * (D / 4);
	sdp_attention_merge_halves_kernel<D, half_t><<<dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream>>>(
		args.partials, args.y, args.n_q, (int)q_blocks, walk.n_split, kQueriesPerBlock, parts_all > 1 ? (int)parts_all : 2);
	return hipGetLastError();
}

// Queries per wave: 16 everywhere (8 waves x 16 queries measured 1.1 - 1.5 x faster than 4 waves x 32: the smaller
// register footprint lets more waves share a SIMD), except head_dim 128 with enough query blocks to fill the chip,
// where 8 waves x 32 queries halve the LDS reads per flop and fit the register file (16 x 4096 x 128 causal: 148 us
// against 172 us).  At head_dim 256 the 32-query form does not fit the registers.
// The skewed kernel serves head_dim 256 (8 / 4 heads x 8192 x 256 with window 4096, one process: softcap 50
// 321 -> 276 us, without softcap 277 -> 264 us; 8 heads causal without softcap 381 -> 355 us).  At head_dim 128 and 64 it
// measured slower than the kernel above (16 x 4096 x 128 causal 128 -> 141 us, 32 x 2048 x 64 causal 45 -> 61 us, before
// its last tenth), and with 32 queries per wave slower at every head dimension.
template <int D>
hipError_t launch_dim(const AttnArgs& args, bool softcap, int64_t batch_heads, hipStream_t stream)
{
	if constexpr (D == 128)
	{
		if (batch_heads * ((args.n_q + 255) / 256) >= 256)
			return softcap ? launch_variant<D, true, 2>(args, batch_heads, stream) : launch_variant<D, false, 2>(args, batch_heads, stream);
	}
	if constexpr (D == 256)
		return softcap ? launch_variant<D, true, 1, true>(args, batch_heads, stream) : launch_variant<D, false, 1, true>(args, batch_heads, stream);
	else
		return softcap ? launch_variant<D, true, 1>(args, batch_heads, stream) : launch_variant<D, false, 1>(args, batch_heads, stream);
}

// ---------------------------------------------------------------------------------------------
// Decode form: very few queries per head (a generation step), long key range.  The fused kernel
// above would give every head one block walking all keys in sequence; here the KEYS are split.
//
// The q_per_kv query heads that share a key / value head, times the n_q queries of each, are the
// (at most 16) "rows" of one 16-query MFMA block, so K and V of a head are read once for all of
// them.  Pass 1: one wave per (key / value head, split of the visible key range).  K fragments
// go straight from global memory into the MFMA operand layout (16 bytes per lane, no LDS); V
// passes through a wave-private LDS tile for the transposing reads.  The wave leaves its
// running maximum, sum and unnormalised accumulators in the workspace.  Pass 2 merges the
// splits of a row: M = max m_i, y = sum o_i 2^(m_i - M) / sum l_i 2^(m_i - M).
// Workspace per (head, split, row): head_dim accumulators + maximum + sum, fp32.
// ---------------------------------------------------------------------------------------------

struct DecodeArgs
{
	AttnArgs a;
	float* ws;              // [kv_heads][splits][rows][D + 2]
	int rows;               // q_per_kv * n_q
	int groups;             // of 16 rows: a wave each
	int splits;
	int tiles_per_split;
	int t_first, t_last;    // visible key tiles of the group
};

template <int D, bool SOFTCAP>
__global__ __launch_bounds__(64) void sdp_decode_partial_kernel(const DecodeArgs da)
{
	extern __shared__ __align__(16) char lds[];           // the V tile: 64 keys x (2 D + 32) bytes
	const AttnArgs& a = da.a;
	constexpr int kPitchV = AttnLds<D>::kPitchV;
	constexpr int KS = D / 32, DC = D / 16, VPR = D / 8;
	constexpr int VPT = kAttnKeysPerTile * D / 8 / 64;    // V vectors per lane per tile

	const int lane = threadIdx.x;
	const int n = lane & 15, g = lane >> 4;
	int split, group;
	if (!decode_locate(da.groups, da.splits, split, group)) return;
	const int kvh = blockIdx.y;
	const half_t* qp = a.q + (int64_t)kvh * da.rows * D;  // the rows of a key / value head are contiguous: [q_per_kv][n_q][D]
	const int row = kDecodeRowsPerWave * group + n;        // this lane's row among them
	const half_t* kp = a.k + (int64_t)kvh * a.n_k * D;
	const half_t* vp = a.v + (int64_t)kvh * a.n_k * D;

	const bool row_ok = row < da.rows;
	const int q_idx = row_ok ? row % a.n_q : 0;             // position of this lane's row among the n_q queries
	half8_t qf[KS];
#pragma unroll
	for (int s = 0; s < KS; ++s)
	{
		half8_t val = {};
		if (row_ok) val = *reinterpret_cast<const half8_t*>(qp + (int64_t)row * D + 32 * s + 8 * g);
		qf[s] = val;
	}
	int vis_hi = a.causal ? q_idx + a.diag : a.n_k - 1;
	if (vis_hi > a.n_k - 1) vis_hi = a.n_k - 1;
	if (!row_ok) vis_hi = -1;                              // padding rows see nothing
	const int vis_lo = a.window > 0 ? q_idx + a.diag - a.window + 1 : 0;

	float m_run = -INFINITY, l_run = 0.0f;
	float4_t o[DC];
#pragma unroll
	for (int c = 0; c < DC; ++c) o[c] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

	const int t0 = da.t_first + split * da.tiles_per_split;
	int t1 = t0 + da.tiles_per_split - 1;
	if (t1 > da.t_last) t1 = da.t_last;
	// The keys are walked in sub-tiles of 32 (one MFMA step of the second product).  The loads of sub-tile u + 1 (K
	// fragments straight into operand layout, V vectors for the wave's LDS tile) are in flight while sub-tile u is
	// multiplied: a wave that loaded, waited and multiplied in turn left the memory system idle half of the time.
	constexpr int kSub = 32;
	constexpr int VPS = kSub * D / 8 / 64;                // V vectors per lane per sub-tile
	half8_t kf[2][2][KS];
	float4_t vr[2][VPS];
	auto fetch = [&](half8_t (&kd)[2][KS], float4_t (&vd)[VPS], int key0) {
#pragma unroll
		for (int kb = 0; kb < 2; ++kb)
		{
			const int key = key0 + 16 * kb + n;
#pragma unroll
			for (int st = 0; st < KS; ++st)
			{
				half8_t val = {};
				if (key < a.n_k) val = *reinterpret_cast<const half8_t*>(kp + (int64_t)key * D + 32 * st + 8 * g);
				kd[kb][st] = val;
			}
		}
#pragma unroll
		for (int i = 0; i < VPS; ++i)
		{
			const int idx = lane + 64 * i;
			const int key = key0 + idx / VPR;
			float4_t val = {};
			if (key < a.n_k) val = __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(vp + (int64_t)key * D + (idx % VPR) * 8));
			vd[i] = val;
		}
	};
	auto consume = [&](const half8_t (&kd)[2][KS], const float4_t (&vd)[VPS], int key0) {
#pragma unroll
		for (int i = 0; i < VPS; ++i)
		{
			const int idx = lane + 64 * i;
			*reinterpret_cast<float4_t*>(lds + (idx / VPR) * kPitchV + (idx % VPR) * 16) = vd[i];
		}
		float4_t s[2];
#pragma unroll
		for (int kb = 0; kb < 2; ++kb)
		{
			s[kb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
			for (int st = 0; st < KS; ++st) s[kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kd[kb][st], qf[st], s[kb], 0, 0, 0);
		}
		float z[2][4];
		float mt = -INFINITY;
#pragma unroll
		for (int kb = 0; kb < 2; ++kb)
#pragma unroll
			for (int r = 0; r < 4; ++r)
			{
				const int key = key0 + 16 * kb + 4 * g + r;
				const float zz = logit2<SOFTCAP>(s[kb][r], a.k_in, a.k_cap);
				z[kb][r] = (key >= vis_lo && key <= vis_hi) ? zz : -INFINITY;
				mt = fmaxf(mt, z[kb][r]);
			}
		mt = max_over_lane_rows(mt);
		const float m_new = fmaxf(m_run, mt);
		const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
		const float corr = fast_exp2(m_run - m_safe);
		float psum = 0.0f;
		half8_t pf;
#pragma unroll
		for (int kb = 0; kb < 2; ++kb)
#pragma unroll
			for (int r = 0; r < 4; ++r)
			{
				const float p = fast_exp2(z[kb][r] - m_safe);
				psum += p;
				pf[4 * kb + r] = (half_t)p;
			}
		l_run = l_run * corr + psum;
		m_run = m_new;
#pragma unroll
		for (int c = 0; c < DC; ++c) o[c] *= corr;

		// the V tile was written by this wave alone: its LDS writes are complete once the wave's counter says so
		__builtin_amdgcn_s_waitcnt(0xC07F);               // lgkmcnt(0)
		__builtin_amdgcn_wave_barrier();
#pragma unroll
		for (int c = 0; c < DC; ++c)
		{
			const char* src = lds + (4 * g + (n >> 2)) * kPitchV + (16 * c + 4 * (n & 3)) * 2;
			const half4_t lo = lds_read_tr_b64(src);
			const half4_t hi = lds_read_tr_b64(src + 16 * kPitchV);
			const half8_t vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
			o[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf, o[c], 0, 0, 0);
		}
		__builtin_amdgcn_s_waitcnt(0xC07F);               // the tile has been read before the next one overwrites it
		__builtin_amdgcn_wave_barrier();
	};
	// sub-tiles u0 .. u1, two per step so that the buffer of a sub-tile is a compile-time constant
	const int u0 = 2 * t0, u1 = 2 * t1 + 1;
	if (u0 <= u1) fetch(kf[0], vr[0], u0 * kSub);
	for (int u = u0; u <= u1; u += 2)
	{
		if (u + 1 <= u1) fetch(kf[1], vr[1], (u + 1) * kSub);
		__builtin_amdgcn_sched_barrier(0);
		consume(kf[0], vr[0], u * kSub);
		if (u + 1 <= u1)
		{
			if (u + 2 <= u1) fetch(kf[0], vr[0], (u + 2) * kSub);
			__builtin_amdgcn_sched_barrier(0);
			consume(kf[1], vr[1], (u + 1) * kSub);
		}
	}

	// partial result of this split: lane (n, g) holds o[row n][16 c + 4 g .. + 3]
	float l = l_run;
	l += __shfl_xor(l, 16);
	l += __shfl_xor(l, 32);
	if (row_ok)
	{
		float* dst = da.ws + (((int64_t)kvh * da.splits + split) * da.rows + row) * (D + 2);
#pragma unroll
		for (int c = 0; c < DC; ++c) *reinterpret_cast<WsFloat4*>(dst + 16 * c + 4 * g) = o[c];
		if (g == 0)
		{
			dst[D] = m_run;
			dst[D + 1] = l;
		}
	}
}

template <int D, bool SOFTCAP>
hipError_t launch_decode_variant(const DecodeArgs& da, int64_t kv_heads, hipStream_t stream)
{
	constexpr int kLdsBytes = kAttnKeysPerTile * AttnLds<D>::kPitchV;
	(void)hipGetLastError();
	sdp_decode_partial_kernel<D, SOFTCAP><<<dim3(decode_blocks(da.groups, da.splits), (unsigned)kv_heads), dim3(64), kLdsBytes, stream>>>(da);
	hipError_t e = hipGetLastError();
	if (e != hipSuccess) return e;
	sdp_decode_merge_kernel<D, half_t><<<dim3((unsigned)da.rows, (unsigned)kv_heads), dim3(256), 0, stream>>>(da.ws, da.a.y, da.rows, da.splits);
	return hipGetLastError();
}

}  // namespace

bool sdp_attention_fwd_f16_supports(int64_t head_dim)
{
	return head_dim == 64 || head_dim == 128 || head_dim == 256;
}

hipError_t launch_sdp_attention_fwd_f16(const void* q, const void* k, const void* v, void* y,
                                        int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                        float alpha, float softcap, int causal, int64_t window, hipStream_t stream,
                                        const void* mask, int64_t mask_stride)
{
	if (batch_heads == 0 || n_q == 0) return hipSuccess;
	AttnArgs args;
	args.q = static_cast<const half_t*>(q);
	args.k = static_cast<const half_t*>(k);
	args.v = static_cast<const half_t*>(v);
	args.y = static_cast<half_t*>(y);
	args.n_q = (int)n_q;
	args.n_k = (int)n_k;
	args.q_per_kv = (int)q_per_kv;
	args.diag = (int)(n_k - n_q);
	args.causal = causal ? 1 : 0;
	args.window = (int)window;
	const bool capped = softcap != 0.0f;
	args.k_in = capped ? 2.0f * kLog2e * alpha / softcap : alpha * kLog2e;
	args.k_cap = capped ? softcap * kLog2e : 0.0f;
	args.partials = nullptr;
	args.mask = static_cast<const half_t*>(mask);
	args.mask_stride = mask_stride;
	args.tile_map = nullptr;
	args.map_words = 0;
	if (mask != nullptr)
	{
		args.causal = 0;
		args.window = 0;
		// The visible-tile map of the mask, at the front of the stream's workspace (the partial results of a split key
		// range go behind it): worth its pass over the mask for large masks and long key ranges
		// (attention_mask_map_wanted), and left out where the stream has no workspace to offer (a capture without a
		// caller's workspace).  For whole query blocks the results are the same bit for bit: the map only saves the loads
		// and barriers of tiles that every wave of a block would skip.
		constexpr int kMaskQueriesPerBlock = 16 * 8;
		const int64_t words = attention_tile_map_words(n_k, kAttnKeysPerTile);
		const size_t map_bytes = (size_t)((n_q + kMaskQueriesPerBlock - 1) / kMaskQueriesPerBlock * words) * sizeof(unsigned long long);
		std::optional<band::WorkspaceReserve> map_hold;
		if (attention_mask_map_wanted(n_q, n_k) && band::workspace_capacity(stream) >= map_bytes + (1u << 16))
		{
			float* front = nullptr;
			hipError_t e = band::workspace_acquire(stream, &front);
			if (e != hipSuccess) return e;
			unsigned long long* map = reinterpret_cast<unsigned long long*>(front);
			e = launch_attention_mask_tile_map(args.mask, mask_stride, n_q, n_k, kMaskQueriesPerBlock, kAttnKeysPerTile, map, stream);
			if (e != hipSuccess) return e;
			args.tile_map = map;
			args.map_words = (int)words;
			map_hold.emplace(map_bytes);
		}
		// sixteen queries per wave at every head dimension: the mask values of a tile take the registers of a second block
#define ANYGPU_ATTN_F16_MASK_DIM(DIM) \
		return capped ? launch_variant<DIM, true, 1, false, true>(args, batch_heads, stream) : launch_variant<DIM, false, 1, false, true>(args, batch_heads, stream)
		switch (head_dim)
		{
		case 64: ANYGPU_ATTN_F16_MASK_DIM(64);
		case 128: ANYGPU_ATTN_F16_MASK_DIM(128);
		default: ANYGPU_ATTN_F16_MASK_DIM(256);
		}
#undef ANYGPU_ATTN_F16_MASK_DIM
	}
	switch (head_dim)
	{
	case 64: return launch_dim<64>(args, capped, batch_heads, stream);
	case 128: return launch_dim<128>(args, capped, batch_heads, stream);
	default: return launch_dim<256>(args, capped, batch_heads, stream);
	}
}

bool sdp_attention_decode_f16_supports(int64_t q_per_kv, int64_t n_q, int64_t head_dim)
{
	return sdp_attention_fwd_f16_supports(head_dim) && q_per_kv >= 1 && n_q >= 1 && q_per_kv * n_q <= kDecodeMaxRows;
}

int64_t sdp_attention_decode_workspace_bytes(int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                             int causal, int64_t window)
{
	if (batch_heads == 0 || n_q == 0) return 0;
	const int64_t kv_heads = batch_heads / q_per_kv;
	const DecodePlan p = plan_decode(kv_heads * ((q_per_kv * n_q + kDecodeRowsPerWave - 1) / kDecodeRowsPerWave), n_q, n_k, causal, window, kAttnKeysPerTile);
	return kv_heads * p.splits * (q_per_kv * n_q) * (head_dim + 2) * (int64_t)sizeof(float);
}

hipError_t launch_sdp_attention_decode_f16(const void* q, const void* k, const void* v, void* y, void* workspace,
                                           int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                           float alpha, float softcap, int causal, int64_t window, hipStream_t stream)
{
	if (batch_heads == 0 || n_q == 0) return hipSuccess;
	const int64_t kv_heads = batch_heads / q_per_kv;
	const DecodePlan p = plan_decode(kv_heads * ((q_per_kv * n_q + kDecodeRowsPerWave - 1) / kDecodeRowsPerWave), n_q, n_k, causal, window, kAttnKeysPerTile);
	DecodeArgs da;
	da.a.q = static_cast<const half_t*>(q);
	da.a.k = static_cast<const half_t*>(k);
	da.a.v = static_cast<const half_t*>(v);
	da.a.y = static_cast<half_t*>(y);
	da.a.n_q = (int)n_q;
	da.a.n_k = (int)n_k;
	da.a.q_per_kv = (int)q_per_kv;
	da.a.diag = (int)(n_k - n_q);
	da.a.causal = causal ? 1 : 0;
	da.a.window = (int)window;
	const bool capped = softcap != 0.0f;
	da.a.k_in = capped ? 2.0f * kLog2e * alpha / softcap : alpha * kLog2e;
	da.a.k_cap = capped ? softcap * kLog2e : 0.0f;
	da.a.partials = nullptr;
	da.ws = static_cast<float*>(workspace);
	da.rows = (int)(q_per_kv * n_q);
	da.groups = (da.rows + kDecodeRowsPerWave - 1) / kDecodeRowsPerWave;
	da.splits = p.splits;
	da.tiles_per_split = p.tiles_per_split;
	da.t_first = p.t_first;
	da.t_last = p.t_last;
#define ANYGPU_DECODE_DIM(DIM) \
	return capped ? launch_decode_variant<DIM, true>(da, kv_heads, stream) : launch_decode_variant<DIM, false>(da, kv_heads, stream)
	switch (head_dim)
	{
	case 64: ANYGPU_DECODE_DIM(64);
	case 128: ANYGPU_DECODE_DIM(128);
	default: ANYGPU_DECODE_DIM(256);
	}
#undef ANYGPU_DECODE_DIM
}

}  // namespace anygpu
