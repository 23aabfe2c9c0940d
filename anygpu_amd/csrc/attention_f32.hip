// Fused scaled-dot-product attention, forward, float32 throughout, for gfx950:
//     y = softmax(mask(softcap(alpha * q k^T))) v        per (batch, head)
// in one kernel, with the true fp32 matrix instruction v_mfma_f32_16x16x4_f32.  The score matrix never
// reaches HBM (8 heads x 8192 x 8192 keys: 2 GiB of fp32 scores written and read twice by the three-launch form).
//
// The structure is the one of the half precision kernel: a wave owns 16 queries, the query of a lane is
// lane % 16 in every product, so row maxima and sums are in-lane loops plus two cross-lane steps, and the
// rescale of the running output is an in-lane multiply.  Per tile of 32 keys:
//   * S^T = K Q^T: first operand K, second operand Q (in registers for the whole kernel).  The summation index
//     of an MFMA is a dummy index: lane group g takes head-dimension elements 16 s + 4 g + e in step (s, e), so
//     that a lane reads its four K values of four consecutive MFMAs with one 16-byte LDS load and holds its Q
//     values as the matching vectors.  A lane ends up with the scores of keys 16 kb + 4 g + r of its query.
//   * scale / softcap / mask, online max / sum in the log2 domain, p = exp2(z - m), all fp32;
//   * O^T += V^T P^T: second operand the p values exactly as they sit in the lane (key slot (kb, r) of lane
//     group g <-> key 16 kb + 4 g + r), first operand V^T: lane (i, g) loads the four columns 64 c + 4 i .. + 3
//     of that key's V row with one 16-byte LDS load, and element e of the vector feeds its own MFMA and
//     accumulator, which therefore holds head-dimension elements 64 c + 4 i' + e: permuted between lanes and
//     accumulators, and un-permuted for free at the store, where the four accumulators of a lane hold four
//     consecutive elements.
// At 32 cycles per MFMA the matrix pipe is the bound by a wide margin (the softmax arithmetic of a tile is
// about 2 % of its MFMA time); the K and V tiles of the next step are in flight meanwhile.
//
// Masks are index rules (causal with the diagonal at n_k - n_q, sliding window); tiles without a visible key
// are skipped.  A query without any visible key gets zeros.
#include "device_utils.hpp"
#include "attention_walk.hpp"
#include "attention_split.hpp"
#include "attention_tile_map.hpp"
#include "gemm_band.hpp"
#include "launch.hpp"

#include <atomic>
#include <optional>

namespace anygpu {

namespace {


struct AttnArgsF32
{
	const float* q;
	const float* k;
	const float* v;
	float* y;
	int n_q, n_k;
	int q_per_kv;          // query heads that share one k / v head
	int diag;              // key j is causally visible to query i iff j <= i + diag
	int causal;
	int window;            // 0: off; else key j is visible iff j > i + diag - window
	float k_in, k_cap;     // logit transform constants (see logit2)
	float* partials;       // key-split blocks leave their partial results here: [head][split slot][part][query][D + 2]
	const float* mask;     // MASK kernels: additive mask [n_q, n_k] shared by all heads (added behind scale and softcap)
	int64_t mask_stride;   // floats between its rows
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

template <int D, int KT>
struct AttnLdsF32
{
	static constexpr int kPitch = D + 8;                      // floats per tile row: 32 bytes of padding
	static constexpr int kStageFloats = 2 * KT * kPitch;      // a K tile and a V tile of KT keys
};

// Scheduling-group masks of __builtin_amdgcn_sched_group_barrier
constexpr int kSchedMfma = 0x008;
constexpr int kSchedDsRead = 0x100;

// vmcnt(0) with the other counters left alone (gfx9 encoding: vmcnt in [3:0] and [15:14], expcnt [6:4], lgkmcnt [11:8])
__device__ __forceinline__ void wait_vmem_all()
{
	__builtin_amdgcn_s_waitcnt(0x0F70);
}

// WAVES waves per block, 16 queries per wave, tiles of KT keys.
// DIRECT (head dimension 256, where a tile row is exactly the 1024 bytes one wave-wide load instruction moves): the
// tiles go from memory straight into LDS, into one of two stages, so no staging registers are held and a block of
// 8 waves (two per SIMD: one multiplies while the other does its softmax arithmetic) fits the register file.
// Otherwise the tiles pass through registers into a single stage.
// MASK: an additive mask tensor instead of (or on top of) the index rules: the four mask values of a lane's four scores
// of a key block are consecutive in memory; they are requested in front of the tile's first product and added behind
// scale and softcap.  A tile that the mask hides from every query of a wave costs the wave no products; a tile that the
// visible-tile map of the mask (attention_tile_map.hpp) has not set for the block is neither loaded nor waited for.
template <int D, bool SOFTCAP, int WAVES, int KT, bool DIRECT, bool MASK>
__global__ __launch_bounds__(64 * WAVES) void sdp_attention_fwd_f32_kernel(const AttnArgsF32 a, const AttnWalk walk)
{
	constexpr int kKeysPerTile = KT;
	static_assert(!DIRECT || D == 256, "one load instruction per tile row");
	constexpr int kQueriesPerBlock = 16 * WAVES;
	constexpr int THREADS = 64 * WAVES;
	extern __shared__ __align__(16) char lds_raw[];
	using L = AttnLdsF32<D, KT>;
	float* const lds_base = reinterpret_cast<float*>(lds_raw);
	typedef __attribute__((address_space(3))) void lds_void;
	typedef const __attribute__((address_space(1))) void global_void;
	constexpr int KS = D / 16;                      // 16-element groups of the head dimension (q k^T: 4 MFMAs each)
	constexpr int DC = D / 64;                      // 64-wide column groups of the output (4 accumulators each)
	constexpr int KB = kKeysPerTile / 16;           // 16-key blocks per tile
	constexpr int VPR = D / 4;                      // 16-byte vectors per row
	constexpr int VPT = kKeysPerTile * VPR / THREADS;   // vectors per thread per tile and matrix
	static_assert(kKeysPerTile * VPR % THREADS == 0, "the tile divides over the threads");

	const int tid = threadIdx.x;
	const int lane = tid & (kWaveSize - 1);
	const int wave = tid >> 6;
	const int n = lane & 15;                        // query inside the wave's block (second MFMA operand index)
	const int g = lane >> 4;                        // lane group: summation slot g of an MFMA
	int bh, q_block, part, parts, split_slot;
	if (!attn_walk_locate_part(walk, blockIdx.x, bh, q_block, part, parts, split_slot)) return;       // the whole block
	const int q0 = q_block * kQueriesPerBlock;
	const float* qp = a.q + (int64_t)bh * a.n_q * D;
	const float* kp = a.k + (int64_t)(bh / a.q_per_kv) * a.n_k * D;
	const float* vp = a.v + (int64_t)(bh / a.q_per_kv) * a.n_k * D;
	float* yp = a.y + (int64_t)bh * a.n_q * D;

	// visible key range of the whole block: from the first key of its first query to the last of its last
	const int q_last = (q0 + kQueriesPerBlock - 1 < a.n_q ? q0 + kQueriesPerBlock - 1 : a.n_q - 1);
	int key_hi = a.n_k - 1;
	if (a.causal && q_last + a.diag < key_hi) key_hi = q_last + a.diag;
	int key_lo = 0;
	if (a.window > 0 && q0 + a.diag - a.window + 1 > 0) key_lo = q0 + a.diag - a.window + 1;
	int t_first = key_lo / kKeysPerTile;
	int t_last = key_hi >= 0 ? key_hi / kKeysPerTile : -1;
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

	// this lane's query as second operand: q[row][16 s + 4 g .. + 3]
	const int q_row = q0 + 16 * wave + n;
	float4_t qf[KS];
#pragma unroll
	for (int s = 0; s < KS; ++s)
	{
		float4_t val = {0.0f, 0.0f, 0.0f, 0.0f};
		if (q_row < a.n_q) val = *reinterpret_cast<const float4_t*>(qp + (int64_t)q_row * D + 16 * s + 4 * g);
		qf[s] = val;
	}
	int vis_hi = a.causal ? q_row + a.diag : a.n_k - 1;
	if (vis_hi > a.n_k - 1) vis_hi = a.n_k - 1;
	const int vis_lo = a.window > 0 ? q_row + a.diag - a.window + 1 : 0;

	float m_run = -INFINITY, l_run = 0.0f;         // l_run: this lane's share of the row sum
	float4_t o[DC][4];
#pragma unroll
	for (int c = 0; c < DC; ++c)
#pragma unroll
		for (int e = 0; e < 4; ++e) o[c][e] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
	// keys visible to every query of this wave need no per-element test: [all_lo, all_hi]
	const int wq0 = q0 + 16 * wave, wq1 = wq0 + 15;
	const int all_hi = a.causal ? (wq0 + a.diag < a.n_k - 1 ? wq0 + a.diag : a.n_k - 1) : a.n_k - 1;
	const int all_lo = a.window > 0 ? wq1 + a.diag - a.window + 1 : 0;

	// DIRECT: wave w moves rows w, w + WAVES, ... of the K tile and of the V tile; rows past the last key are
	// replaced by the last one (their scores are masked, their p is 0)
	auto tile_direct = [&](int t, int stage) {
		float* k_dst = lds_base + stage * L::kStageFloats;
		float* v_dst = k_dst + kKeysPerTile * L::kPitch;
		const int w = __builtin_amdgcn_readfirstlane(wave);
#pragma unroll
		for (int i = 0; i < kKeysPerTile / WAVES; ++i)
		{
			const int row = w + WAVES * i;
			int key = t * kKeysPerTile + row;
			key = key < a.n_k ? key : a.n_k - 1;
			__builtin_amdgcn_global_load_lds((global_void*)(kp + (int64_t)key * D + 4 * lane), (lds_void*)(k_dst + row * L::kPitch), 16, 0, 0);
			__builtin_amdgcn_global_load_lds((global_void*)(vp + (int64_t)key * D + 4 * lane), (lds_void*)(v_dst + row * L::kPitch), 16, 0, 0);
		}
	};

	float4_t kr[DIRECT ? 1 : VPT], vr[DIRECT ? 1 : VPT];
	auto tile_load = [&](int t) {
#pragma unroll
		for (int i = 0; i < (DIRECT ? 0 : VPT); ++i)
		{
			const int idx = tid + THREADS * i;
			const int row = idx / VPR, col = idx % VPR;
			const int key = t * kKeysPerTile + row;
			float4_t kv = {0.0f, 0.0f, 0.0f, 0.0f}, vv = {0.0f, 0.0f, 0.0f, 0.0f};
			if (key < a.n_k)
			{
				kv = *reinterpret_cast<const float4_t*>(kp + (int64_t)key * D + col * 4);
				vv = *reinterpret_cast<const float4_t*>(vp + (int64_t)key * D + col * 4);
			}
			kr[i] = kv;
			vr[i] = vv;
		}
	};
	auto tile_store = [&]() {
		float* k_dst = lds_base;
		float* v_dst = k_dst + kKeysPerTile * L::kPitch;
#pragma unroll
		for (int i = 0; i < (DIRECT ? 0 : VPT); ++i)
		{
			const int idx = tid + THREADS * i;
			const int row = idx / VPR, col = idx % VPR;
			*reinterpret_cast<float4_t*>(k_dst + row * L::kPitch + col * 4) = kr[i];
			*reinterpret_cast<float4_t*>(v_dst + row * L::kPitch + col * 4) = vr[i];
		}
	};

	// MASK: the mask values of this lane's scores of tile t, times log2(e): four consecutive floats per key block, at any
	// alignment; keys past the end and rows past the last query read nothing (their scores are masked by the rules)
	float4_t mk_next[MASK ? KB : 1];
	auto load_mask = [&](float4_t (&dst)[MASK ? KB : 1], int t) {
		typedef float4_t LooseF4 __attribute__((aligned(4)));
#pragma unroll
		for (int kb = 0; kb < (MASK ? KB : 0); ++kb)
		{
			const int key = t * kKeysPerTile + 16 * kb + 4 * g;
			float4_t val = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
			if (q_row < a.n_q)
			{
				const float* src = a.mask + (int64_t)q_row * a.mask_stride + key;
				if (key + 3 < a.n_k) val = *reinterpret_cast<const LooseF4*>(src) * kLog2e;
				else
				{
#pragma unroll
					for (int r = 0; r < 4; ++r)
						if (key + r < a.n_k) val[r] = src[r] * kLog2e;
				}
			}
			dst[kb] = val;
		}
	};
	// MASK: the walk visits the tiles that the map has set (all of them without a map); t_next is the tile after t on
	// that walk, the stages alternate along it
	if constexpr (MASK) t_first = attention_next_visible_tile(map_row, t_first, t_last);
	if (t_first <= t_last)
	{
		if constexpr (MASK) load_mask(mk_next, t_first);
		if constexpr (DIRECT) tile_direct(t_first, 0);
		else tile_load(t_first);
	}
	int t_next = 0, stage_m = 0;
	for (int t = t_first; t <= t_last; t = MASK ? t_next : t + 1, stage_m ^= 1)
	{
		const float* k_lds = lds_base;
		const int stage = MASK ? stage_m : (t - t_first) & 1;
		if constexpr (MASK) t_next = attention_next_visible_tile(map_row, t + 1, t_last);
		else t_next = t + 1;
		if constexpr (DIRECT)
		{
			// own loads of tile t have landed; behind the barrier everybody's have, and everybody is done with the
			// stage of the tile before, which the loads of the next tile overwrite
			wait_vmem_all();
			__syncthreads();
			if (t_next <= t_last) tile_direct(t_next, stage ^ 1);
			k_lds = lds_base + stage * L::kStageFloats;
		}
		else
		{
			__syncthreads();                       // the previous tile has been read by everybody
			tile_store();
			__syncthreads();
			if (t_next <= t_last) tile_load(t_next);      // in flight while this tile is used
		}
		const float* v_lds = k_lds + kKeysPerTile * L::kPitch;

		// the mask values of this lane's scores of the tile (log2 domain) were requested a tile ahead; those of the next
		// tile go out now.  A tile in which the mask hides every key from every query of the wave costs the wave nothing
		// further (under a causal mask tensor that is half of the tiles).
		float4_t mk[MASK ? KB : 1];
		if constexpr (MASK)
		{
			bool any_visible = false;
#pragma unroll
			for (int kb = 0; kb < KB; ++kb)
			{
				mk[kb] = mk_next[kb];
#pragma unroll
				for (int r = 0; r < 4; ++r) any_visible |= mk[kb][r] > -INFINITY;
			}
			if (t_next <= t_last) load_mask(mk_next, t_next);
			if (__builtin_amdgcn_ballot_w64(any_visible) == 0) continue;
		}

		// ---- S^T = K Q^T: s[kb][r] = score of key 16 kb + 4 g + r against this lane's query ----
		// The K vectors of step st + 1 are read from LDS before the MFMAs of step st are issued (the scheduling
		// groups pin that order: left alone the compiler puts every read right in front of its first use and the
		// matrix pipe drains while the wave waits for LDS).
		float4_t s[KB];
#pragma unroll
		for (int kb = 0; kb < KB; ++kb) s[kb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
		float4_t kf[2][KB];
		auto read_k = [&](float4_t (&dst)[KB], int st) {
#pragma unroll
			for (int kb = 0; kb < KB; ++kb)
				dst[kb] = *reinterpret_cast<const float4_t*>(k_lds + (16 * kb + n) * L::kPitch + 16 * st + 4 * g);
		};
		read_k(kf[0], 0);
		__builtin_amdgcn_sched_group_barrier(kSchedDsRead, KB, 0);
#pragma unroll
		for (int st = 0; st < KS; ++st)
		{
			if (st + 1 < KS) read_k(kf[(st + 1) & 1], st + 1);
#pragma unroll
			for (int e = 0; e < 4; ++e)
#pragma unroll
				for (int kb = 0; kb < KB; ++kb)
					s[kb] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[st & 1][kb][e], qf[st][e], s[kb], 0, 0, 0);
			// the reads go out behind the step's first MFMA: the wait in front of that MFMA then covers exactly the
			// vectors it needs, not the ones just requested
			__builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
			if (st + 1 < KS) __builtin_amdgcn_sched_group_barrier(kSchedDsRead, KB, 0);
			__builtin_amdgcn_sched_group_barrier(kSchedMfma, 4 * KB - 1, 0);
		}

		// ---- online softmax ----
		const int tile_key0 = t * kKeysPerTile;
		const bool interior = tile_key0 >= all_lo && tile_key0 + kKeysPerTile - 1 <= all_hi;   // wave-uniform
		float z[KB][4];
		float mt = -INFINITY;
		if (interior && !MASK)
		{
#pragma unroll
			for (int kb = 0; kb < KB; ++kb)
#pragma unroll
				for (int r = 0; r < 4; ++r)
				{
					z[kb][r] = logit2<SOFTCAP>(s[kb][r], a.k_in, a.k_cap);
					mt = fmaxf(mt, z[kb][r]);
				}
		}
		else
		{
#pragma unroll
			for (int kb = 0; kb < KB; ++kb)
#pragma unroll
				for (int r = 0; r < 4; ++r)
				{
					const int key = tile_key0 + 16 * kb + 4 * g + r;
					const float zz = logit2<SOFTCAP>(s[kb][r], a.k_in, a.k_cap) + (MASK ? mk[MASK ? kb : 0][r] : 0.0f);
					z[kb][r] = (key >= vis_lo && key <= vis_hi) ? zz : -INFINITY;
					mt = fmaxf(mt, z[kb][r]);
				}
		}
		mt = max_over_lane_rows(mt);
		const float m_new = fmaxf(m_run, mt);
		const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;   // nothing visible so far: every term is exp2(-inf) = 0
		float psum = 0.0f;
		float p[KB][4];
#pragma unroll
		for (int kb = 0; kb < KB; ++kb)
#pragma unroll
			for (int r = 0; r < 4; ++r)
			{
				p[kb][r] = fast_exp2(z[kb][r] - m_safe);
				psum += p[kb][r];
			}
		// the running maximum settles after a few tiles; when no query of the wave raised it, the rescale
		// factor is 1 everywhere and the pass over the accumulators is skipped
		if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0)
		{
			const float corr = fast_exp2(m_run - m_safe);
			l_run *= corr;
#pragma unroll
			for (int c = 0; c < DC; ++c)
#pragma unroll
				for (int e = 0; e < 4; ++e) o[c][e] *= corr;
		}
		l_run += psum;
		m_run = m_new;

		// ---- O^T += V^T P^T, the V vectors of key slot i + 1 read before the MFMAs of slot i ----
		float4_t vf[2][DC];
		auto read_v = [&](float4_t (&dst)[DC], int slot) {
			const int kb = slot >> 2, r = slot & 3;
#pragma unroll
			for (int c = 0; c < DC; ++c)
				dst[c] = *reinterpret_cast<const float4_t*>(v_lds + (16 * kb + 4 * g + r) * L::kPitch + 64 * c + 4 * n);
		};
		read_v(vf[0], 0);
		__builtin_amdgcn_sched_group_barrier(kSchedDsRead, DC, 0);
#pragma unroll
		for (int slot = 0; slot < 4 * KB; ++slot)
		{
			if (slot + 1 < 4 * KB) read_v(vf[(slot + 1) & 1], slot + 1);
#pragma unroll
			for (int c = 0; c < DC; ++c)
#pragma unroll
				for (int e = 0; e < 4; ++e)
					o[c][e] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[slot & 1][c][e], p[slot >> 2][slot & 3], o[c][e], 0, 0, 0);
			__builtin_amdgcn_sched_group_barrier(kSchedMfma, 1, 0);
			if (slot + 1 < 4 * KB) __builtin_amdgcn_sched_group_barrier(kSchedDsRead, DC, 0);
			__builtin_amdgcn_sched_group_barrier(kSchedMfma, 4 * DC - 1, 0);
		}
	}

	// ---- normalise and store: register r of accumulator (c, e) is y[row][64 c + 4 (4 g + r) + e] ----
	float l = l_run;
	l += __shfl_xor(l, 16);
	l += __shfl_xor(l, 32);
	if (parts > 1)
	{
		// unnormalised accumulators, running maximum and sum of this half of the keys
		if (q_row < a.n_q)
		{
			float* dst = a.partials + ((((int64_t)bh * walk.n_split + split_slot) * parts + part) * kQueriesPerBlock + (q_row - q0)) * (D + 2);
#pragma unroll
			for (int c = 0; c < DC; ++c)
#pragma unroll
				for (int r = 0; r < 4; ++r)
					*reinterpret_cast<WsFloat4*>(dst + 64 * c + 16 * g + 4 * r) = float4_t{o[c][0][r], o[c][1][r], o[c][2][r], o[c][3][r]};
			if (g == 0)
			{
				dst[D] = m_run;
				dst[D + 1] = l;
			}
		}
		return;
	}
	const float inv = l > 0.0f ? 1.0f / l : 0.0f;
	if (q_row < a.n_q)
	{
#pragma unroll
		for (int c = 0; c < DC; ++c)
#pragma unroll
			for (int r = 0; r < 4; ++r)
			{
				const float4_t out = {o[c][0][r] * inv, o[c][1][r] * inv, o[c][2][r] * inv, o[c][3][r] * inv};
				*reinterpret_cast<float4_t*>(yp + (int64_t)q_row * D + 64 * c + 16 * g + 4 * r) = out;
			}
	}
}

template <int D, bool SOFTCAP, bool MASK>
hipError_t launch_variant_f32(const AttnArgsF32& args_in, int64_t batch_heads, hipStream_t stream)
{
	// head dimension 256: 8 waves (two per SIMD) on tiles of 32 keys in two stages, 130 KB, one block per CU.  Two
	// alternatives with two blocks of 4 waves per CU, for a better balance of long and short blocks under the causal
	// rule, measured 5 - 12 % slower: tiles of 16 keys, and one K and one V buffer refilled in turn.
	constexpr bool DIRECT = (D == 256);
	constexpr int WAVES = DIRECT ? 8 : 4;
	constexpr int KT = DIRECT ? 32 : 64;
	auto kernel = sdp_attention_fwd_f32_kernel<D, SOFTCAP, WAVES, KT, DIRECT, MASK>;
	constexpr int kLdsBytes = AttnLdsF32<D, KT>::kStageFloats * 4 * (DIRECT ? 2 : 1);
	constexpr int kQueriesPerBlock = 16 * WAVES;
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
	AttnArgsF32 args = args_in;
	const int64_t q_blocks = (args.n_q + kQueriesPerBlock - 1) / kQueriesPerBlock;
	args.tile_map = nullptr;
	args.map_words = 0;
	std::optional<band::WorkspaceReserve> map_hold;
	bool mask_two_parts = false;
	if constexpr (MASK)
	{
		// The visible-tile map of the mask, at the front of the stream's workspace (the partial results of a split key
		// range go behind it): worth its pass over the mask for large masks and long key ranges
		// (attention_mask_map_wanted), and left out where the stream has no workspace to offer (a capture without a
		// caller's workspace).  For whole query blocks the results are the same bit for bit: the map only saves the loads
		// and barriers of tiles that every wave of a block would skip.
		const int64_t words = attention_tile_map_words(args.n_k, KT);
		const size_t map_bytes = (size_t)(q_blocks * words) * sizeof(unsigned long long);
		// With as many blocks as one to four rounds of the chip the rounds do not even out where the mask leaves the
		// blocks unequal shares of their key range (a sliding window: the late query blocks carry the full window, the
		// early ones little): every block then goes out in two parts, each with half of its VISIBLE tiles.  Their
		// partial results may take more than the library's own workspace holds to begin with; it grows for them as
		// it does for operand copies (eager launches only), before anything points into it.
		const int64_t blocks = q_blocks * batch_heads;
		const int cus = device_cu_count();
		size_t two_parts_bytes = 0;
		if (blocks >= cus && blocks < 4 * (int64_t)cus && (args.n_k + KT - 1) / KT >= 32)
			two_parts_bytes = (size_t)2 * blocks * kQueriesPerBlock * (D + 2) * sizeof(float);
		const size_t map_room = (map_bytes + 255) / 256 * 256 + (1u << 16);
		if (two_parts_bytes > 0 && band::workspace_copy_capacity(stream) < map_room + two_parts_bytes) two_parts_bytes = 0;
		if (attention_mask_map_wanted(args.n_q, args.n_k) && (two_parts_bytes > 0 || band::workspace_capacity(stream) >= map_room))
		{
			float* front = nullptr;
			hipError_t e = band::workspace_acquire(stream, &front, two_parts_bytes > 0 ? map_room + two_parts_bytes : 0);
			if (e != hipSuccess) return e;
			mask_two_parts = two_parts_bytes > 0;
			unsigned long long* map = reinterpret_cast<unsigned long long*>(front);
			e = launch_attention_mask_tile_map(args.mask, args.mask_stride, args.n_q, args.n_k, kQueriesPerBlock, KT, map, stream);
			if (e != hipSuccess) return e;
			args.tile_map = map;
			args.map_words = (int)words;
			map_hold.emplace(map_bytes);
		}
	}
	const AttnSplitPlan plan = plan_attention_split(args.n_q, args.n_k, args.causal, args.diag, args.window, batch_heads,
	                                                kQueriesPerBlock, KT, D, band::workspace_capacity(stream));
	// (or, with too few query blocks for the chip, every block in several parts of its key range)
	int64_t parts_all = plan.n_split > 0 ? 1 : plan_attention_parts(args.n_q, args.n_k, args.causal, args.diag, batch_heads, kQueriesPerBlock,
	                                                                  KT, D, band::workspace_capacity(stream));
	if (mask_two_parts && plan.n_split == 0 && parts_all == 1) parts_all = 2;
	args.partials = nullptr;
	if (plan.n_split > 0 || parts_all > 1)
	{
		const hipError_t ws_err = band::workspace_acquire(stream, &args.partials);
		if (ws_err != hipSuccess) return ws_err;
	}
	const AttnWalk walk = make_attn_walk(q_blocks, batch_heads, args.q_per_kv, plan.n_split, plan.n_big, parts_all);
	if (attn_walk_blocks(walk) > 0x7FFFFFFFLL) return hipErrorInvalidValue;
	kernel<<<dim3((unsigned)attn_walk_blocks(walk)), dim3(64 * WAVES), kLdsBytes, stream>>>(args, walk);
	const hipError_t err = hipGetLastError();
	if (err != hipSuccess || walk.n_split == 0) return err;
	const int64_t items = batch_heads * walk.n_split * kQueriesPerBlock * (D / 4);
	sdp_attention_merge_halves_kernel<D, float><<<dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream>>>(
		args.partials, args.y, args.n_q, (int)q_blocks, walk.n_split, kQueriesPerBlock, parts_all > 1 ? (int)parts_all : 2);
	return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// Decode form: very few queries per head (a generation step), long key range: the KEYS are split.
//
// The q_per_kv query heads that share a key / value head, times the n_q queries of each, are the (at most 16)
// rows of one 16-query MFMA block, so K and V of a head are read once for all of them.  Pass 1: one wave per
// (key / value head, split of the visible key range) walks its keys in tiles of 16.  Both operands come straight
// from global memory in MFMA operand layout, no LDS: the K vectors as in the fused kernel, and the V vectors with
// the permuted accumulators described at the top (a lane loads four consecutive columns of a V row).  The wave
// leaves its running maximum, sum and unnormalised accumulators in the workspace.  Pass 2 merges the splits of a
// row: M = max m_i, y = sum o_i 2^(m_i - M) / sum l_i 2^(m_i - M).
// Workspace per (head, split, row): head_dim accumulators + maximum + sum, fp32.
// ---------------------------------------------------------------------------------------------
constexpr int kDecodeKeysPerTile = 16;

struct DecodeArgsF32
{
	AttnArgsF32 a;
	float* ws;              // [kv_heads][splits][rows][D + 2]
	int rows;               // q_per_kv * n_q
	int groups;             // of 16 rows: a wave each
	int splits;
	int tiles_per_split;
	int t_first, t_last;    // visible key tiles of the group
};

template <int D, bool SOFTCAP>
__global__ __launch_bounds__(64) void sdp_decode_partial_f32_kernel(const DecodeArgsF32 da)
{
	const AttnArgsF32& a = da.a;
	constexpr int KS = D / 16, DC = D / 64;
	const int lane = threadIdx.x;
	const int n = lane & 15, g = lane >> 4;
	int split, group;
	if (!decode_locate(da.groups, da.splits, split, group)) return;
	const int kvh = blockIdx.y;
	const float* qp = a.q + (int64_t)kvh * da.rows * D;  // the rows of a key / value head are contiguous: [q_per_kv][n_q][D]
	const int row = kDecodeRowsPerWave * group + n;        // this lane's row among them
	const float* kp = a.k + (int64_t)kvh * a.n_k * D;
	const float* vp = a.v + (int64_t)kvh * a.n_k * D;

	const bool row_ok = row < da.rows;
	const int q_idx = row_ok ? row % a.n_q : 0;             // position of this lane's row among the n_q queries
	float4_t qf[KS];
#pragma unroll
	for (int s = 0; s < KS; ++s)
	{
		float4_t val = {0.0f, 0.0f, 0.0f, 0.0f};
		if (row_ok) val = *reinterpret_cast<const float4_t*>(qp + (int64_t)row * D + 16 * s + 4 * g);
		qf[s] = val;
	}
	int vis_hi = a.causal ? q_idx + a.diag : a.n_k - 1;
	if (vis_hi > a.n_k - 1) vis_hi = a.n_k - 1;
	if (!row_ok) vis_hi = -1;                              // padding rows see nothing
	const int vis_lo = a.window > 0 ? q_idx + a.diag - a.window + 1 : 0;

	float m_run = -INFINITY, l_run = 0.0f;
	float4_t o[DC][4];
#pragma unroll
	for (int c = 0; c < DC; ++c)
#pragma unroll
		for (int e = 0; e < 4; ++e) o[c][e] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

	const int t0 = da.t_first + split * da.tiles_per_split;
	int t1 = t0 + da.tiles_per_split - 1;
	if (t1 > da.t_last) t1 = da.t_last;
	// All loads of a tile are issued before the first use; keys past the end are replaced by the last one (their
	// scores are masked).  A K load instruction covers half of each 128-byte line it touches, so it stays a plain
	// load (the other half is the next instruction's); a V load covers whole lines and is non-temporal.
	auto fetch = [&](float4_t (&kd)[KS], float4_t (&vd)[4][DC], int key0) {
		{
			int key = key0 + n;
			key = key < a.n_k ? key : a.n_k - 1;
#pragma unroll
			for (int st = 0; st < KS; ++st) kd[st] = *reinterpret_cast<const float4_t*>(kp + (int64_t)key * D + 16 * st + 4 * g);
		}
#pragma unroll
		for (int r = 0; r < 4; ++r)
		{
			int key = key0 + 4 * g + r;
			key = key < a.n_k ? key : a.n_k - 1;
#pragma unroll
			for (int c = 0; c < DC; ++c)
				vd[r][c] = __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(vp + (int64_t)key * D + 64 * c + 4 * n));
		}
	};
	auto consume = [&](const float4_t (&kd)[KS], const float4_t (&vd)[4][DC], int key0) {
		float4_t s = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
		for (int st = 0; st < KS; ++st)
#pragma unroll
			for (int e = 0; e < 4; ++e) s = __builtin_amdgcn_mfma_f32_16x16x4f32(kd[st][e], qf[st][e], s, 0, 0, 0);

		float z[4];
		float mt = -INFINITY;
#pragma unroll
		for (int r = 0; r < 4; ++r)
		{
			const int key = key0 + 4 * g + r;
			const float zz = logit2<SOFTCAP>(s[r], a.k_in, a.k_cap);
			z[r] = (key >= vis_lo && key <= vis_hi) ? zz : -INFINITY;
			mt = fmaxf(mt, z[r]);
		}
		mt = max_over_lane_rows(mt);
		const float m_new = fmaxf(m_run, mt);
		const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
		const float corr = fast_exp2(m_run - m_safe);
		float psum = 0.0f;
		float p[4];
#pragma unroll
		for (int r = 0; r < 4; ++r)
		{
			p[r] = fast_exp2(z[r] - m_safe);
			psum += p[r];
		}
		l_run = l_run * corr + psum;
		m_run = m_new;
#pragma unroll
		for (int c = 0; c < DC; ++c)
#pragma unroll
			for (int e = 0; e < 4; ++e) o[c][e] *= corr;
#pragma unroll
		for (int r = 0; r < 4; ++r)
#pragma unroll
			for (int c = 0; c < DC; ++c)
#pragma unroll
				for (int e = 0; e < 4; ++e) o[c][e] = __builtin_amdgcn_mfma_f32_16x16x4f32(vd[r][c][e], p[r], o[c][e], 0, 0, 0);
	};
	if constexpr (D <= 128)
	{
		// two register buffers: the loads of tile t + 1 are in flight while tile t is multiplied (at head_dim 256 a
		// second buffer does not fit beside the accumulators)
		float4_t kf[2][KS], vf[2][4][DC];
		if (t0 <= t1) fetch(kf[0], vf[0], t0 * kDecodeKeysPerTile);
		for (int t = t0; t <= t1; t += 2)
		{
			if (t + 1 <= t1) fetch(kf[1], vf[1], (t + 1) * kDecodeKeysPerTile);
			__builtin_amdgcn_sched_barrier(0);
			consume(kf[0], vf[0], t * kDecodeKeysPerTile);
			if (t + 1 <= t1)
			{
				if (t + 2 <= t1) fetch(kf[0], vf[0], (t + 2) * kDecodeKeysPerTile);
				__builtin_amdgcn_sched_barrier(0);
				consume(kf[1], vf[1], (t + 1) * kDecodeKeysPerTile);
			}
		}
	}
	else
	{
		for (int t = t0; t <= t1; ++t)
		{
			float4_t kf[KS], vf[4][DC];
			fetch(kf, vf, t * kDecodeKeysPerTile);
			consume(kf, vf, t * kDecodeKeysPerTile);
		}
	}

	// partial result of this split: register r of accumulator (c, e) is o[row n][64 c + 16 g + 4 r + e]
	float l = l_run;
	l += __shfl_xor(l, 16);
	l += __shfl_xor(l, 32);
	if (row_ok)
	{
		float* dst = da.ws + (((int64_t)kvh * da.splits + split) * da.rows + row) * (D + 2);
#pragma unroll
		for (int c = 0; c < DC; ++c)
#pragma unroll
			for (int r = 0; r < 4; ++r)
				*reinterpret_cast<WsFloat4*>(dst + 64 * c + 16 * g + 4 * r) = float4_t{o[c][0][r], o[c][1][r], o[c][2][r], o[c][3][r]};
		if (g == 0)
		{
			dst[D] = m_run;
			dst[D + 1] = l;
		}
	}
}

template <int D, bool SOFTCAP>
hipError_t launch_decode_variant_f32(const DecodeArgsF32& da, int64_t kv_heads, hipStream_t stream)
{
	(void)hipGetLastError();
	sdp_decode_partial_f32_kernel<D, SOFTCAP><<<dim3(decode_blocks(da.groups, da.splits), (unsigned)kv_heads), dim3(64), 0, stream>>>(da);
	hipError_t e = hipGetLastError();
	if (e != hipSuccess) return e;
	sdp_decode_merge_kernel<D, float><<<dim3((unsigned)da.rows, (unsigned)kv_heads), dim3(256), 0, stream>>>(da.ws, da.a.y, da.rows, da.splits);
	return hipGetLastError();
}

}  // namespace

bool sdp_attention_fwd_f32_supports(int64_t head_dim)
{
	return head_dim == 64 || head_dim == 128 || head_dim == 256;
}

hipError_t launch_sdp_attention_fwd_f32(const float* q, const float* k, const float* v, float* y,
                                        int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                        float alpha, float softcap, int causal, int64_t window, hipStream_t stream,
                                        const float* mask, int64_t mask_stride)
{
	if (batch_heads == 0 || n_q == 0) return hipSuccess;
	AttnArgsF32 args;
	args.q = q;
	args.k = k;
	args.v = v;
	args.y = y;
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
	args.mask = mask;
	args.mask_stride = mask_stride;
#define ANYGPU_ATTN_F32_DIM(DIM) \
	if (mask != nullptr) \
		return capped ? launch_variant_f32<DIM, true, true>(args, batch_heads, stream) : launch_variant_f32<DIM, false, true>(args, batch_heads, stream); \
	return capped ? launch_variant_f32<DIM, true, false>(args, batch_heads, stream) : launch_variant_f32<DIM, false, false>(args, batch_heads, stream)
	switch (head_dim)
	{
	case 64: ANYGPU_ATTN_F32_DIM(64);
	case 128: ANYGPU_ATTN_F32_DIM(128);
	default: ANYGPU_ATTN_F32_DIM(256);
	}
#undef ANYGPU_ATTN_F32_DIM
}

bool sdp_attention_decode_f32_supports(int64_t q_per_kv, int64_t n_q, int64_t head_dim)
{
	return sdp_attention_fwd_f32_supports(head_dim) && q_per_kv >= 1 && n_q >= 1 && q_per_kv * n_q <= kDecodeMaxRows;
}

int64_t sdp_attention_decode_f32_workspace_bytes(int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                                 int causal, int64_t window)
{
	if (batch_heads == 0 || n_q == 0) return 0;
	const int64_t kv_heads = batch_heads / q_per_kv;
	const DecodePlan p = plan_decode(kv_heads * ((q_per_kv * n_q + kDecodeRowsPerWave - 1) / kDecodeRowsPerWave), n_q, n_k, causal, window, kDecodeKeysPerTile);
	return kv_heads * p.splits * (q_per_kv * n_q) * (head_dim + 2) * (int64_t)sizeof(float);
}

hipError_t launch_sdp_attention_decode_f32(const float* q, const float* k, const float* v, float* y, void* workspace,
                                           int64_t batch_heads, int64_t q_per_kv, int64_t n_q, int64_t n_k, int64_t head_dim,
                                           float alpha, float softcap, int causal, int64_t window, hipStream_t stream)
{
	if (batch_heads == 0 || n_q == 0) return hipSuccess;
	const int64_t kv_heads = batch_heads / q_per_kv;
	const DecodePlan p = plan_decode(kv_heads * ((q_per_kv * n_q + kDecodeRowsPerWave - 1) / kDecodeRowsPerWave), n_q, n_k, causal, window, kDecodeKeysPerTile);
	DecodeArgsF32 da;
	da.a.q = q;
	da.a.k = k;
	da.a.v = v;
	da.a.y = y;
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
#define ANYGPU_DECODE_F32_DIM(DIM) \
	return capped ? launch_decode_variant_f32<DIM, true>(da, kv_heads, stream) : launch_decode_variant_f32<DIM, false>(da, kv_heads, stream)
	switch (head_dim)
	{
	case 64: ANYGPU_DECODE_F32_DIM(64);
	case 128: ANYGPU_DECODE_F32_DIM(128);
	default: ANYGPU_DECODE_F32_DIM(256);
	}
#undef ANYGPU_DECODE_F32_DIM
}

}  // namespace anygpu
