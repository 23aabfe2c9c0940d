// Row softmax for gfx950 with the attention prologue (scale, logit softcap, causal and
// sliding-window masks) fused in.  HBM-bound: every visible input element is read once and
// every output element written once, with 16-byte accesses.
//
// Fast kernel: one wave owns one row and keeps it in registers (VPL 16-byte vectors per
// lane), runs an online max/sum over the vectors as they arrive, combines the 64 lane
// states with DPP reductions, then normalises from registers.  Vectors that lie wholly
// outside the visible key interval [lo, hi] of the row are never loaded; their outputs are
// stored as zeros.
// Short rows (up to 64 vectors) share a wave four at a time; rows longer than a block's registers hold are walked
// twice by a block of 1024 threads with 16-byte accesses, at any width, stride or alignment.
// An additive mask tensor [q_len, cols] shared by the heads of a batch is read with ordinary (cached) loads, and the
// blocks are dealt so that the heads of a mask row run side by side on one XCD (block_rows).
#include "device_utils.hpp"
#include "launch.hpp"

#include <algorithm>

namespace anygpu {

struct SoftmaxArgs
{
	const void* x;
	void* y;
	int64_t rows, cols;
	int64_t xs, ys;        // row strides, elements
	int64_t q_len, diag;
	float alpha;
	float inv_cap;         // 1 / softcap, 0 when the softcap is off
	float cap_log2e;       // softcap * log2(e)
	float alpha_log2e;     // alpha * log2(e), used when the softcap is off
	int causal;
	int64_t window;
	const void* mask;      // optional additive mask [q_len, cols] of the element type (NULL: none)
	int64_t mask_stride;   // elements between mask rows
	int heads;             // > 1: rows = heads x q_len share the mask rows and the blocks are dealt as block_rows() says
};

template <typename T> struct Vec16;
template <> struct Vec16<half_t> { using type = half8_t; };
template <> struct Vec16<float> { using type = float4_t; };

// Query index of a row: which mask row / causal diagonal it belongs to.
__device__ __forceinline__ int64_t query_of_row(const SoftmaxArgs& a, int64_t row)
{
	return a.q_len > 0 ? (int64_t)((uint32_t)row % (uint32_t)a.q_len) : row;
}

// First row of a block that works on `per_block` consecutive rows, or -1 for a block without rows.  Plain: block b
// takes rows b * per_block on.  With a mask tensor shared by `heads` heads (rows = heads x q_len, row = head * q_len +
// query) the blocks that read one mask row should run at the same time on the same XCD, so that the row comes out of
// that XCD's L2 for all heads but one: consecutive blocks go to the eight XCDs in turn, so block b = 8 s + x takes head
// s % heads of query group 8 (s / heads) + x, and the launch has ceil(groups / 8) * 8 * heads blocks.
__device__ __forceinline__ int64_t block_rows(const SoftmaxArgs& a, int per_block, int64_t* rows_end)
{
	if (a.heads <= 1)
	{
		*rows_end = a.rows;
		return (int64_t)blockIdx.x * per_block;
	}
	const uint32_t x = blockIdx.x % 8u, slot = blockIdx.x / 8u;
	const uint32_t head = slot % (uint32_t)a.heads;
	const int64_t group = (int64_t)(slot / (uint32_t)a.heads) * 8 + x;
	const int64_t q0 = group * per_block;
	*rows_end = (int64_t)(head + 1) * a.q_len;
	return q0 < a.q_len ? (int64_t)head * a.q_len + q0 : -1;
}

// blocks of such a launch
static inline unsigned blocks_for_rows(const SoftmaxArgs& a, int per_block)
{
	if (a.heads <= 1) return (unsigned)((a.rows + per_block - 1) / per_block);
	const int64_t groups = (a.q_len + per_block - 1) / per_block;
	return (unsigned)((groups + 7) / 8 * 8 * a.heads);
}

// Visible key interval of a row, inclusive on both ends; empty when hi < lo.
struct RowSpan { int64_t lo, hi; };

__device__ __forceinline__ RowSpan row_span(const SoftmaxArgs& a, int64_t row)
{
	const int64_t i = query_of_row(a, row);   // rows and q_len fit 32 bits (checked by the entry point)
	RowSpan s;
	s.hi = a.cols - 1;
	s.lo = 0;
	if (a.causal) s.hi = min(s.hi, i + a.diag);
	if (a.window > 0) s.lo = max(s.lo, i + a.diag - a.window + 1);
	s.hi = max(s.hi, (int64_t)-1);
	s.lo = min(s.lo, a.cols);
	return s;
}

// Logit in the log2 domain: log2(e) * softcap(alpha * x).
__device__ __forceinline__ float logit2(const SoftmaxArgs& a, float x)
{
	if (a.inv_cap != 0.0f)
	{
		return a.cap_log2e * tanh_f32(x * a.alpha * a.inv_cap);
	}
	return x * a.alpha_log2e;
}

// Running (max, sum) state of the online softmax, in the log2 domain.
struct OnlineState
{
	float m = -INFINITY;
	float s = 0.0f;
};

// exp2(a - b) where b is the running maximum: b = -inf only while nothing finite was seen,
// in which case a is -inf as well and the term must be 0, not NaN.
__device__ __forceinline__ float exp2_shift(float a, float b)
{
	return fast_exp2(a - (b == -INFINITY ? 0.0f : b));
}

// LOOSE: rows may start at any element (not only at 16-byte boundaries) and cols need not be a multiple of
// the vector length.  Vector accesses then go out at element alignment (global memory takes them; the
// compiler is told through the type) and the last, partial vector of a row is moved element by element.
// GROUP: threads that share a row: 16 (a row of lanes per row, four rows per wave and sixteen per block, for rows of up
// to 64 vectors: a wave per row would leave most of its lanes without a vector and few bytes in flight), 64 (a wave per
// row, four rows per block) or 256 (the block per row, for rows longer than a wave's registers hold).
// MASK: the launch has a mask tensor; its vectors are loaded beside the row's and kept in registers like them.
template <typename T, int VPL, bool LOOSE, int GROUP, bool MASK>
__global__ __launch_bounds__(256) void softmax_rows_wave_kernel(const SoftmaxArgs a)
{
	static_assert(GROUP == 16 || GROUP == 64 || GROUP == 256, "a row of lanes, a wave or the block per row");
	constexpr int EPV = 16 / (int)sizeof(T);
	using Vec = typename Vec16<T>::type;
	typedef Vec LooseVec __attribute__((aligned(sizeof(T))));
	constexpr int kWaveSize = GROUP;               // from here on "lane" counts inside the group and strides are the group's
	__shared__ float red_m[4], red_s[4];

	const int lane = threadIdx.x & (GROUP - 1);
	int64_t rows_end;
	const int64_t first_row = block_rows(a, 256 / GROUP, &rows_end);
	const int64_t row = first_row + (GROUP == 16 ? (threadIdx.x >> 4) : GROUP == 64 ? (threadIdx.x >> 6) : 0);
	if (first_row < 0 || row >= rows_end) return;  // uniform over the group

	const RowSpan span = row_span(a, row);
	const T* __restrict__ xr = static_cast<const T*>(a.x) + row * a.xs;
	T* __restrict__ yr = static_cast<T*>(a.y) + row * a.ys;
	const int tail = LOOSE ? (int)(a.cols % EPV) : 0;             // elements of a partial last vector
	const int nvec = (int)(a.cols / EPV) + (tail ? 1 : 0);
	const int lo = (int)span.lo, hi = (int)span.hi;
	// vector v of a row: whole vectors in one access, the partial last one element by element (zeros behind it)
	auto fetch = [&](const T* base, int v) {
		Vec val = {};
		if (LOOSE && tail && v == nvec - 1)
		{
#pragma unroll
			for (int e = 0; e < EPV; ++e)
				if (e < tail) val[e] = base[(int64_t)v * EPV + e];
		}
		else if (LOOSE) val = __builtin_nontemporal_load(reinterpret_cast<const LooseVec*>(base) + v);
		else val = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(base) + v);
		return val;
	};
	auto put = [&](T* base, int v, Vec val) {
		if (LOOSE && tail && v == nvec - 1)
		{
#pragma unroll
			for (int e = 0; e < EPV; ++e)
				if (e < tail) base[(int64_t)v * EPV + e] = val[e];
		}
		else if (LOOSE) __builtin_nontemporal_store(val, reinterpret_cast<LooseVec*>(base) + v);
		else __builtin_nontemporal_store(val, reinterpret_cast<Vec*>(base) + v);
	};
	// additive mask row of this query, shared by all heads: ordinary loads, so that it stays in the caches for them
	const T* __restrict__ mrow = MASK ? static_cast<const T*>(a.mask) + query_of_row(a, row) * a.mask_stride : nullptr;
	auto fetch_mask = [&](int v) {
		Vec mv = {};
		if (LOOSE && tail && v == nvec - 1)
		{
#pragma unroll
			for (int e = 0; e < EPV; ++e)
				if (e < tail) mv[e] = mrow[(int64_t)v * EPV + e];
		}
		else if (LOOSE) mv = *(reinterpret_cast<const LooseVec*>(mrow) + v);
		else mv = *(reinterpret_cast<const Vec*>(mrow) + v);
		return mv;
	};

	Vec raw[VPL];
	Vec mraw[MASK ? VPL : 1];
#pragma unroll
	for (int t = 0; t < VPL; ++t)
	{
		const int v = lane + kWaveSize * t;
		const int e0 = v * EPV;
		const bool need = (v < nvec) && (e0 <= hi) && (e0 + EPV - 1 >= lo);
		Vec val = {};
		if (need) val = fetch(xr, v);
		raw[t] = val;
		if constexpr (MASK)
		{
			Vec mv = {};
			if (need) mv = fetch_mask(v);
			mraw[t] = mv;
		}
	}
	auto mask_of = [&](int t, float (&mk)[EPV]) {
#pragma unroll
		for (int e = 0; e < EPV; ++e) mk[e] = MASK ? (float)mraw[MASK ? t : 0][e] * kLog2e : 0.0f;   // -inf and float lowest both end at -inf
	};

	OnlineState st;
#pragma unroll
	for (int t = 0; t < VPL; ++t)
	{
		const int v = lane + kWaveSize * t;
		const int e0 = v * EPV;
		const bool need = (v < nvec) && (e0 <= hi) && (e0 + EPV - 1 >= lo);
		if (need)
		{
			float z[EPV], mk[EPV];
			mask_of(t, mk);
			float vmax = -INFINITY;
#pragma unroll
			for (int e = 0; e < EPV; ++e)
			{
				const int j = e0 + e;
				const float zz = logit2(a, (float)raw[t][e]) + mk[e];
				z[e] = (j >= lo && j <= hi) ? zz : -INFINITY;
				vmax = fmaxf(vmax, z[e]);
			}
			const float mn = fmaxf(st.m, vmax);
			float acc = st.s * exp2_shift(st.m, mn);
#pragma unroll
			for (int e = 0; e < EPV; ++e) acc += exp2_shift(z[e], mn);
			st.s = acc;
			st.m = mn;
		}
	}

	float M = GROUP == 16 ? row_allreduce(st.m, MaxOp()) : wave_allreduce(st.m, MaxOp());
	float S = GROUP == 16 ? row_allreduce(st.s * exp2_shift(st.m, M), SumOp()) : wave_allreduce(st.s * exp2_shift(st.m, M), SumOp());
	if constexpr (GROUP == 256)
	{
		const int wave = threadIdx.x >> 6;
		if ((threadIdx.x & 63) == 0)
		{
			red_m[wave] = M;
			red_s[wave] = S;
		}
		__syncthreads();
		M = fmaxf(fmaxf(red_m[0], red_m[1]), fmaxf(red_m[2], red_m[3]));
		S = 0.0f;
#pragma unroll
		for (int w = 0; w < 4; ++w) S += red_s[w] * exp2_shift(red_m[w], M);
	}
	const float inv = S > 0.0f ? 1.0f / S : 0.0f;

#pragma unroll
	for (int t = 0; t < VPL; ++t)
	{
		const int v = lane + kWaveSize * t;
		const int e0 = v * EPV;
		if (v < nvec)
		{
			Vec out = {};
			const bool need = (e0 <= hi) && (e0 + EPV - 1 >= lo);
			if (need)
			{
				float mk[EPV];
				mask_of(t, mk);
#pragma unroll
				for (int e = 0; e < EPV; ++e)
				{
					const int j = e0 + e;
					const float p = exp2_shift(logit2(a, (float)raw[t][e]) + mk[e], M) * inv;
					out[e] = (T)((j >= lo && j <= hi) ? p : 0.0f);
				}
			}
			put(yr, v, out);
		}
	}
}

// ---------------------------------------------------------------------------------------------
// fp16 fast kernel.  One wave per row, the VISIBLE part of the row in registers: lane l owns the
// 16-byte vectors 64 (c_lo + t) + l (t < VPL), where c_lo is the 64-vector chunk of the row that
// holds the first visible key, so a sliding window of W keys needs (W / 8 + 63) / 64 + 1 vectors per
// lane however long the row is.  Vectors without a visible key are never loaded; they are stored as zeros.
//
// One pass over the registers runs the online max/sum recurrence per vector and leaves
// e = exp2(z - m_t) (m_t = running maximum after vector t) in the registers as halves, in place
// of the input; the sum is accumulated in fp32 from the unrounded values.  After the DPP
// reductions a second pass over the registers multiplies by exp2(m_t - M) / S in fp32 and rounds
// to the fp16 output.  The logit transform (scale, softcap) therefore runs once per element.
// ---------------------------------------------------------------------------------------------
template <bool SOFTCAP>
__device__ __forceinline__ float logit2_fast(float x, float k_in, float k_cap)
{
	// without softcap: k_in = alpha * log2(e)
	// with softcap:    cap * log2(e) * tanh(alpha x / cap) = k_cap - 2 k_cap / (1 + exp2(x * k_in)),
	//                  k_in = 2 log2(e) alpha / cap, k_cap = cap * log2(e); saturates to +-k_cap
	if constexpr (SOFTCAP)
	{
		const float t = fast_exp2(x * k_in);
		return fmaf(fast_rcp(1.0f + t), -2.0f * k_cap, k_cap);
	}
	return x * k_in;
}

template <int VPL, bool SOFTCAP>
__global__ __launch_bounds__(256) void softmax_rows_f16_window_kernel(const SoftmaxArgs a)
{
	constexpr int EPV = 8;
	const int lane = threadIdx.x & (kWaveSize - 1);
	const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	if (row >= a.rows) return;  // uniform over the wave
	const RowSpan span = row_span(a, row);
	const half8_t* __restrict__ xr = reinterpret_cast<const half8_t*>(static_cast<const half_t*>(a.x) + row * a.xs);
	half8_t* __restrict__ yr = reinterpret_cast<half8_t*>(static_cast<half_t*>(a.y) + row * a.ys);
	const int nvec = (int)(a.cols / EPV);
	const int lo = (int)span.lo, hi = (int)span.hi;
	const half8_t zeros = {};

	if (hi < lo)
	{
		for (int v = lane; v < nvec; v += kWaveSize) __builtin_nontemporal_store(zeros, yr + v);
		return;
	}
	const int v_lo = lo / EPV, v_hi = hi / EPV;
	// Every load and store of the wave covers one whole 1 KB chunk of the row (64 vectors from a multiple of 64), whatever
	// the visible interval: lanes outside it load nothing and store zeros.  A run of stores that starts inside a chunk
	// leaves the memory partial lines at both ends of every instruction, and a launch whose runs start at an odd vector
	// writes a fifth slower for it (8 heads x 8192 x 8192, window 4096: 295 -> 272 us).
	const int c_lo = v_lo / kWaveSize, c_hi = v_hi / kWaveSize;

	half8_t reg[VPL];
#pragma unroll
	for (int t = 0; t < VPL; ++t)
	{
		const int v = (c_lo + t) * kWaveSize + lane;
		half8_t val = {};
		if (v >= v_lo && v <= v_hi) val = __builtin_nontemporal_load(xr + v);
		reg[t] = val;
	}

	const float k_in = SOFTCAP ? 2.0f * kLog2e * a.alpha * a.inv_cap : a.alpha_log2e;
	const float k_cap = a.cap_log2e;

	OnlineState st;
	float m_at[VPL];
#pragma unroll
	for (int t = 0; t < VPL; ++t)
	{
		const int v = (c_lo + t) * kWaveSize + lane;
		m_at[t] = -INFINITY;
		if (v >= v_lo && v <= v_hi)
		{
			float z[EPV];
#pragma unroll
			for (int e = 0; e < EPV; ++e) z[e] = logit2_fast<SOFTCAP>((float)reg[t][e], k_in, k_cap);
			if (v == v_lo || v == v_hi)
			{
				// only the two end vectors can hold keys outside [lo, hi]
#pragma unroll
				for (int e = 0; e < EPV; ++e)
				{
					const int j = v * EPV + e;
					if (j < lo || j > hi) z[e] = -INFINITY;
				}
			}
			float vmax = z[0];
#pragma unroll
			for (int e = 1; e < EPV; ++e) vmax = fmaxf(vmax, z[e]);
			const float mn = fmaxf(st.m, vmax);
			const float shift = (mn == -INFINITY) ? 0.0f : mn;
			float acc = st.s * fast_exp2(st.m - shift);
			half8_t ev;
#pragma unroll
			for (int e = 0; e < EPV; ++e)
			{
				const float p = fast_exp2(z[e] - shift);
				acc += p;
				ev[e] = (half_t)p;
			}
			reg[t] = ev;
			m_at[t] = mn;
			st.s = acc;
			st.m = mn;
		}
	}

	const float M = wave_allreduce(st.m, MaxOp());
	const float S = wave_allreduce(st.s * exp2_shift(st.m, M), SumOp());
	const float inv = S > 0.0f ? 1.0f / S : 0.0f;

	// the whole row goes out in address order, chunk by chunk: zeros, the chunks with visible keys, zeros
	for (int c = 0; c < c_lo; ++c)
		__builtin_nontemporal_store(zeros, yr + c * kWaveSize + lane);
#pragma unroll
	for (int t = 0; t < VPL; ++t)
	{
		const int v = (c_lo + t) * kWaveSize + lane;
		if (c_lo + t <= c_hi && v < nvec)
		{
			half8_t out = zeros;
			if (v >= v_lo && v <= v_hi)
			{
				const float scale = exp2_shift(m_at[t], M) * inv;
#pragma unroll
				for (int e = 0; e < EPV; ++e) out[e] = (half_t)((float)reg[t][e] * scale);
			}
			__builtin_nontemporal_store(out, yr + v);
		}
	}
	for (int v = (c_hi + 1) * kWaveSize + lane; v < nvec; v += kWaveSize) __builtin_nontemporal_store(zeros, yr + v);
}

template <int VPL>
static hipError_t launch_f16_window(const SoftmaxArgs& a, hipStream_t stream)
{
	const unsigned blocks = (unsigned)((a.rows + 3) / 4);
	discard_stale_error();
	if (a.inv_cap != 0.0f)
		softmax_rows_f16_window_kernel<VPL, true><<<dim3(blocks), dim3(256), 0, stream>>>(a);
	else
		softmax_rows_f16_window_kernel<VPL, false><<<dim3(blocks), dim3(256), 0, stream>>>(a);
	return hipGetLastError();
}

// Rows longer than a block's registers hold (more than 32768 elements: the logits of an output head): a block of 1024
// threads per row walks the row twice with 16-byte accesses, four per thread in flight: first the online maximum and
// sum, then, the row coming out of the L2 this time, the probabilities.  The vectors are aligned to the row's own start
// (rows of any length and pitch); where the result row, or the row of a mask tensor, is not aligned alike its vectors
// move at element alignment.
template <typename T>
__global__ __launch_bounds__(1024) void softmax_rows_long_kernel(const SoftmaxArgs a)
{
	constexpr int EPV = 16 / (int)sizeof(T);
	constexpr int kThreads = 1024, kAhead = 4;
	using Vec = typename Vec16<T>::type;
	typedef Vec LooseVec __attribute__((aligned(sizeof(T))));
	__shared__ float red_m[16], red_s[16];

	int64_t rows_end;
	const int64_t row = block_rows(a, 1, &rows_end);
	if (row < 0) return;
	const RowSpan span = row_span(a, row);
	const T* __restrict__ xr = static_cast<const T*>(a.x) + row * a.xs;
	T* __restrict__ yr = static_cast<T*>(a.y) + row * a.ys;
	const T* __restrict__ mrow = a.mask ? static_cast<const T*>(a.mask) + query_of_row(a, row) * a.mask_stride : nullptr;
	auto mask_at = [&](int64_t j) { return mrow ? (float)mrow[j] * kLog2e : 0.0f; };
	auto mask_vec = [&](int64_t e0) { return mrow ? *reinterpret_cast<const LooseVec*>(mrow + e0) : Vec{}; };
	// elements [0, head): one by one; then nvec whole vectors at 16-byte boundaries of x; then the rest one by one
	const int64_t to_boundary = (int64_t)(((16 - reinterpret_cast<uintptr_t>(xr) % 16) % 16) / sizeof(T));
	const int64_t head = to_boundary < a.cols ? to_boundary : a.cols;
	const int64_t nvec = (a.cols - head) / EPV;
	const int64_t rest = head + nvec * EPV;
	const Vec* __restrict__ xv = reinterpret_cast<const Vec*>(xr + head);
	const bool y_aligned = reinterpret_cast<uintptr_t>(yr + head) % 16 == 0;
	const int64_t lo = span.lo, hi = span.hi;
	const int tid = threadIdx.x;

	OnlineState st;
	auto take_one = [&](int64_t j) {
		if (j < lo || j > hi) return;
		const float z = logit2(a, (float)xr[j]) + mask_at(j);
		const float mn = fmaxf(st.m, z);
		st.s = st.s * exp2_shift(st.m, mn) + exp2_shift(z, mn);
		st.m = mn;
	};
	auto take_vec = [&](int64_t v, const Vec& val, const Vec& mval) {
		const int64_t e0 = head + v * EPV;
		if (e0 > hi || e0 + EPV - 1 < lo) return;
		float z[EPV];
		float vmax = -INFINITY;
#pragma unroll
		for (int e = 0; e < EPV; ++e)
		{
			const int64_t j = e0 + e;
			z[e] = (j >= lo && j <= hi) ? logit2(a, (float)val[e]) + (float)mval[e] * kLog2e : -INFINITY;
			vmax = fmaxf(vmax, z[e]);
		}
		const float mn = fmaxf(st.m, vmax);
		float acc = st.s * exp2_shift(st.m, mn);
#pragma unroll
		for (int e = 0; e < EPV; ++e) acc += exp2_shift(z[e], mn);
		st.s = acc;
		st.m = mn;
	};
	if (tid < head) take_one(tid);
	for (int64_t j = rest + tid; j < a.cols; j += kThreads) take_one(j);
	for (int64_t v0 = tid; v0 < nvec; v0 += (int64_t)kThreads * kAhead)
	{
		Vec val[kAhead], mval[kAhead];
#pragma unroll
		for (int u = 0; u < kAhead; ++u)
		{
			const int64_t v = v0 + (int64_t)u * kThreads;
			const int64_t e0 = head + v * EPV;
			val[u] = Vec{};
			mval[u] = Vec{};
			if (v < nvec && e0 <= hi && e0 + EPV - 1 >= lo)
			{
				val[u] = xv[v];
				mval[u] = mask_vec(e0);
			}
		}
#pragma unroll
		for (int u = 0; u < kAhead; ++u)
		{
			const int64_t v = v0 + (int64_t)u * kThreads;
			if (v < nvec) take_vec(v, val[u], mval[u]);
		}
	}

	const int wave = tid >> 6;
	const float wm = wave_allreduce(st.m, MaxOp());
	const float ws = wave_allreduce(st.s * exp2_shift(st.m, wm), SumOp());
	if ((tid & 63) == 0)
	{
		red_m[wave] = wm;
		red_s[wave] = ws;
	}
	__syncthreads();
	float M = -INFINITY;
#pragma unroll
	for (int w = 0; w < 16; ++w) M = fmaxf(M, red_m[w]);
	float S = 0.0f;
#pragma unroll
	for (int w = 0; w < 16; ++w) S += red_s[w] * exp2_shift(red_m[w], M);
	const float inv = S > 0.0f ? 1.0f / S : 0.0f;

	auto put_one = [&](int64_t j) {
		const float p = (j >= lo && j <= hi) ? exp2_shift(logit2(a, (float)xr[j]) + mask_at(j), M) * inv : 0.0f;
		yr[j] = (T)p;
	};
	if (tid < head) put_one(tid);
	for (int64_t j = rest + tid; j < a.cols; j += kThreads) put_one(j);
	for (int64_t v0 = tid; v0 < nvec; v0 += (int64_t)kThreads * kAhead)
	{
		Vec val[kAhead], mval[kAhead];
#pragma unroll
		for (int u = 0; u < kAhead; ++u)
		{
			const int64_t v = v0 + (int64_t)u * kThreads;
			const int64_t e0 = head + v * EPV;
			val[u] = Vec{};
			mval[u] = Vec{};
			if (v < nvec && e0 <= hi && e0 + EPV - 1 >= lo)
			{
				val[u] = xv[v];
				mval[u] = mask_vec(e0);
			}
		}
#pragma unroll
		for (int u = 0; u < kAhead; ++u)
		{
			const int64_t v = v0 + (int64_t)u * kThreads;
			if (v >= nvec) continue;
			const int64_t e0 = head + v * EPV;
			Vec out = {};
			if (e0 <= hi && e0 + EPV - 1 >= lo)
			{
#pragma unroll
				for (int e = 0; e < EPV; ++e)
				{
					const int64_t j = e0 + e;
					out[e] = (T)((j >= lo && j <= hi) ? exp2_shift(logit2(a, (float)val[u][e]) + (float)mval[u][e] * kLog2e, M) * inv : 0.0f);
				}
			}
			if (y_aligned) __builtin_nontemporal_store(out, reinterpret_cast<Vec*>(yr + e0));
			else *reinterpret_cast<LooseVec*>(yr + e0) = out;
		}
	}
}

template <typename T, int VPL, bool LOOSE = false, int GROUP = 64>
static hipError_t launch_wave(const SoftmaxArgs& a, hipStream_t stream)
{
	const unsigned blocks = blocks_for_rows(a, 256 / GROUP);
	discard_stale_error();
	if (a.mask != nullptr) softmax_rows_wave_kernel<T, VPL, LOOSE, GROUP, true><<<dim3(blocks), dim3(256), 0, stream>>>(a);
	else softmax_rows_wave_kernel<T, VPL, LOOSE, GROUP, false><<<dim3(blocks), dim3(256), 0, stream>>>(a);
	return hipGetLastError();
}

// rows longer than a wave holds: the block per row, 256 * VPL vectors in registers
template <typename T, bool LOOSE>
static hipError_t launch_long_rows(const SoftmaxArgs& a, int64_t nvec, hipStream_t stream)
{
	if (nvec <= 256 * 4) return launch_wave<T, 4, LOOSE, 256>(a, stream);       // (rows with a mask tensor: a wave takes fewer)
	if (nvec <= 256 * 8) return launch_wave<T, 8, LOOSE, 256>(a, stream);
	return launch_wave<T, 16, LOOSE, 256>(a, stream);       // (the caller checks the capacity: 256 x 16 vectors)
}

template <typename T>
hipError_t launch_softmax_rows(const void* x, void* y, int64_t rows, int64_t cols, int64_t xs, int64_t ys,
                               int64_t q_len, int64_t diag, float alpha, float softcap, int causal,
                               int64_t window, const void* mask, int64_t mask_stride, hipStream_t stream)
{
	if (rows == 0 || cols == 0) return hipSuccess;

	SoftmaxArgs a;
	a.x = x; a.y = y; a.rows = rows; a.cols = cols; a.xs = xs; a.ys = ys;
	a.q_len = q_len; a.diag = diag; a.alpha = alpha;
	a.inv_cap = softcap != 0.0f ? 1.0f / softcap : 0.0f;
	a.cap_log2e = softcap * kLog2e;
	a.alpha_log2e = alpha * kLog2e;
	a.causal = causal; a.window = window;
	a.mask = mask; a.mask_stride = mask_stride;
	// (several heads over one mask: the blocks are dealt so that the heads of a mask row meet in one L2)
	a.heads = (mask != nullptr && q_len > 0 && rows > q_len && rows % q_len == 0 && rows / q_len <= 65536) ? (int)(rows / q_len) : 1;

	constexpr int EPV = 16 / (int)sizeof(T);
	const bool vec_ok = (cols % EPV == 0) && (xs % EPV == 0) && (ys % EPV == 0) &&
	                    (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(y) % 16 == 0) &&
	                    (mask == nullptr || (mask_stride % EPV == 0 && reinterpret_cast<uintptr_t>(mask) % 16 == 0));
	const int64_t nvec = cols / EPV;
	// short rows (up to 64 vectors: 512 halves, 256 floats): sixteen lanes per row, four rows per wave
	if (vec_ok && nvec <= 64 && rows >= 64)
	{
		if (nvec <= 16) return launch_wave<T, 1, false, 16>(a, stream);
		if (nvec <= 32) return launch_wave<T, 2, false, 16>(a, stream);
		return launch_wave<T, 4, false, 16>(a, stream);       // (twice as many vectors per lane: slower than a wave per row)
	}
	if (!vec_ok && (cols + EPV - 1) / EPV <= 64 && rows >= 64)
	{
		const int64_t loose = (cols + EPV - 1) / EPV;
		if (loose <= 16) return launch_wave<T, 1, true, 16>(a, stream);
		if (loose <= 32) return launch_wave<T, 2, true, 16>(a, stream);
		return launch_wave<T, 4, true, 16>(a, stream);
	}
	if constexpr (sizeof(T) == 2)
	{
		// vectors a row can touch: its visible keys (the window when causal + window, else the
		// whole row) plus one for an interval that starts inside a vector
		const int64_t span = (causal && window > 0) ? std::min<int64_t>(cols, window) : cols;
		int64_t span_vecs = std::min<int64_t>(nvec, (span + EPV - 1) / EPV + 1);
		// (the kernel counts in whole chunks of 64 vectors from the chunk the interval starts in; without a window every
		// interval starts at the start of the row)
		if (window > 0) span_vecs = std::min<int64_t>((nvec + kWaveSize - 1) / kWaveSize * kWaveSize, span_vecs + kWaveSize - 1);
		if (vec_ok && mask == nullptr)
		{
			if (span_vecs <= kWaveSize * 1) return launch_f16_window<1>(a, stream);
			if (span_vecs <= kWaveSize * 2) return launch_f16_window<2>(a, stream);
			if (span_vecs <= kWaveSize * 4) return launch_f16_window<4>(a, stream);
			if (span_vecs <= kWaveSize * 6) return launch_f16_window<6>(a, stream);
			if (span_vecs <= kWaveSize * 9) return launch_f16_window<9>(a, stream);
			if (span_vecs <= kWaveSize * 12) return launch_f16_window<12>(a, stream);
			if (span_vecs <= kWaveSize * 16) return launch_f16_window<16>(a, stream);
		}
	}
	// A wave holds up to 16 vectors per lane of its row (32 of float32 fit the registers, but leave a SIMD with too few
	// waves: 16384 x 8192 float32 353 us that way, 185 us with the block per row); the block per row up to 16 as well
	// (32768 halves, 16384 floats); longer rows, and long rows too few to give every CU a block, are walked twice by
	// 1024 threads (8192 x 32768 float32: 751 us in registers, 426 us walked twice; 128 x 32768 halves: 18 -> 10 us).
	constexpr int kMaxVpl = 16;
	const bool walk_twice = nvec > (int64_t)256 * kMaxVpl || (nvec > 2048 && rows < 256);
	if (vec_ok && walk_twice)
	{
		discard_stale_error();
		softmax_rows_long_kernel<T><<<dim3(blocks_for_rows(a, 1)), dim3(1024), 0, stream>>>(a);
		return hipGetLastError();
	}
	// (with a mask tensor, whose vectors sit in registers beside the row's, a wave takes up to 8 vectors per lane)
	if (vec_ok && nvec <= (int64_t)kWaveSize * (mask ? 8 : kMaxVpl))
	{
		if (nvec <= kWaveSize * 1) return launch_wave<T, 1>(a, stream);
		if (nvec <= kWaveSize * 2) return launch_wave<T, 2>(a, stream);
		if (nvec <= kWaveSize * 4) return launch_wave<T, 4>(a, stream);
		if (nvec <= kWaveSize * 8) return launch_wave<T, 8>(a, stream);
		return launch_wave<T, 16>(a, stream);
	}
	if (vec_ok && nvec <= (int64_t)256 * kMaxVpl) return launch_long_rows<T, false>(a, nvec, stream);
	// rows at element alignment, any width: the same wave kernel with element-aligned vector accesses
	const int64_t nvec_loose = (cols + EPV - 1) / EPV;
	if (!vec_ok && nvec_loose <= (int64_t)kWaveSize * (mask ? 8 : kMaxVpl))
	{
		if (nvec_loose <= kWaveSize * 1) return launch_wave<T, 1, true>(a, stream);
		if (nvec_loose <= kWaveSize * 2) return launch_wave<T, 2, true>(a, stream);
		if (nvec_loose <= kWaveSize * 4) return launch_wave<T, 4, true>(a, stream);
		if (nvec_loose <= kWaveSize * 8) return launch_wave<T, 8, true>(a, stream);
		return launch_wave<T, 16, true>(a, stream);
	}
	if (!vec_ok && nvec_loose <= (int64_t)256 * kMaxVpl && !(nvec_loose > 2048 && rows < 256))
		return launch_long_rows<T, true>(a, nvec_loose, stream);
	discard_stale_error();
	softmax_rows_long_kernel<T><<<dim3(blocks_for_rows(a, 1)), dim3(1024), 0, stream>>>(a);
	return hipGetLastError();
}

template hipError_t launch_softmax_rows<half_t>(const void*, void*, int64_t, int64_t, int64_t, int64_t, int64_t,
                                                 int64_t, float, float, int, int64_t, const void*, int64_t, hipStream_t);
template hipError_t launch_softmax_rows<float>(const void*, void*, int64_t, int64_t, int64_t, int64_t, int64_t,
                                                int64_t, float, float, int, int64_t, const void*, int64_t, hipStream_t);

}  // namespace anygpu
