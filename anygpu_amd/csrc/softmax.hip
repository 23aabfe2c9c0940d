// Row softmax for gfx950 with the attention prologue (scale, logit softcap, causal and
// sliding-window masks) fused in.  HBM-bound: every visible input element is read once and
// every output element written once, with 16-byte accesses.
//
// Fast kernel: one wave owns one row and keeps it in registers (VPL 16-byte vectors per
// lane), runs an online max/sum over the vectors as they arrive, combines the 64 lane
// states with DPP reductions, then normalises from registers.  Vectors that lie wholly
// outside the visible key interval [lo, hi] of the row are never loaded; their outputs are
// stored as zeros.
// General kernel: one 256-thread block per row with scalar accesses for any width, stride
// or alignment; it reads the visible part of the row twice.
#include "device_utils.hpp"
#include "launch.hpp"

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
};

template <typename T> struct Vec16;
template <> struct Vec16<half_t> { using type = half8_t; };
template <> struct Vec16<float> { using type = float4_t; };

// Visible key interval of a row, inclusive on both ends; empty when hi < lo.
struct RowSpan { int64_t lo, hi; };

__device__ __forceinline__ RowSpan row_span(const SoftmaxArgs& a, int64_t row)
{
	int64_t i = row;
	if (a.q_len > 0)
	{
		// rows and q_len are validated to fit 32 bits by the host entry point
		i = (int64_t)((uint32_t)row % (uint32_t)a.q_len);
	}
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

template <typename T, int VPL>
__global__ __launch_bounds__(256) void softmax_rows_wave_kernel(const SoftmaxArgs a)
{
	constexpr int EPV = 16 / (int)sizeof(T);
	using Vec = typename Vec16<T>::type;

	const int lane = threadIdx.x & (kWaveSize - 1);
	const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
	if (row >= a.rows) return;  // uniform over the wave

	const RowSpan span = row_span(a, row);
	const T* __restrict__ xr = static_cast<const T*>(a.x) + row * a.xs;
	T* __restrict__ yr = static_cast<T*>(a.y) + row * a.ys;
	const int nvec = (int)(a.cols / EPV);
	const int lo = (int)span.lo, hi = (int)span.hi;

	Vec raw[VPL];
#pragma unroll
	for (int t = 0; t < VPL; ++t)
	{
		const int v = lane + kWaveSize * t;
		const int e0 = v * EPV;
		const bool need = (v < nvec) && (e0 <= hi) && (e0 + EPV - 1 >= lo);
		Vec val = {};
		if (need) val = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(xr) + v);
		raw[t] = val;
	}

	OnlineState st;
#pragma unroll
	for (int t = 0; t < VPL; ++t)
	{
		const int v = lane + kWaveSize * t;
		const int e0 = v * EPV;
		const bool need = (v < nvec) && (e0 <= hi) && (e0 + EPV - 1 >= lo);
		if (need)
		{
			float z[EPV];
			float vmax = -INFINITY;
#pragma unroll
			for (int e = 0; e < EPV; ++e)
			{
				const int j = e0 + e;
				const float zz = logit2(a, (float)raw[t][e]);
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

	const float M = wave_allreduce(st.m, MaxOp());
	const float S = wave_allreduce(st.s * exp2_shift(st.m, M), SumOp());
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
#pragma unroll
				for (int e = 0; e < EPV; ++e)
				{
					const int j = e0 + e;
					const float p = exp2_shift(logit2(a, (float)raw[t][e]), M) * inv;
					out[e] = (T)((j >= lo && j <= hi) ? p : 0.0f);
				}
			}
			__builtin_nontemporal_store(out, reinterpret_cast<Vec*>(yr) + v);
		}
	}
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_rows_block_kernel(const SoftmaxArgs a)
{
	__shared__ float red_m[4];
	__shared__ float red_s[4];

	const int64_t row = blockIdx.x;
	const RowSpan span = row_span(a, row);
	const T* __restrict__ xr = static_cast<const T*>(a.x) + row * a.xs;
	T* __restrict__ yr = static_cast<T*>(a.y) + row * a.ys;

	OnlineState st;
	for (int64_t j = span.lo + threadIdx.x; j <= span.hi; j += blockDim.x)
	{
		const float z = logit2(a, (float)xr[j]);
		const float mn = fmaxf(st.m, z);
		st.s = st.s * exp2_shift(st.m, mn) + exp2_shift(z, mn);
		st.m = mn;
	}

	const int wave = threadIdx.x >> 6;
	const float wm = wave_allreduce(st.m, MaxOp());
	const float ws = wave_allreduce(st.s * exp2_shift(st.m, wm), SumOp());
	if ((threadIdx.x & (kWaveSize - 1)) == 0)
	{
		red_m[wave] = wm;
		red_s[wave] = ws;
	}
	__syncthreads();
	float M = fmaxf(fmaxf(red_m[0], red_m[1]), fmaxf(red_m[2], red_m[3]));
	float S = 0.0f;
#pragma unroll
	for (int w = 0; w < 4; ++w) S += red_s[w] * exp2_shift(red_m[w], M);
	const float inv = S > 0.0f ? 1.0f / S : 0.0f;

	for (int64_t j = threadIdx.x; j < a.cols; j += blockDim.x)
	{
		float p = 0.0f;
		if (j >= span.lo && j <= span.hi) p = exp2_shift(logit2(a, (float)xr[j]), M) * inv;
		yr[j] = (T)p;
	}
}

template <typename T, int VPL>
static hipError_t launch_wave(const SoftmaxArgs& a, hipStream_t stream)
{
	const unsigned blocks = (unsigned)((a.rows + 3) / 4);
	discard_stale_error();
	softmax_rows_wave_kernel<T, VPL><<<dim3(blocks), dim3(256), 0, stream>>>(a);
	return hipGetLastError();
}

template <typename T>
hipError_t launch_softmax_rows(const void* x, void* y, int64_t rows, int64_t cols, int64_t xs, int64_t ys,
                               int64_t q_len, int64_t diag, float alpha, float softcap, int causal,
                               int64_t window, hipStream_t stream)
{
	if (rows == 0 || cols == 0) return hipSuccess;

	SoftmaxArgs a;
	a.x = x; a.y = y; a.rows = rows; a.cols = cols; a.xs = xs; a.ys = ys;
	a.q_len = q_len; a.diag = diag; a.alpha = alpha;
	a.inv_cap = softcap != 0.0f ? 1.0f / softcap : 0.0f;
	a.cap_log2e = softcap * kLog2e;
	a.alpha_log2e = alpha * kLog2e;
	a.causal = causal; a.window = window;

	constexpr int EPV = 16 / (int)sizeof(T);
	const bool vec_ok = (cols % EPV == 0) && (xs % EPV == 0) && (ys % EPV == 0) &&
	                    (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(y) % 16 == 0);
	const int64_t nvec = cols / EPV;
	constexpr int kMaxVpl = sizeof(T) == 2 ? 16 : 32;
	if (vec_ok && nvec <= (int64_t)kWaveSize * kMaxVpl)
	{
		if (nvec <= kWaveSize * 1) return launch_wave<T, 1>(a, stream);
		if (nvec <= kWaveSize * 2) return launch_wave<T, 2>(a, stream);
		if (nvec <= kWaveSize * 4) return launch_wave<T, 4>(a, stream);
		if (nvec <= kWaveSize * 8) return launch_wave<T, 8>(a, stream);
		if (nvec <= kWaveSize * 16) return launch_wave<T, 16>(a, stream);
		if constexpr (kMaxVpl >= 32) return launch_wave<T, 32>(a, stream);
	}
	discard_stale_error();
	softmax_rows_block_kernel<T><<<dim3((unsigned)rows), dim3(256), 0, stream>>>(a);
	return hipGetLastError();
}

template hipError_t launch_softmax_rows<half_t>(const void*, void*, int64_t, int64_t, int64_t, int64_t, int64_t,
                                                 int64_t, float, float, int, int64_t, hipStream_t);
template hipError_t launch_softmax_rows<float>(const void*, void*, int64_t, int64_t, int64_t, int64_t, int64_t,
                                                int64_t, float, float, int, int64_t, hipStream_t);

}  // namespace anygpu
