// Depthwise causal conv1d + bias + SiLU for gfx950.  Layout [batch, chan, seqlen] with the
// sequence axis contiguous, so every (batch, chan) pair is one independent row.  HBM-bound:
// x is read once, y written once, 16 bytes per lane per access.
//
// Tiled kernel: a 256-thread block owns a tile of 256 * U consecutive 16-byte vectors of one
// row.  Each lane needs the width-1 samples in front of its vector; they are the tail of the
// neighbouring lane's vector, so every lane publishes the tail of its vector in LDS and reads
// its left neighbour's after one barrier.  The halo in front of the whole tile comes from
// global memory (zeros at the start of a row).
// Element kernel: one thread per output sample, for sequence lengths or pointers that do not
// allow 16-byte row access.
#include "device_utils.hpp"
#include "launch.hpp"

namespace anygpu {

constexpr int kMaxWidth = 4;
constexpr int kHalo = kMaxWidth - 1;

template <typename T> struct ConvVec;
template <> struct ConvVec<half_t> { using type = half8_t; using tail_type = half4_t; };
template <> struct ConvVec<float> { using type = float4_t; using tail_type = float4_t; };

__device__ __forceinline__ float silu_f32(float v)
{
	// v / (1 + e^{-v})
	return v * fast_rcp(1.0f + fast_exp2(-v * kLog2e));
}

// The taps of a channel right-aligned into four slots: slot 3 multiplies the current sample,
// slot 3 - d the sample d steps back.  Slots below 4 - WIDTH do not exist and are skipped.
template <int WIDTH>
__device__ __forceinline__ float conv_point(const float (&wv)[kMaxWidth], float bias, float xm3, float xm2, float xm1, float x0)
{
	const float xs[kMaxWidth] = { xm3, xm2, xm1, x0 };
	float acc = 0.0f;
#pragma unroll
	for (int k = kMaxWidth - WIDTH; k < kMaxWidth; ++k) acc += wv[k] * xs[k];
	acc += bias;
	return silu_f32(acc);
}

// LOOSE: rows may start at any element and seqlen need not be a multiple of the vector length: vector
// accesses go out at element alignment, the partial last vector of a row is moved element by element.
template <typename T, int WIDTH, int U, bool LOOSE>
__global__ __launch_bounds__(256) void causal_conv1d_silu_tile_kernel(
	const T* __restrict__ x, const T* __restrict__ w, const T* __restrict__ bias, T* __restrict__ y,
	int chan, int seqlen, int tiles_per_row)
{
	constexpr int EPV = 16 / (int)sizeof(T);
	constexpr int TPV = (int)(sizeof(typename ConvVec<T>::tail_type) / sizeof(T));  // samples in a published tail
	using Vec = typename ConvVec<T>::type;
	using Tail = typename ConvVec<T>::tail_type;
	typedef Vec LooseVec __attribute__((aligned(sizeof(T))));
	typedef Tail LooseTail __attribute__((aligned(sizeof(T))));

	__shared__ Tail tails[U][256];

	const int tid = threadIdx.x;
	const int row = blockIdx.x / tiles_per_row;           // (batch, chan) pair
	const int tile = blockIdx.x - row * tiles_per_row;
	const int ch = row % chan;
	const int rest = LOOSE ? seqlen % EPV : 0;               // samples of a partial last vector
	const int nvec = seqlen / EPV + (rest ? 1 : 0);
	const int v_base = tile * (256 * U);

	const T* __restrict__ xr = x + (int64_t)row * seqlen;
	T* __restrict__ yr = y + (int64_t)row * seqlen;

	float wv[kMaxWidth] = { 0.f, 0.f, 0.f, 0.f };
#pragma unroll
	for (int k = 0; k < WIDTH; ++k) wv[kMaxWidth - WIDTH + k] = (float)w[(int64_t)ch * WIDTH + k];
	const float bv = (float)bias[ch];

	Vec xv[U];
#pragma unroll
	for (int u = 0; u < U; ++u)
	{
		const int v = v_base + u * 256 + tid;
		Vec val = {};
		if (v < nvec)
		{
			if (LOOSE && rest && v == nvec - 1)
			{
#pragma unroll
				for (int e = 0; e < EPV; ++e)
					if (e < rest) val[e] = xr[(int64_t)v * EPV + e];
			}
			else if (LOOSE) val = __builtin_nontemporal_load(reinterpret_cast<const LooseVec*>(xr) + v);
			else val = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(xr) + v);
		}
		xv[u] = val;
	}
	// halo in front of the tile: the TPV samples that end where the tile starts
	Tail front = {};
	if (tid == 0 && v_base > 0)
	{
		if (LOOSE) front = *reinterpret_cast<const LooseTail*>(xr + (int64_t)v_base * EPV - TPV);
		else front = *reinterpret_cast<const Tail*>(xr + (int64_t)v_base * EPV - TPV);
	}

#pragma unroll
	for (int u = 0; u < U; ++u)
	{
		Tail t;
#pragma unroll
		for (int e = 0; e < TPV; ++e) t[e] = xv[u][EPV - TPV + e];
		tails[u][tid] = t;
	}
	__syncthreads();

#pragma unroll
	for (int u = 0; u < U; ++u)
	{
		const int v = v_base + u * 256 + tid;
		if (v >= nvec) continue;
		Tail prev;
		if (tid > 0) prev = tails[u][tid - 1];
		else if (u > 0) prev = tails[u - 1][255];
		else prev = front;

		float s[kHalo + EPV];
#pragma unroll
		for (int e = 0; e < kHalo; ++e) s[e] = (float)prev[TPV - kHalo + e];
#pragma unroll
		for (int e = 0; e < EPV; ++e) s[kHalo + e] = (float)xv[u][e];

		Vec out;
#pragma unroll
		for (int e = 0; e < EPV; ++e)
		{
			out[e] = (T)conv_point<WIDTH>(wv, bv, s[e], s[e + 1], s[e + 2], s[e + 3]);
		}
		if (LOOSE && rest && v == nvec - 1)
		{
#pragma unroll
			for (int e = 0; e < EPV; ++e)
				if (e < rest) yr[(int64_t)v * EPV + e] = out[e];
		}
		else if (LOOSE) __builtin_nontemporal_store(out, reinterpret_cast<LooseVec*>(yr) + v);
		else __builtin_nontemporal_store(out, reinterpret_cast<Vec*>(yr) + v);
	}
}

// Short rows: a row has fewer vectors than a tile of the kernel above has slots, so the tile would be mostly idle.
// Here the (row, vector) pairs of the whole tensor are numbered consecutively and a block takes 256 of them,
// whichever rows they belong to; a thread finds its halo in its left neighbour's tail unless its vector is
// the first of a row (zeros) or the first of the block (global memory).  Taps and bias are loaded per thread.
template <typename T, int WIDTH, bool LOOSE>
__global__ __launch_bounds__(256) void causal_conv1d_silu_short_rows_kernel(
	const T* __restrict__ x, const T* __restrict__ w, const T* __restrict__ bias, T* __restrict__ y,
	int chan, int seqlen, int nvec, int64_t total_vecs)
{
	constexpr int EPV = 16 / (int)sizeof(T);
	constexpr int TPV = (int)(sizeof(typename ConvVec<T>::tail_type) / sizeof(T));
	using Vec = typename ConvVec<T>::type;
	using Tail = typename ConvVec<T>::tail_type;
	typedef Vec LooseVec __attribute__((aligned(sizeof(T))));
	typedef Tail LooseTail __attribute__((aligned(sizeof(T))));
	__shared__ Tail tails[256];

	const int tid = threadIdx.x;
	const int64_t g = (int64_t)blockIdx.x * 256 + tid;
	const bool live = g < total_vecs;
	const int64_t row = live ? g / nvec : 0;
	const int v = live ? (int)(g - row * nvec) : 0;
	const int rest = LOOSE ? seqlen % EPV : 0;
	const bool partial = LOOSE && rest && v == nvec - 1;
	const T* __restrict__ xr = x + row * seqlen;
	T* __restrict__ yr = y + row * seqlen;

	Vec xv = {};
	if (live)
	{
		if (partial)
		{
#pragma unroll
			for (int e = 0; e < EPV; ++e)
				if (e < rest) xv[e] = xr[(int64_t)v * EPV + e];
		}
		else if (LOOSE) xv = __builtin_nontemporal_load(reinterpret_cast<const LooseVec*>(xr) + v);
		else xv = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(xr) + v);
	}
	Tail front = {};
	if (tid == 0 && live && v > 0)
	{
		if (LOOSE) front = *reinterpret_cast<const LooseTail*>(xr + (int64_t)v * EPV - TPV);
		else front = *reinterpret_cast<const Tail*>(xr + (int64_t)v * EPV - TPV);
	}
	Tail mine;
#pragma unroll
	for (int e = 0; e < TPV; ++e) mine[e] = xv[EPV - TPV + e];
	tails[tid] = mine;
	__syncthreads();
	if (!live) return;

	Tail prev = {};
	if (v > 0) prev = tid > 0 ? tails[tid - 1] : front;

	const int ch = (int)(row % chan);
	float wv[kMaxWidth] = { 0.f, 0.f, 0.f, 0.f };
#pragma unroll
	for (int k = 0; k < WIDTH; ++k) wv[kMaxWidth - WIDTH + k] = (float)w[(int64_t)ch * WIDTH + k];
	const float bv = (float)bias[ch];

	float s[kHalo + EPV];
#pragma unroll
	for (int e = 0; e < kHalo; ++e) s[e] = (float)prev[TPV - kHalo + e];
#pragma unroll
	for (int e = 0; e < EPV; ++e) s[kHalo + e] = (float)xv[e];
	Vec out;
#pragma unroll
	for (int e = 0; e < EPV; ++e) out[e] = (T)conv_point<WIDTH>(wv, bv, s[e], s[e + 1], s[e + 2], s[e + 3]);
	if (partial)
	{
#pragma unroll
		for (int e = 0; e < EPV; ++e)
			if (e < rest) yr[(int64_t)v * EPV + e] = out[e];
	}
	else if (LOOSE) __builtin_nontemporal_store(out, reinterpret_cast<LooseVec*>(yr) + v);
	else __builtin_nontemporal_store(out, reinterpret_cast<Vec*>(yr) + v);
}

template <typename T, int WIDTH>
__global__ __launch_bounds__(256) void causal_conv1d_silu_element_kernel(
	const T* __restrict__ x, const T* __restrict__ w, const T* __restrict__ bias, T* __restrict__ y,
	int chan, int seqlen, int64_t total)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (idx >= total) return;
	const int64_t row = idx / seqlen;
	const int s = (int)(idx - row * seqlen);
	const int ch = (int)(row % chan);

	float wv[kMaxWidth] = { 0.f, 0.f, 0.f, 0.f };
#pragma unroll
	for (int k = 0; k < WIDTH; ++k) wv[kMaxWidth - WIDTH + k] = (float)w[(int64_t)ch * WIDTH + k];
	const float bv = (float)bias[ch];

	const T* __restrict__ xr = x + row * seqlen;
	float xs[kMaxWidth];
#pragma unroll
	for (int k = 0; k < kMaxWidth; ++k)
	{
		const int pos = s + k - kHalo;
		xs[k] = (k >= kMaxWidth - WIDTH && pos >= 0) ? (float)xr[pos] : 0.0f;
	}
	y[idx] = (T)conv_point<WIDTH>(wv, bv, xs[0], xs[1], xs[2], xs[3]);
}

template <typename T, int WIDTH>
static hipError_t launch_width(const void* x, const void* w, const void* bias, void* y,
                               int64_t batch, int64_t chan, int64_t seqlen, hipStream_t stream)
{
	constexpr int EPV = 16 / (int)sizeof(T);
	constexpr int U = 2;
	const int64_t rows = batch * chan;
	const T* xp = static_cast<const T*>(x);
	const T* wp = static_cast<const T*>(w);
	const T* bp = static_cast<const T*>(bias);
	T* yp = static_cast<T*>(y);

	const bool vec_ok = (seqlen % EPV == 0) && (reinterpret_cast<uintptr_t>(x) % 16 == 0) &&
	                    (reinterpret_cast<uintptr_t>(y) % 16 == 0);
	{
		// vectors per row, a partial last one included; rows shorter than the halo take the element kernel
		const int64_t nvec = (seqlen + EPV - 1) / EPV;
		const int64_t tiles_per_row = (nvec + 256 * U - 1) / (256 * U);
		const int64_t blocks = rows * tiles_per_row;
		if (nvec < 256 * U && seqlen >= EPV && (rows * nvec + 255) / 256 <= 0x7FFFFFFFLL)
		{
			// short rows: blocks over the consecutive (row, vector) pairs
			const int64_t total_vecs = rows * nvec;
			const dim3 grid((unsigned)((total_vecs + 255) / 256));
			discard_stale_error();
			if (vec_ok)
				causal_conv1d_silu_short_rows_kernel<T, WIDTH, false><<<grid, dim3(256), 0, stream>>>(
					xp, wp, bp, yp, (int)chan, (int)seqlen, (int)nvec, total_vecs);
			else
				causal_conv1d_silu_short_rows_kernel<T, WIDTH, true><<<grid, dim3(256), 0, stream>>>(
					xp, wp, bp, yp, (int)chan, (int)seqlen, (int)nvec, total_vecs);
			return hipGetLastError();
		}
		if (blocks <= 0x7FFFFFFFLL && seqlen >= EPV)
		{
			discard_stale_error();
			if (vec_ok)
				causal_conv1d_silu_tile_kernel<T, WIDTH, U, false><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
					xp, wp, bp, yp, (int)chan, (int)seqlen, (int)tiles_per_row);
			else
				causal_conv1d_silu_tile_kernel<T, WIDTH, U, true><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
					xp, wp, bp, yp, (int)chan, (int)seqlen, (int)tiles_per_row);
			return hipGetLastError();
		}
	}
	const int64_t total = rows * seqlen;
	const int64_t blocks = (total + 255) / 256;
	discard_stale_error();
	causal_conv1d_silu_element_kernel<T, WIDTH><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(
		xp, wp, bp, yp, (int)chan, (int)seqlen, total);
	return hipGetLastError();
}

template <typename T>
hipError_t launch_causal_conv1d_silu(const void* x, const void* w, const void* bias, void* y,
                                     int64_t batch, int64_t chan, int64_t seqlen, int width,
                                     hipStream_t stream)
{
	if (batch == 0 || chan == 0 || seqlen == 0) return hipSuccess;
	switch (width)
	{
	case 1: return launch_width<T, 1>(x, w, bias, y, batch, chan, seqlen, stream);
	case 2: return launch_width<T, 2>(x, w, bias, y, batch, chan, seqlen, stream);
	case 3: return launch_width<T, 3>(x, w, bias, y, batch, chan, seqlen, stream);
	default: return launch_width<T, 4>(x, w, bias, y, batch, chan, seqlen, stream);
	}
}

// Decode step: one new sample per (batch, chan) row.  `state` keeps the width - 1 samples in
// front of it, oldest first, [batch, chan, width - 1]; it is shifted by one and takes the new
// sample.  One thread per row: the row's state, taps, bias and sample are a few bytes each.
template <typename T, int WIDTH>
__global__ __launch_bounds__(256) void causal_conv1d_silu_update_kernel(
	const T* __restrict__ x, T* __restrict__ state, const T* __restrict__ w, const T* __restrict__ bias,
	T* __restrict__ y, int chan, int64_t rows)
{
	const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (row >= rows) return;
	const int ch = (int)(row % chan);
	T* st = state + row * (WIDTH - 1);
	T hist[WIDTH];
#pragma unroll
	for (int k = 0; k < WIDTH - 1; ++k) hist[k] = st[k];
	hist[WIDTH - 1] = x[row];
	float acc = 0.0f;
#pragma unroll
	for (int k = 0; k < WIDTH; ++k) acc += (float)w[(int64_t)ch * WIDTH + k] * (float)hist[k];
	acc += (float)bias[ch];
	y[row] = (T)silu_f32(acc);
#pragma unroll
	for (int k = 0; k < WIDTH - 1; ++k) st[k] = hist[k + 1];
}

template <typename T>
hipError_t launch_causal_conv1d_silu_update(const void* x, void* state, const void* w, const void* bias, void* y,
                                            int64_t batch, int64_t chan, int width, hipStream_t stream)
{
	const int64_t rows = batch * chan;
	if (rows == 0) return hipSuccess;
	const dim3 grid((unsigned)((rows + 255) / 256));
	const T* xp = static_cast<const T*>(x);
	T* sp = static_cast<T*>(state);
	const T* wp = static_cast<const T*>(w);
	const T* bp = static_cast<const T*>(bias);
	T* yp = static_cast<T*>(y);
	discard_stale_error();
	switch (width)
	{
	case 1: causal_conv1d_silu_update_kernel<T, 1><<<grid, dim3(256), 0, stream>>>(xp, sp, wp, bp, yp, (int)chan, rows); break;
	case 2: causal_conv1d_silu_update_kernel<T, 2><<<grid, dim3(256), 0, stream>>>(xp, sp, wp, bp, yp, (int)chan, rows); break;
	case 3: causal_conv1d_silu_update_kernel<T, 3><<<grid, dim3(256), 0, stream>>>(xp, sp, wp, bp, yp, (int)chan, rows); break;
	default: causal_conv1d_silu_update_kernel<T, 4><<<grid, dim3(256), 0, stream>>>(xp, sp, wp, bp, yp, (int)chan, rows); break;
	}
	return hipGetLastError();
}

template hipError_t launch_causal_conv1d_silu_update<half_t>(const void*, void*, const void*, const void*, void*, int64_t, int64_t,
                                                              int, hipStream_t);
template hipError_t launch_causal_conv1d_silu_update<float>(const void*, void*, const void*, const void*, void*, int64_t, int64_t,
                                                             int, hipStream_t);

template hipError_t launch_causal_conv1d_silu<half_t>(const void*, const void*, const void*, void*, int64_t, int64_t,
                                                       int64_t, int, hipStream_t);
template hipError_t launch_causal_conv1d_silu<float>(const void*, const void*, const void*, void*, int64_t, int64_t,
                                                      int64_t, int, hipStream_t);

}  // namespace anygpu
