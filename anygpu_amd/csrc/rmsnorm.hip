// Gated RMS normalisation over the last axis for gfx950:
//   g = x * silu(z)   (g = x when there is no gate)
//   y = g / sqrt(mean(g^2) + eps) * (w + delta),   delta = 1 for zero-centred weights, else 0
// The step between the SSD scan and the output projection of a Mamba2 mixer.  HBM-bound: x and z are
// read once, y is written once, the row lives in registers between the sum of squares and the
// scaling.  16-byte accesses; the row length picks how many threads share a row (a row of 16 lanes, a wave or the
// 256-thread block: short rows would leave most of a block without a vector) and how many vectors a thread keeps (1, 2,
// 4 or 8: up to 8192 floats or 16384 halves).  Longer rows are walked twice by a block of 1024 threads, the second time
// out of the L2; rows whose length or pointers do not allow 16-byte access take a scalar two-pass kernel.
#include "device_utils.hpp"
#include "launch.hpp"

namespace anygpu {

namespace {

template <typename T> struct NormVec;
template <> struct NormVec<float> { typedef float4_t type; static constexpr int kLen = 4; };
template <> struct NormVec<half_t> { typedef half8_t type; static constexpr int kLen = 8; };

__device__ __forceinline__ float silu_gate(float v) { return v * fast_rcp(1.0f + fast_exp2(-v * kLog2e)); }

// sum over the 256 threads of a block; every thread gets the result
__device__ __forceinline__ float block_sum(float v, float* slots)
{
	v = wave_allreduce(v, SumOp());
	if ((threadIdx.x & (kWaveSize - 1)) == 0) slots[threadIdx.x >> 6] = v;
	__syncthreads();
	return (slots[0] + slots[1]) + (slots[2] + slots[3]);
}

// GROUP threads share a row (16, 64 or 256), 256 / GROUP rows share a block.
template <typename T, int VPT, bool GATED, int GROUP>
__global__ __launch_bounds__(256) void gated_rmsnorm_row_kernel(
	const T* __restrict__ x, const T* __restrict__ z, const T* __restrict__ w, T* __restrict__ y,
	int64_t rows, int cols, float eps, float delta)
{
	static_assert(GROUP == 16 || GROUP == 64 || GROUP == 256, "a row of lanes, a wave or the block per row");
	typedef typename NormVec<T>::type vec_t;
	constexpr int VEC = NormVec<T>::kLen;
	__shared__ float slots[4];
	const int64_t row = (int64_t)blockIdx.x * (256 / GROUP) + threadIdx.x / GROUP;
	const int lane = threadIdx.x % GROUP;
	if (row >= rows) return;                    // uniform over the group (GROUP == 256: never taken)
	const vec_t* xr = reinterpret_cast<const vec_t*>(x + row * cols);
	const vec_t* zr = reinterpret_cast<const vec_t*>(z + row * cols);
	const vec_t* wr = reinterpret_cast<const vec_t*>(w);
	vec_t* yr = reinterpret_cast<vec_t*>(y + row * cols);
	const int nvec = cols / VEC;

	float g[VPT][VEC];
	float ss = 0.0f;
#pragma unroll
	for (int i = 0; i < VPT; ++i)
	{
		const int v = lane + GROUP * i;
		vec_t xv = {}, zv = {};
		if (v < nvec)
		{
			xv = __builtin_nontemporal_load(xr + v);
			if (GATED) zv = __builtin_nontemporal_load(zr + v);
		}
#pragma unroll
		for (int e = 0; e < VEC; ++e)
		{
			const float val = GATED ? (float)xv[e] * silu_gate((float)zv[e]) : (float)xv[e];
			g[i][e] = val;
			ss += val * val;
		}
	}
	ss = GROUP == 16 ? row_allreduce(ss, SumOp()) : GROUP == 64 ? wave_allreduce(ss, SumOp()) : block_sum(ss, slots);
	const float scale = 1.0f / sqrtf(ss / (float)cols + eps);
#pragma unroll
	for (int i = 0; i < VPT; ++i)
	{
		const int v = lane + GROUP * i;
		if (v < nvec)
		{
			const vec_t wv = wr[v];
			vec_t out;
#pragma unroll
			for (int e = 0; e < VEC; ++e) out[e] = (T)(g[i][e] * scale * ((float)wv[e] + delta));
			__builtin_nontemporal_store(out, yr + v);
		}
	}
}

// Rows longer than a block keeps in registers: 1024 threads walk the row twice with 16-byte accesses, four per thread
// in flight (the second time the row comes out of the L2).
template <typename T, bool GATED>
__global__ __launch_bounds__(1024) void gated_rmsnorm_long_kernel(
	const T* __restrict__ x, const T* __restrict__ z, const T* __restrict__ w, T* __restrict__ y,
	int64_t cols, float eps, float delta)
{
	typedef typename NormVec<T>::type vec_t;
	constexpr int VEC = NormVec<T>::kLen, kThreads = 1024, kAhead = 4;
	__shared__ float slots[16];
	const int64_t row = blockIdx.x;
	const vec_t* xr = reinterpret_cast<const vec_t*>(x + row * cols);
	const vec_t* zr = reinterpret_cast<const vec_t*>(z + row * cols);
	const vec_t* wr = reinterpret_cast<const vec_t*>(w);
	vec_t* yr = reinterpret_cast<vec_t*>(y + row * cols);
	const int64_t nvec = cols / VEC;
	float ss = 0.0f;
	for (int64_t v0 = threadIdx.x; v0 < nvec; v0 += (int64_t)kThreads * kAhead)
	{
		vec_t xv[kAhead], zv[kAhead];
#pragma unroll
		for (int u = 0; u < kAhead; ++u)
		{
			const int64_t v = v0 + (int64_t)u * kThreads;
			xv[u] = vec_t{};
			zv[u] = vec_t{};
			if (v < nvec)
			{
				xv[u] = xr[v];
				if (GATED) zv[u] = zr[v];
			}
		}
#pragma unroll
		for (int u = 0; u < kAhead; ++u)
#pragma unroll
			for (int e = 0; e < VEC; ++e)
			{
				const float val = GATED ? (float)xv[u][e] * silu_gate((float)zv[u][e]) : (float)xv[u][e];
				ss += val * val;
			}
	}
	ss = wave_allreduce(ss, SumOp());
	if ((threadIdx.x & (kWaveSize - 1)) == 0) slots[threadIdx.x >> 6] = ss;
	__syncthreads();
	ss = 0.0f;
#pragma unroll
	for (int i = 0; i < 16; ++i) ss += slots[i];
	const float scale = 1.0f / sqrtf(ss / (float)cols + eps);
	for (int64_t v0 = threadIdx.x; v0 < nvec; v0 += (int64_t)kThreads * kAhead)
	{
		vec_t xv[kAhead], zv[kAhead], wv[kAhead];
#pragma unroll
		for (int u = 0; u < kAhead; ++u)
		{
			const int64_t v = v0 + (int64_t)u * kThreads;
			xv[u] = vec_t{};
			zv[u] = vec_t{};
			wv[u] = vec_t{};
			if (v < nvec)
			{
				xv[u] = xr[v];
				if (GATED) zv[u] = zr[v];
				wv[u] = wr[v];
			}
		}
#pragma unroll
		for (int u = 0; u < kAhead; ++u)
		{
			const int64_t v = v0 + (int64_t)u * kThreads;
			if (v >= nvec) continue;
			vec_t out;
#pragma unroll
			for (int e = 0; e < VEC; ++e)
			{
				const float val = GATED ? (float)xv[u][e] * silu_gate((float)zv[u][e]) : (float)xv[u][e];
				out[e] = (T)(val * scale * ((float)wv[u][e] + delta));
			}
			__builtin_nontemporal_store(out, yr + v);
		}
	}
}

template <typename T, bool GATED>
__global__ __launch_bounds__(256) void gated_rmsnorm_two_pass_kernel(
	const T* __restrict__ x, const T* __restrict__ z, const T* __restrict__ w, T* __restrict__ y,
	int64_t cols, float eps, float delta)
{
	__shared__ float slots[4];
	const int64_t row = blockIdx.x;
	const T* xr = x + row * cols;
	const T* zr = z + row * cols;
	T* yr = y + row * cols;
	float ss = 0.0f;
	for (int64_t c = threadIdx.x; c < cols; c += 256)
	{
		const float val = GATED ? (float)xr[c] * silu_gate((float)zr[c]) : (float)xr[c];
		ss += val * val;
	}
	ss = block_sum(ss, slots);
	const float scale = 1.0f / sqrtf(ss / (float)cols + eps);
	for (int64_t c = threadIdx.x; c < cols; c += 256)
	{
		const float val = GATED ? (float)xr[c] * silu_gate((float)zr[c]) : (float)xr[c];
		yr[c] = (T)(val * scale * ((float)w[c] + delta));
	}
}

template <typename T, bool GATED>
hipError_t launch_gated(const T* x, const T* z, const T* w, T* y, int64_t rows, int64_t cols, float eps, float delta,
                        hipStream_t stream)
{
	constexpr int VEC = NormVec<T>::kLen;
	const dim3 grid((unsigned)rows), block(256);
	const bool vec_ok = cols % VEC == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
	                    reinterpret_cast<uintptr_t>(w) % 16 == 0 && (!GATED || reinterpret_cast<uintptr_t>(z) % 16 == 0);
	const int64_t nvec = cols / VEC;
	discard_stale_error();
#define ANYGPU_NORM_ROWS(VPT, GROUP) \
	gated_rmsnorm_row_kernel<T, VPT, GATED, GROUP><<<dim3((unsigned)((rows + 256 / GROUP - 1) / (256 / GROUP))), block, 0, stream>>>( \
		x, z, w, y, rows, (int)cols, eps, delta)
	if (vec_ok && nvec <= 16) ANYGPU_NORM_ROWS(1, 16);
	else if (vec_ok && nvec <= 32) ANYGPU_NORM_ROWS(2, 16);
	else if (vec_ok && nvec <= 64) ANYGPU_NORM_ROWS(1, 64);
	else if (vec_ok && nvec <= 128) ANYGPU_NORM_ROWS(2, 64);
	else if (vec_ok && nvec <= 256) ANYGPU_NORM_ROWS(1, 256);
	else if (vec_ok && nvec <= 512) ANYGPU_NORM_ROWS(2, 256);
	else if (vec_ok && nvec <= 1024) ANYGPU_NORM_ROWS(4, 256);
	else if (vec_ok && nvec <= 2048) ANYGPU_NORM_ROWS(8, 256);
	else if (vec_ok)
		gated_rmsnorm_long_kernel<T, GATED><<<grid, dim3(1024), 0, stream>>>(x, z, w, y, cols, eps, delta);
	else
		gated_rmsnorm_two_pass_kernel<T, GATED><<<grid, block, 0, stream>>>(x, z, w, y, cols, eps, delta);
#undef ANYGPU_NORM_ROWS
	return hipGetLastError();
}

}  // namespace

template <typename T>
hipError_t launch_gated_rmsnorm(const void* x, const void* z, const void* w, void* y, int64_t rows, int64_t cols,
                                float eps, int zero_centered, hipStream_t stream)
{
	if (rows == 0 || cols == 0) return hipSuccess;
	const float delta = zero_centered ? 1.0f : 0.0f;
	const T* xp = static_cast<const T*>(x);
	const T* wp = static_cast<const T*>(w);
	T* yp = static_cast<T*>(y);
	if (z != nullptr) return launch_gated<T, true>(xp, static_cast<const T*>(z), wp, yp, rows, cols, eps, delta, stream);
	return launch_gated<T, false>(xp, xp, wp, yp, rows, cols, eps, delta, stream);
}

template hipError_t launch_gated_rmsnorm<float>(const void*, const void*, const void*, void*, int64_t, int64_t, float, int, hipStream_t);
template hipError_t launch_gated_rmsnorm<half_t>(const void*, const void*, const void*, void*, int64_t, int64_t, float, int, hipStream_t);

}  // namespace anygpu
