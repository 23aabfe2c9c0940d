// Gated RMS normalisation over the last axis for gfx950:
//   g = x * silu(z)   (g = x when there is no gate)
//   y = g / sqrt(mean(g^2) + eps) * (w + delta),   delta = 1 for zero-centred weights, else 0
// The step between the SSD scan and the output projection of a Mamba2 mixer.  HBM-bound: x and z are
// read once, y is written once, the row lives in registers between the sum of squares and the
// scaling.  One 256-thread block per row, 16-byte accesses; the row length picks how many vectors a
// thread keeps (1, 2, 4 or 8: up to 8192 floats or 16384 halves).  Longer rows, and rows whose
// length or pointers do not allow 16-byte access, take a two-pass kernel that reads x and z twice.
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

template <typename T, int VPT, bool GATED>
__global__ __launch_bounds__(256) void gated_rmsnorm_row_kernel(
	const T* __restrict__ x, const T* __restrict__ z, const T* __restrict__ w, T* __restrict__ y,
	int cols, float eps, float delta)
{
	typedef typename NormVec<T>::type vec_t;
	constexpr int VEC = NormVec<T>::kLen;
	__shared__ float slots[4];
	const int64_t row = blockIdx.x;
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
		const int v = threadIdx.x + 256 * i;
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
	ss = block_sum(ss, slots);
	const float scale = 1.0f / sqrtf(ss / (float)cols + eps);
#pragma unroll
	for (int i = 0; i < VPT; ++i)
	{
		const int v = threadIdx.x + 256 * i;
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
	if (vec_ok && nvec <= 256)
		gated_rmsnorm_row_kernel<T, 1, GATED><<<grid, block, 0, stream>>>(x, z, w, y, (int)cols, eps, delta);
	else if (vec_ok && nvec <= 512)
		gated_rmsnorm_row_kernel<T, 2, GATED><<<grid, block, 0, stream>>>(x, z, w, y, (int)cols, eps, delta);
	else if (vec_ok && nvec <= 1024)
		gated_rmsnorm_row_kernel<T, 4, GATED><<<grid, block, 0, stream>>>(x, z, w, y, (int)cols, eps, delta);
	else if (vec_ok && nvec <= 2048)
		gated_rmsnorm_row_kernel<T, 8, GATED><<<grid, block, 0, stream>>>(x, z, w, y, (int)cols, eps, delta);
	else
		gated_rmsnorm_two_pass_kernel<T, GATED><<<grid, block, 0, stream>>>(x, z, w, y, cols, eps, delta);
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
