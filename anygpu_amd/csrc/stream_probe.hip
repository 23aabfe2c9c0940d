// Measurement hook: a plain streaming kernel (read n bytes, write n bytes, 16 bytes per lane and access) in the
// launch geometries a memory-bound kernel of this library can choose from, so that a benchmark can state what
// read + write bandwidth the memory system of the box at hand gives such a kernel, in the same run as the kernels
// it judges against that figure.
#include "device_utils.hpp"
#include "launch.hpp"

namespace anygpu {

typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));

// A block copies VPL * blockDim.x consecutive vectors: vector u * blockDim.x + tid for u < VPL, all loads issued before
// the first store.  ROUNDS > 0: the grid is smaller than the tile count and a block walks tiles blockIdx.x,
// + gridDim.x, ... (a persistent launch).
template <int VPL, bool NT_LOAD, bool NT_STORE>
__global__ void stream_copy_kernel(const uint4_t* __restrict__ src, uint4_t* __restrict__ dst, int64_t nvec, int64_t tiles)
{
	const int per_tile = VPL * (int)blockDim.x;
	for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x)
	{
		const int64_t base = tile * per_tile + threadIdx.x;
		uint4_t v[VPL];
#pragma unroll
		for (int u = 0; u < VPL; ++u)
		{
			const int64_t i = base + (int64_t)u * blockDim.x;
			if (i < nvec) v[u] = NT_LOAD ? __builtin_nontemporal_load(src + i) : src[i];
		}
#pragma unroll
		for (int u = 0; u < VPL; ++u)
		{
			const int64_t i = base + (int64_t)u * blockDim.x;
			if (i < nvec)
			{
				if (NT_STORE) __builtin_nontemporal_store(v[u], dst + i);
				else dst[i] = v[u];
			}
		}
	}
}

template <int VPL>
static hipError_t launch_vpl(const void* src, void* dst, int64_t nvec, int block, int nt_load, int nt_store, int64_t grid_limit,
                             hipStream_t stream)
{
	const int64_t tiles = (nvec + (int64_t)VPL * block - 1) / ((int64_t)VPL * block);
	const int64_t grid = grid_limit > 0 && grid_limit < tiles ? grid_limit : tiles;
	const auto* s = static_cast<const uint4_t*>(src);
	auto* d = static_cast<uint4_t*>(dst);
	if (nt_load && nt_store) stream_copy_kernel<VPL, true, true><<<dim3((unsigned)grid), dim3(block), 0, stream>>>(s, d, nvec, tiles);
	else if (nt_load) stream_copy_kernel<VPL, true, false><<<dim3((unsigned)grid), dim3(block), 0, stream>>>(s, d, nvec, tiles);
	else if (nt_store) stream_copy_kernel<VPL, false, true><<<dim3((unsigned)grid), dim3(block), 0, stream>>>(s, d, nvec, tiles);
	else stream_copy_kernel<VPL, false, false><<<dim3((unsigned)grid), dim3(block), 0, stream>>>(s, d, nvec, tiles);
	return hipGetLastError();
}

hipError_t launch_stream_probe(const void* src, void* dst, int64_t nvec, int block, int vectors_per_lane, int nt_load,
                               int nt_store, int64_t grid_limit, hipStream_t stream)
{
	discard_stale_error();
	switch (vectors_per_lane)
	{
	case 1: return launch_vpl<1>(src, dst, nvec, block, nt_load, nt_store, grid_limit, stream);
	case 2: return launch_vpl<2>(src, dst, nvec, block, nt_load, nt_store, grid_limit, stream);
	case 4: return launch_vpl<4>(src, dst, nvec, block, nt_load, nt_store, grid_limit, stream);
	case 8: return launch_vpl<8>(src, dst, nvec, block, nt_load, nt_store, grid_limit, stream);
	default: return hipErrorInvalidValue;
	}
}

}  // namespace anygpu
