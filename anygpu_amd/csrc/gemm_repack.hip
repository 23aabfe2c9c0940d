// Aligned copies of GEMM operands the MFMA kernels cannot fetch as they lie.
//
// The tile kernels fetch operands in aligned 16-byte chunks along K.  An operand that starts at an odd address, has a row
// pitch or a K that is no multiple of 8 elements, or (weights stored [K, N]) an N that is none, used to fall to a kernel
// that loads element by element and ran at a third of the speed.  Instead such an operand is copied once into the
// stream's workspace as k-contiguous rows of a pitch that is a multiple of 64 elements, zeros behind K, and the product
// runs on the copy with the ordinary kernels: a copy moves the operand twice through HBM (4096 x 4100 halves: 34 MB read,
// 34 MB written) where the product itself takes several times that long.
#include "device_utils.hpp"
#include "launch.hpp"

namespace anygpu {

namespace {

typedef unsigned uint4_t __attribute__((ext_vector_type(4)));

// The 16 bytes at `from` (any alignment), of which the first `valid` (0 .. 16) are data and the rest come back as zeros.
// Read as the one or two aligned 16-byte vectors that hold them and shifted into place: a lane that fetched element by
// element would keep the memory pipeline busy with 2 bytes per lane and instruction (a copy of 34 MB took 19 us that
// way).  Each vector holds at least one byte of data, so nothing outside the pages of the operand is touched.
__device__ __forceinline__ uint4_t load_16_bytes_anywhere(const char* from, int valid)
{
	uint4_t out = {0u, 0u, 0u, 0u};
	if (valid <= 0) return out;
	const uintptr_t s = reinterpret_cast<uintptr_t>(from);
	const unsigned r = (unsigned)(s & 15);
	const uint4_t* base = reinterpret_cast<const uint4_t*>(s - r);
	const uint4_t lo = base[0];
	uint4_t hi = {0u, 0u, 0u, 0u};
	if (r + (unsigned)valid > 16) hi = base[1];
	const unsigned w[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
	const unsigned q = r >> 2, shift = r & 3;
	unsigned t[5];
#pragma unroll
	for (int i = 0; i < 5; ++i) t[i] = q == 0 ? w[i] : q == 1 ? w[i + 1] : q == 2 ? w[i + 2] : w[(i + 3) & 7];
#pragma unroll
	for (int i = 0; i < 4; ++i)
	{
		const unsigned word = __builtin_amdgcn_alignbyte(t[i + 1], t[i], shift);
		const int have = valid - 4 * i;                     // data bytes in this word
		out[i] = have >= 4 ? word : have <= 0 ? 0u : (word & (0xFFFFFFFFu >> (8 * (4 - have))));
	}
	return out;
}

// dst[row][c] = (row < rows && c < cols) ? src[row][c] : 0 for row < rows_dst, c < ld_dst; one thread per 16 bytes of dst
template <typename T>
__global__ __launch_bounds__(256) void repack_rows_kernel(const T* __restrict__ src, int64_t ld_src, int64_t rows, int64_t cols,
                                                          T* __restrict__ dst, int64_t ld_dst, int64_t rows_dst)
{
	constexpr int kPer = 16 / sizeof(T);
	const int64_t chunks = ld_dst / kPer;
	const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (item >= rows_dst * chunks) return;
	const int64_t row = item / chunks, c0 = (item % chunks) * kPer;
	const int64_t left = row < rows ? cols - c0 : 0;
	const int valid = left >= kPer ? 16 : left <= 0 ? 0 : (int)(left * sizeof(T));
	*reinterpret_cast<uint4_t*>(dst + row * ld_dst + c0) =
		load_16_bytes_anywhere(reinterpret_cast<const char*>(src + row * ld_src + c0), valid);
}

// dst[n][k] = k < k_rows ? src[k][n] : 0 for k < ld_dst (a multiple of 64), n < n_cols: 64 x 64 tiles through LDS, read
// along n and written along k, both in 16-byte vectors
template <typename T>
__global__ __launch_bounds__(256) void repack_transposed_kernel(const T* __restrict__ src, int64_t ld_src, int64_t k_rows, int64_t n_cols,
                                                                T* __restrict__ dst, int64_t ld_dst)
{
	constexpr int kPer = 16 / sizeof(T);
	typedef T Vec __attribute__((ext_vector_type(kPer)));
	constexpr int kPitch = 64 + kPer;                       // elements; keeps every tile row 16-byte aligned
	__shared__ __align__(16) T tile[64 * kPitch];
	const int64_t k0 = (int64_t)blockIdx.x * 64, n0 = (int64_t)blockIdx.y * 64;
	const int t = threadIdx.x;
	constexpr int kVecsPerRow = 64 / kPer;
#pragma unroll
	for (int i = 0; i < 64 * kVecsPerRow / 256; ++i)
	{
		const int v = t + 256 * i;
		const int k = v / kVecsPerRow, nc = (v % kVecsPerRow) * kPer;
		const int64_t left = n_cols - (n0 + nc);
		const int valid = k0 + k >= k_rows ? 0 : left >= kPer ? 16 : left <= 0 ? 0 : (int)(left * sizeof(T));
		*reinterpret_cast<uint4_t*>(tile + k * kPitch + nc) =
			load_16_bytes_anywhere(reinterpret_cast<const char*>(src + (k0 + k) * ld_src + n0 + nc), valid);
	}
	__syncthreads();
#pragma unroll
	for (int i = 0; i < 64 * kVecsPerRow / 256; ++i)
	{
		const int v = t + 256 * i;
		const int n = v / kVecsPerRow, kc = (v % kVecsPerRow) * kPer;
		if (n0 + n >= n_cols) continue;
		Vec out;
#pragma unroll
		for (int e = 0; e < kPer; ++e) out[e] = tile[(kc + e) * kPitch + n];
		*reinterpret_cast<Vec*>(dst + (n0 + n) * ld_dst + k0 + kc) = out;
	}
}

}  // namespace

hipError_t launch_repack_rows(const void* src, int64_t ld_src, int64_t rows, int64_t cols, void* dst, int64_t ld_dst,
                              int elem_bytes, hipStream_t stream, int64_t rows_dst)
{
	(void)hipGetLastError();
	if (rows_dst < rows) rows_dst = rows;
	const int64_t items = rows_dst * (ld_dst / (16 / elem_bytes));
	const dim3 grid((unsigned)((items + 255) / 256));
	if (elem_bytes == 2)
		repack_rows_kernel<uint16_t><<<grid, dim3(256), 0, stream>>>(static_cast<const uint16_t*>(src), ld_src, rows, cols, static_cast<uint16_t*>(dst), ld_dst, rows_dst);
	else
		repack_rows_kernel<uint32_t><<<grid, dim3(256), 0, stream>>>(static_cast<const uint32_t*>(src), ld_src, rows, cols, static_cast<uint32_t*>(dst), ld_dst, rows_dst);
	return hipGetLastError();
}

hipError_t launch_repack_transposed(const void* src, int64_t ld_src, int64_t k_rows, int64_t n_cols, void* dst, int64_t ld_dst,
                                    int elem_bytes, hipStream_t stream)
{
	(void)hipGetLastError();
	const dim3 grid((unsigned)(ld_dst / 64), (unsigned)((n_cols + 63) / 64));
	if (elem_bytes == 2)
		repack_transposed_kernel<uint16_t><<<grid, dim3(256), 0, stream>>>(static_cast<const uint16_t*>(src), ld_src, k_rows, n_cols, static_cast<uint16_t*>(dst), ld_dst);
	else
		repack_transposed_kernel<uint32_t><<<grid, dim3(256), 0, stream>>>(static_cast<const uint32_t*>(src), ld_src, k_rows, n_cols, static_cast<uint32_t*>(dst), ld_dst);
	return hipGetLastError();
}

}  // namespace anygpu
