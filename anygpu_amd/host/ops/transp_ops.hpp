// Transpose of a 2-D host tensor.  The path needs it in one place only: weights stored [out, in] are
// turned into [in, out] on the host when they are loaded (GPU products that can take the [out, in]
// storage directly use tensor_mm_nt instead).  Reference: srcs/ops/transp_ops.hpp:12-47.
#ifndef __TRANSP_OPS__
#define __TRANSP_OPS__

#include "tensor.hpp"
#include "core_concepts.hpp"

template<NotHalfFloatType dtype>
inline Tensor<dtype, CPU> tensor_transp(const Tensor<dtype, CPU>& x)
{
	ACASSERT(x.dim == 2, "transpose expects 2 dimensional tensors");
	const int64 rows = x.shape[0], cols = x.shape[1];
	Tensor<dtype, CPU> y(std::vector<int64>({ cols, rows }));
	const dtype* src = x.buffer();
	dtype* dst = y.buffer();
	for (int64 c = 0; c < cols; ++c)            // walk the result row by row
		for (int64 r = 0; r < rows; ++r)
			dst[c * y.stride[0] + r * y.stride[1]] = src[r * x.stride[0] + c * x.stride[1]];
	return y;
}

#endif  // __TRANSP_OPS__
