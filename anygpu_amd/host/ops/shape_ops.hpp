// Metadata-only shape operators: new views over an existing buffer, no data movement
// (reference: srcs/ops/shape_ops.hpp:10-41).
#ifndef __SHAPE_OPS__
#define __SHAPE_OPS__

#include "tensor.hpp"
#include "core_concepts.hpp"

/* The same buffer seen with another (dense, row-major) shape. */
template<ArithmeticType dtype, Device device>
inline Tensor<dtype, device> tensor_view(const Tensor<dtype, device>& x, const std::vector<int64>& new_shape)
{
	Tensor<dtype, device> y(x);
	y.id = GlobalUUIDGenerator::generate_id();
	y.name.clear();
	y.dim = calc_dim(new_shape);
	y.shape = cvt_vector2array(new_shape);
	y.stride = cvt_vector2array(calc_default_stride(new_shape));
	return y;
}

/* `splits` equal pieces along axis 0, each a view at its own byte offset. */
template<ArithmeticType dtype, Device device>
inline std::vector<Tensor<dtype, device>> tensor_split(const Tensor<dtype, device>& x, const int64 splits)
{
	std::vector<Tensor<dtype, device>> pieces(static_cast<size_t>(splits), x);
	const int64 rows_per_piece = x.shape[0] / splits;
	for (int64 ix = 0; ix < splits; ++ix)
	{
		auto& y = pieces[static_cast<size_t>(ix)];
		y.name.clear();
		y.shape[0] = rows_per_piece;
		y.stride = calc_default_stride(y.dim, y.shape);
		y.offset = x.offset + ix * rows_per_piece * y.stride[0] * static_cast<int64>(sizeof(dtype));
	}
	return pieces;
}

#endif  // __SHAPE_OPS__
