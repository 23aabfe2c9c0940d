// .dat tensor files: little-endian int32 dim, int32 shape[dim], int32 dtype code, then the raw
// elements in default (row-major) order.  dtype codes: INT8 0, INT16 1, INT32 2, BFLOAT16 3,
// FLOAT16 4, FLOAT32 5, FLOAT64 6.  Reference: srcs/io/dat_file.hpp:8-94 (reader only there;
// the writer here is the mirror image, matching scripts/dnn_inspector/dnninspect/tensor.py:76-110).
#ifndef __DAT_FILE__
#define __DAT_FILE__

#include "tensor.hpp"

namespace dat_detail {

template<typename T> constexpr int32 dtype_code()
{
	if constexpr (std::is_same_v<T, int8>) return 0;
	else if constexpr (std::is_same_v<T, int16>) return 1;
	else if constexpr (std::is_same_v<T, int32>) return 2;
	else if constexpr (std::is_same_v<T, bfloat16>) return 3;
	else if constexpr (std::is_same_v<T, float16>) return 4;
	else if constexpr (std::is_same_v<T, float32>) return 5;
	else
	{
		static_assert(std::is_same_v<T, float64>, "Unsupported data type");
		return 6;
	}
}

}  // namespace dat_detail

/* Reads a tensor; a missing file or a dtype code other than T's is fail-stop. */
template<typename T = float32>
inline Tensor<T, CPU> load_tensor(const std::string& file_path)
{
	std::ifstream file(file_path, std::ios::binary);
	const std::string open_msg = "Unable to open file: " + file_path;
	ACASSERT(file.is_open(), open_msg.c_str());

	auto read_i32 = [&file]() { int32 v = 0; file.read(reinterpret_cast<char*>(&v), sizeof(v)); return v; };

	const int32 dim = read_i32();
	ACASSERT(dim > 0 && dim <= MAX_TENSOR_DIM, "Tensor data file has an unsupported number of dimensions");
	std::vector<int64> shape(static_cast<size_t>(dim));
	for (auto& s : shape) s = read_i32();
	const int32 code = read_i32();
	const std::string type_msg = "Data type in tensor data file expected to be " + represent_datatype<T>();
	ACASSERT(code == dat_detail::dtype_code<T>(), type_msg.c_str());

	Tensor<T, CPU> tensor(shape);
	file.read(reinterpret_cast<char*>(tensor.buffer()), static_cast<std::streamsize>(sizeof(T) * tensor.numel()));
	if (!file)
	{
		const std::string msg = "Error during processing tensor data file: " + file_path;
		log_error(msg.c_str());
	}
	return tensor;
}

/* Writes a dense host tensor. */
template<typename T>
inline void save_tensor(const Tensor<T, CPU>& tensor, const std::string& file_path)
{
	std::ofstream file(file_path, std::ios::binary);
	const std::string open_msg = "Unable to open file: " + file_path;
	ACASSERT(file.is_open(), open_msg.c_str());
	auto write_i32 = [&file](int32 v) { file.write(reinterpret_cast<const char*>(&v), sizeof(v)); };
	write_i32(static_cast<int32>(tensor.dim));
	for (int64 ix = 0; ix < tensor.dim; ++ix) write_i32(static_cast<int32>(tensor.shape[ix]));
	write_i32(dat_detail::dtype_code<T>());
	file.write(reinterpret_cast<const char*>(tensor.buffer()), static_cast<std::streamsize>(sizeof(T) * tensor.numel()));
}

#endif  // __DAT_FILE__
