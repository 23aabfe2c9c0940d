#include "core.hpp"

#include <numeric>

bool equal(const int64 dim, const DimArray& lhs, const DimArray& rhs)
{
	return std::equal(lhs.begin(), lhs.begin() + dim, rhs.begin());
}

void increment_index(const int64 dim, const Shape& shape, Index& index)
{
	// odometer step, last axis fastest; wraps to all zeros after the last element
	for (int64 axis = dim - 1; axis >= 0; --axis)
	{
		if (index[axis] + 1 < shape[axis])
		{
			index[axis] += 1;
			return;
		}
		index[axis] = 0;
	}
}

int64 calculate_offset(const int64 dim, const Stride& strides, const Index& index)
{
	return std::inner_product(strides.begin(), strides.begin() + dim, index.begin(), int64(0));
}

std::string represent_datatype(const DataType dtype)
{
	const auto ix = static_cast<unsigned int>(dtype);
	ACASSERT(ix < std::size(datatype_table), "Unknown data type");
	return datatype_table[ix].name;
}

std::ostream& operator<<(std::ostream& os, const DataType dtype)
{
	return os << represent_datatype(dtype);
}

std::string represent_device(const Device device)
{
	ACASSERT(device == CPU || device == CUDA, "Unknown device type");
	return device == CPU ? "CPU" : "CUDA";
}

std::ostream& operator<<(std::ostream& os, const Device device)
{
	return os << represent_device(device);
}

std::string represent_array(const int64 dim, const DimArray& arr)
{
	std::stringstream ss;
	ss << "[";
	for (int64 ix = 0; ix < dim; ++ix)
	{
		ss << (ix ? ", " : "") << arr[ix];
	}
	ss << "]";
	return ss.str();
}

unsigned int calc_req_num_blocks(unsigned int num_elements, unsigned int block_size)
{
	return (num_elements + block_size - 1) / block_size;
}

int64 GlobalUUIDGenerator::next_id = 0;

int64 GlobalUUIDGenerator::generate_id()
{
	return next_id++;
}

int64 calc_default_size(const std::vector<int64>& shape)
{
	return std::accumulate(shape.begin(), shape.end(), int64(1), std::multiplies<int64>());
}

int64 calc_default_size(const int64 dim, const DimArray& shape)
{
	return std::accumulate(shape.begin(), shape.begin() + dim, int64(1), std::multiplies<int64>());
}

std::vector<int64> calc_default_stride(const std::vector<int64>& shape)
{
	std::vector<int64> stride(shape.size(), 1);
	for (int64 axis = calc_dim(shape) - 2; axis >= 0; --axis)
	{
		stride[axis] = stride[axis + 1] * shape[axis + 1];
	}
	return stride;
}

DimArray calc_default_stride(const int64 dim, const DimArray& shape)
{
	DimArray stride = {};
	if (dim > 0) stride[dim - 1] = 1;
	for (int64 axis = dim - 2; axis >= 0; --axis)
	{
		stride[axis] = stride[axis + 1] * shape[axis + 1];
	}
	return stride;
}

DimArray cvt_vector2array(const std::vector<int64>& v)
{
	DimArray arr = {};
	std::copy(v.begin(), v.end(), arr.begin());
	return arr;
}

std::vector<int64> cvt_array2vector(const int64 dim, const DimArray& arr)
{
	return std::vector<int64>(arr.begin(), arr.begin() + dim);
}

int64 calc_dim(const std::vector<int64>& v)
{
	return static_cast<int64>(v.size());
}

void log_message(LogLevel llevel, const std::string& msg)
{
	static const char* prefix[] = { "\033[33m[INFO    ", "\033[36m[WARNING ", "\033[91m[ERROR   " };
	std::cout << prefix[static_cast<int>(llevel)] << "] " << msg << "\033[m" << std::endl;
}

void fail_assert(const char* file, int line, const char* msg)
{
	std::cout << file << " " << line << '\n';
	log_error(msg);
	std::exit(1);
}

void fail_runtime(int code, const char* what, const char* file, int line)
{
	std::stringstream ss;
	ss << "code: " << code << " file: " << file << " ln: " << line << " in: " << what << "\n";
	log_error(ss.str().c_str());
	std::exit(1);
}
