// Core vocabulary of the host layer: element type aliases, the Device tag, shape helpers,
// logging / assertion macros and the error-check macros used around runtime calls.
//
// Same public names as the reference's srcs/core/core.hpp (dtype aliases :32-41, DimArray :62-67,
// Device :75-79, DataType :81-93, get_datatype_enum :101-145, ACASSERT :408-422,
// CUDA_CHECK :445-475) so that operator, model and test code written against it compiles
// unchanged.  `Device::CUDA` is kept as the tag for "the GPU"; behind it sits HIP on gfx950.
// This header pulls in no GPU runtime header: device memory is reached through
// device_memory.hpp, so host-only translation units build with any C++20 compiler.
#ifndef __CORE__
#define __CORE__

#include <algorithm>
#include <array>
#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <filesystem>
#include <fstream>
#include <functional>
#include <iostream>
#include <sstream>
#include <string>
#include <type_traits>
#include <unordered_map>
#include <vector>

#include "small_floats.hpp"

/* element types */

using int8 = char;
using int16 = short signed int;
using int32 = signed int;
using int64 = long long;
using bfloat16 = anygpu_host::BFloat16;
using float16 = _Float16;
using float32 = float;
using float64 = double;
using fp8e4m3 = anygpu_host::Fp8E4M3;
using fp8e5m2 = anygpu_host::Fp8E5M2;

enum Device
{
	CPU,
	CUDA   // the GPU: an MI355X driven through HIP
};

enum class DataType
{
	INT8,
	INT16,
	INT32,
	INT64,
	BFLOAT16,
	FLOAT16,
	FLOAT32,
	FLOAT64,
	FP8E4M3,
	FP8E5M2
};

// One row per DataType enumerator, in enumerator order.
struct DataTypeInfo
{
	const char* name;
	int64 bits;
	int64 bytes;   // sub-byte types count as one byte for alignment purposes
};

inline constexpr DataTypeInfo datatype_table[] = {
	{ "INT8", 8, 1 },     { "INT16", 16, 2 },    { "INT32", 32, 4 },   { "INT64", 64, 8 },   { "BFLOAT16", 16, 2 },
	{ "FLOAT16", 16, 2 }, { "FLOAT32", 32, 4 },  { "FLOAT64", 64, 8 }, { "FP8E4M3", 8, 1 },  { "FP8E5M2", 8, 1 },
};

template<typename T> inline int64 get_bitsize()
{
	return static_cast<int64>(sizeof(T) * 8);
}

template<typename T> inline DataType get_datatype_enum()
{
	if constexpr (std::is_same_v<T, float32>) return DataType::FLOAT32;
	else if constexpr (std::is_same_v<T, float64>) return DataType::FLOAT64;
	else if constexpr (std::is_same_v<T, float16>) return DataType::FLOAT16;
	else if constexpr (std::is_same_v<T, bfloat16>) return DataType::BFLOAT16;
	else if constexpr (std::is_same_v<T, fp8e4m3>) return DataType::FP8E4M3;
	else if constexpr (std::is_same_v<T, fp8e5m2>) return DataType::FP8E5M2;
	else if constexpr (std::is_same_v<T, int32>) return DataType::INT32;
	else if constexpr (std::is_same_v<T, int64>) return DataType::INT64;
	else if constexpr (std::is_same_v<T, int16>) return DataType::INT16;
	else
	{
		static_assert(std::is_same_v<T, int8>, "unknown data type");
		return DataType::INT8;
	}
}

std::string represent_datatype(const DataType dtype);
template<typename dtype> inline std::string represent_datatype() { return represent_datatype(get_datatype_enum<dtype>()); }
std::ostream& operator<<(std::ostream& os, const DataType dtype);
std::string represent_device(const Device device);
std::ostream& operator<<(std::ostream& os, const Device device);

/* shapes */

const int MAX_TENSOR_DIM = 8;

using DimArray = std::array<int64, MAX_TENSOR_DIM>;
using Shape = DimArray;
using Stride = DimArray;
using Index = DimArray;

bool equal(const int64 dim, const DimArray& lhs, const DimArray& rhs);
void increment_index(const int64 dim, const Shape& shape, Index& index);
int64 calculate_offset(const int64 dim, const Stride& strides, const Index& index);
std::string represent_array(const int64 dim, const DimArray& arr);   // "[d1, d2, d3]"

int64 calc_default_size(const std::vector<int64>& shape);
int64 calc_default_size(const int64 dim, const DimArray& shape);
std::vector<int64> calc_default_stride(const std::vector<int64>& shape);
DimArray calc_default_stride(const int64 dim, const DimArray& shape);
DimArray cvt_vector2array(const std::vector<int64>& v);
std::vector<int64> cvt_array2vector(const int64 dim, const DimArray& arr);
int64 calc_dim(const std::vector<int64>& v);

/* conversions */

template<typename T>
inline std::vector<T> cvt_int_vector_to_any(const std::vector<int>& hdata)
{
	std::vector<T> out_data(hdata.size());
	std::transform(hdata.begin(), hdata.end(), out_data.begin(),
		[](int v) { return static_cast<T>(static_cast<float>(v)); });
	return out_data;
}

template<typename T>
inline float32 cvt_any_to_float32(const T value)
{
	return static_cast<float32>(value);
}

/* ids, alignment */

class GlobalUUIDGenerator
{
public:
	static int64 generate_id();

private:
	static int64 next_id;
};

constexpr int64 BYTE_EXP = 3;
constexpr int64 BYTE_SIZE = 8;
constexpr int64 ALIGNMENT_EXP = 8;
constexpr int64 ALIGNMENT_SIZE = 256;

struct alignas(ALIGNMENT_SIZE) AlignedType
{
	char data[ALIGNMENT_SIZE];
};

/* logging and assertions: failures are fail-stop (message, then exit(1)) */

enum class LogLevel
{
	LEVEL_INFO,
	LEVEL_WARNING,
	LEVEL_ERROR
};

void log_message(LogLevel llevel, const std::string& msg);
inline void log_info(const char* cmsg) { log_message(LogLevel::LEVEL_INFO, cmsg); }
inline void log_warning(const char* cmsg) { log_message(LogLevel::LEVEL_WARNING, cmsg); }
inline void log_error(const char* cmsg) { log_message(LogLevel::LEVEL_ERROR, cmsg); }

[[noreturn]] void fail_assert(const char* file, int line, const char* msg);
[[noreturn]] void fail_runtime(int code, const char* what, const char* file, int line);

#ifdef AC_WITH_ASSERT
#define ACASSERT( expression, msg )                          \
	do {                                                     \
		if (!(expression)) fail_assert(__FILE__, __LINE__, (msg)); \
	} while (0)
#else
#define ACASSERT( expression, msg ) ((void)0)
#endif

/* launch geometry (kept for API parity; the HIP launchers size their own grids) */

struct LaunchDim
{
	unsigned int x = 1, y = 1, z = 1;
};

struct KernelParameters
{
	LaunchDim grid_size;
	LaunchDim block_size;
};

unsigned int calc_req_num_blocks(unsigned int num_elements, unsigned int block_size);

/* Prints the properties of GPU 0 (name, compute units, LDS, memory, launch limits). */
std::string print_cuda_device_props();

/*
  Error checks around runtime and kernel-library calls.  `fn` evaluates to an integer status
  where 0 is success: a hipError_t, or a code of the anygpu C ABI.
*/
#define HIP_CHECK( fn )                                                  \
	do {                                                                 \
		const int res__ = static_cast<int>(fn);                          \
		if (res__ != 0) fail_runtime(res__, #fn, __FILE__, __LINE__);    \
	} while (0)

#define CUDA_CHECK( fn ) HIP_CHECK( fn )

int last_device_error();   // reads and clears the runtime's last-error slot
#define CUDA_CHECK_LAST_ERROR( ) HIP_CHECK( last_device_error() )
#define HIP_CHECK_LAST_ERROR( ) HIP_CHECK( last_device_error() )

#endif  // __CORE__
