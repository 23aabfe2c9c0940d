// Tensor<dtype, device>: a shape/stride view over a reference-counted flat buffer that lives
// either in host memory (Device::CPU) or in the GPU's HBM (Device::CUDA, backed by HIP).
//
// Field names, constructors and free functions follow the reference's srcs/core/tensor.hpp
// (MemoryBuffer :19-128, Tensor :147-247, copies :319-370, cvt_tensor_datatype :388-410,
// factories :465-547, compatibility checks :560-581) so that code written against it compiles
// unchanged.  Every new buffer is zero-filled; host buffers are 256-byte aligned.
#ifndef __TENSOR__
#define __TENSOR__

#include <memory>
#include <random>

#include "core.hpp"
#include "device_memory.hpp"

/*
  Flat storage for tensor elements, owned by one or more tensors.
    id       - unique per buffer
    capacity - size in bytes
    buffer   - start address (host pointer or device pointer, depending on `device`)
*/
template<Device device>
struct MemoryBuffer
{
	int64 id;
	int64 capacity;
	char* buffer;

	explicit MemoryBuffer() : id(GlobalUUIDGenerator::generate_id()), capacity(0), buffer(nullptr) {}

	explicit MemoryBuffer(const int64 capacity) : id(GlobalUUIDGenerator::generate_id()), capacity(capacity), buffer(nullptr)
	{
		acquire();
	}

	explicit MemoryBuffer(const int64 data_bit_size, const std::vector<int64>& shape)
		: MemoryBuffer(bytes_for(calc_default_size(shape), data_bit_size)) {}

	explicit MemoryBuffer(const int64 data_bit_size, const int64 dim, const Shape& shape)
		: MemoryBuffer(bytes_for(calc_default_size(dim, shape), data_bit_size)) {}

	MemoryBuffer(const MemoryBuffer&) = delete;
	MemoryBuffer& operator=(const MemoryBuffer&) = delete;

	~MemoryBuffer()
	{
		if (buffer == nullptr) return;
		if constexpr (device == Device::CPU) std::free(buffer);
		else device_memory::release(buffer);
		buffer = nullptr;
		capacity = 0;
	}

	// bytes needed for `elements` elements of `bits` bits each, rounded up to whole bytes
	static int64 bytes_for(const int64 elements, const int64 bits)
	{
		return (elements * bits + BYTE_SIZE - 1) >> BYTE_EXP;
	}

private:
	void acquire()
	{
		if (capacity <= 0) return;
		if constexpr (device == Device::CPU)
		{
			const int64 rounded = ((capacity + ALIGNMENT_SIZE - 1) >> ALIGNMENT_EXP) << ALIGNMENT_EXP;
			buffer = static_cast<char*>(std::aligned_alloc(ALIGNMENT_SIZE, static_cast<size_t>(rounded)));
			if (buffer == nullptr) fail_runtime(-1, "host allocation", __FILE__, __LINE__);
			std::memset(buffer, 0, static_cast<size_t>(rounded));
		}
		else
		{
			static_assert(device == Device::CUDA, "unknown device");
			buffer = device_memory::allocate_zeroed(capacity);
		}
	}
};


/*
  A tensor is a view: several tensors may share one buffer (views, splits, slices without copy).
    id        - unique per tensor object
    dim       - number of axes (<= MAX_TENSOR_DIM)
    offset    - start of this view inside the buffer, in BYTES
    alignment - alignment requirement of the innermost axis, in bytes
    shape / stride - extents and element strides per axis
*/
template<typename dtype, Device device = Device::CUDA>
struct Tensor
{
	int64 id;
	int64 dim;
	int64 offset;
	int64 alignment;
	Shape shape;
	Stride stride;
	std::string name;

	// first element of the view (offset applied)
	dtype* buffer() const { return reinterpret_cast<dtype*>(mem_buffer->buffer + offset); }

	// start of the underlying buffer (offset not applied)
	char* raw_buffer() const { return mem_buffer->buffer; }

	// number of elements, ignoring stride padding
	int64 numel() const { return calc_default_size(dim, shape); }

	// number of element slots spanned, stride padding included
	int64 size() const { return shape[0] * stride[0]; }

	// bytes held by the underlying buffer
	int64 capacity() const { return mem_buffer->capacity; }

	int64 buffer_id() const { return mem_buffer->id; }

	Tensor<dtype, CPU> copy_to_host() const;
	Tensor<dtype, CUDA> copy_to_cuda() const;

	Tensor() : id(GlobalUUIDGenerator::generate_id()), dim(0), offset(0), alignment(1), shape{}, stride{} {}

	// raw byte buffer, no shape yet
	explicit Tensor(const int64 capacity) : Tensor()
	{
		mem_buffer = std::make_shared<MemoryBuffer<device>>(capacity);
	}

	// dense tensor, default (row-major) strides
	explicit Tensor(const std::vector<int64>& shape) : Tensor()
	{
		dim = calc_dim(shape);
		this->shape = cvt_vector2array(shape);
		this->stride = cvt_vector2array(calc_default_stride(shape));
		mem_buffer = std::make_shared<MemoryBuffer<device>>(get_bitsize<dtype>(), shape);
	}

	explicit Tensor(const int64 dim, const Shape& shape) : Tensor()
	{
		this->dim = dim;
		this->shape = shape;
		this->stride = calc_default_stride(dim, shape);
		mem_buffer = std::make_shared<MemoryBuffer<device>>(get_bitsize<dtype>(), dim, shape);
	}

	// explicit strides; the buffer spans shape[0] * stride[0] elements
	explicit Tensor(const int64 dim, const Shape& shape, const Stride& stride) : Tensor()
	{
		this->dim = dim;
		this->shape = shape;
		this->stride = stride;
		mem_buffer = std::make_shared<MemoryBuffer<device>>(static_cast<int64>(sizeof(dtype)) * shape[0] * stride[0]);
	}

	// dense tensor initialised from host values
	explicit Tensor(const std::vector<int64>& shape, const std::vector<dtype>& hdata) : Tensor(shape)
	{
		const int64 bytes = static_cast<int64>(sizeof(dtype) * hdata.size());
		ACASSERT(bytes <= mem_buffer->capacity, "more initial values than tensor elements");
		if constexpr (device == Device::CPU)
			std::memcpy(mem_buffer->buffer, hdata.data(), static_cast<size_t>(bytes));
		else
			device_memory::copy_to_device(mem_buffer->buffer, reinterpret_cast<const char*>(hdata.data()), bytes);
	}

private:
	std::shared_ptr<MemoryBuffer<device>> mem_buffer;

	// copies the WHOLE underlying buffer to `target_device`, keeping the view description
	template<Device target_device>
	Tensor<dtype, target_device> clone_to() const
	{
		const int64 bytes = mem_buffer->capacity;
		Tensor<dtype, target_device> t(bytes);
		t.dim = dim;
		t.shape = shape;
		t.stride = stride;
		t.alignment = alignment;
		t.offset = offset;
		t.name = name;
		char* dst = t.raw_buffer();
		const char* src = raw_buffer();
		if constexpr (device == CPU && target_device == CPU) std::memcpy(dst, src, static_cast<size_t>(bytes));
		else if constexpr (device == CPU && target_device == CUDA) device_memory::copy_to_device(dst, src, bytes);
		else if constexpr (device == CUDA && target_device == CPU) device_memory::copy_from_device(dst, src, bytes);
		else device_memory::copy_on_device(dst, src, bytes);
		return t;
	}
};

template<typename dtype, Device device>
Tensor<dtype, CPU> Tensor<dtype, device>::copy_to_host() const { return clone_to<CPU>(); }

template<typename dtype, Device device>
Tensor<dtype, CUDA> Tensor<dtype, device>::copy_to_cuda() const { return clone_to<CUDA>(); }

template<typename dtype, Device device, Device trg_device>
inline Tensor<dtype, trg_device> copy_to_device(const Tensor<dtype, device>& t)
{
	if constexpr (trg_device == CPU) return t.copy_to_host();
	else
	{
		static_assert(trg_device == CUDA, "unknown device");
		return t.copy_to_cuda();
	}
}

/*
  Element type conversion on the host.  Only float32 targets exist: this is the up-cast the
  half-precision tests use to obtain a float32 CPU reference from fp16 data.
*/
template<typename trg_dtype, typename src_dtype>
inline Tensor<trg_dtype, CPU> cvt_tensor_datatype(const Tensor<src_dtype, CPU>& tensor)
{
	static_assert(std::is_same_v<trg_dtype, float32>, "unknown target data type");
	Tensor<trg_dtype, CPU> converted(tensor.dim, tensor.shape, tensor.stride);
	const int64 n = tensor.size();
	const src_dtype* src = tensor.buffer();
	trg_dtype* dst = converted.buffer();
	for (int64 ix = 0; ix < n; ++ix) dst[ix] = cvt_any_to_float32(src[ix]);
	return converted;
}

/* The opposite direction (float32 -> any element type, round to nearest), for building half inputs. */
template<typename trg_dtype>
inline Tensor<trg_dtype, CPU> cvt_tensor_from_float32(const Tensor<float32, CPU>& tensor)
{
	Tensor<trg_dtype, CPU> converted(tensor.dim, tensor.shape, tensor.stride);
	const int64 n = tensor.size();
	const float32* src = tensor.buffer();
	trg_dtype* dst = converted.buffer();
	for (int64 ix = 0; ix < n; ++ix) dst[ix] = static_cast<trg_dtype>(src[ix]);
	return converted;
}

/*
  Multi-line description of a host tensor with the first `head` buffer elements.
*/
template<typename dtype>
inline std::string represent_tensor(const Tensor<dtype, CPU>& tensor, const int64 head = 5)
{
	std::stringstream ss;
	ss << "-- Tensor -- \n";
	ss << "  name:       " << tensor.name << "\n";
	ss << "  id:         " << tensor.id << "\n";
	ss << "  dtype:      " << get_datatype_enum<dtype>() << "\n";
	ss << "  dim:        " << tensor.dim << "\n";
	ss << "  alignment:  " << tensor.alignment << "\n";
	ss << "  offset:     " << tensor.offset << "\n";
	ss << "  shape:      " << represent_array(tensor.dim, tensor.shape) << "\n";
	ss << "  stride:     " << represent_array(tensor.dim, tensor.stride) << "\n";
	ss << "  capacity:   " << tensor.capacity() << "\n";
	ss << "  buffer content: \n      [";
	const int64 total = tensor.size();
	const int64 shown = std::min(head, total);
	const dtype* data = tensor.buffer();
	for (int64 ix = 0; ix < shown; ++ix) ss << (ix ? ", " : "") << cvt_any_to_float32(data[ix]);
	if (shown < total) ss << ", ...";
	ss << "] \n";
	return ss.str();
}

/* ---- factories ---- */

namespace tensor_factory {

template<typename dtype, Device device, typename Gen>
inline Tensor<dtype, device> from_int_generator(const std::vector<int64>& shape, Gen&& gen)
{
	std::vector<int> host_data(static_cast<size_t>(calc_default_size(shape)));
	for (auto& v : host_data) v = gen();
	return Tensor<dtype, device>(shape, cvt_int_vector_to_any<dtype>(host_data));
}

}  // namespace tensor_factory

/* Integers drawn uniformly from 0..10 (exact in every float type, so sums are order independent). */
template<typename dtype, Device device>
inline Tensor<dtype, device> crt_random_tensor(const std::vector<int64>& shape, const int64 seed = 10)
{
	std::default_random_engine eng(seed);
	std::uniform_int_distribution<int> uni_dist(0, 10);
	return tensor_factory::from_int_generator<dtype, device>(shape, [&] { return uni_dist(eng); });
}

/* Samples of N(0, 1), generated in float32 and rounded to dtype. */
template<typename dtype, Device device>
inline Tensor<dtype, device> crt_random_normal_tensor(const std::vector<int64>& shape, const int64 seed = 10)
{
	std::default_random_engine eng(seed);
	std::normal_distribution<float32> norm_dist(0.f, 1.f);
	std::vector<dtype> host_data(static_cast<size_t>(calc_default_size(shape)));
	for (auto& v : host_data) v = static_cast<dtype>(norm_dist(eng));
	return Tensor<dtype, device>(shape, host_data);
}

/* Samples of U(lo, hi), generated in float32 and rounded to dtype (benchmark inputs). */
template<typename dtype, Device device>
inline Tensor<dtype, device> crt_random_uniform_tensor(const std::vector<int64>& shape, const int64 seed = 10,
                                                       const float32 lo = -1.f, const float32 hi = 1.f)
{
	std::default_random_engine eng(seed);
	std::uniform_real_distribution<float32> dist(lo, hi);
	std::vector<dtype> host_data(static_cast<size_t>(calc_default_size(shape)));
	for (auto& v : host_data) v = static_cast<dtype>(dist(eng));
	return Tensor<dtype, device>(shape, host_data);
}

/* Element ix holds ix % 10: easy to reproduce in any other framework. */
template<typename dtype, Device device>
inline Tensor<dtype, device> crt_pattern_tensor(const std::vector<int64>& shape)
{
	int counter = 0;
	return tensor_factory::from_int_generator<dtype, device>(shape, [&] { return (counter++) % 10; });
}

template<typename dtype, Device device>
inline Tensor<dtype, device> crt_ones_tensor(const std::vector<int64>& shape)
{
	return tensor_factory::from_int_generator<dtype, device>(shape, [] { return 1; });
}

/* ---- compatibility checks ---- */

/* Same dim, shape and strides: element offsets coincide, elementwise loops may run over the buffers. */
template<typename dtype, Device device>
inline bool elementwise_compatible(const Tensor<dtype, device>& lhs, const Tensor<dtype, device>& rhs)
{
	return lhs.dim == rhs.dim && equal(lhs.dim, lhs.shape, rhs.shape) && equal(lhs.dim, lhs.stride, rhs.stride);
}

template<typename dtype, Device device>
inline bool matmul_compatible(const Tensor<dtype, device>& lhs, const Tensor<dtype, device>& rhs)
{
	return lhs.dim == 2 && rhs.dim == 2 && lhs.shape[1] == rhs.shape[0];
}

/* Launch geometry for one thread per element, 256 threads per block. */
template<typename dtype, Device device>
inline KernelParameters calc_kernel_prms_pointwise(const Tensor<dtype, device>& tensor)
{
	const unsigned int threads_per_block = 256;
	KernelParameters kpms = {};
	kpms.block_size = { threads_per_block, 1, 1 };
	kpms.grid_size = { calc_req_num_blocks(static_cast<unsigned int>(tensor.size()), threads_per_block), 1, 1 };
	return kpms;
}

#endif  // __TENSOR__
