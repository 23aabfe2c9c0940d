#include "device_memory.hpp"
#include "core.hpp"

#include <hip/hip_runtime_api.h>

namespace device_memory {

char* allocate_zeroed(long long bytes)
{
	if (bytes <= 0) return nullptr;
	void* ptr = nullptr;
	HIP_CHECK(hipMalloc(&ptr, static_cast<size_t>(bytes)));
	HIP_CHECK(hipMemset(ptr, 0, static_cast<size_t>(bytes)));
	return static_cast<char*>(ptr);
}

void release(char* ptr)
{
	if (ptr != nullptr) HIP_CHECK(hipFree(ptr));
}

void copy_to_device(char* dst_device, const char* src_host, long long bytes)
{
	if (bytes > 0) HIP_CHECK(hipMemcpy(dst_device, src_host, static_cast<size_t>(bytes), hipMemcpyHostToDevice));
}

void copy_from_device(char* dst_host, const char* src_device, long long bytes)
{
	if (bytes > 0) HIP_CHECK(hipMemcpy(dst_host, src_device, static_cast<size_t>(bytes), hipMemcpyDeviceToHost));
}

void copy_on_device(char* dst_device, const char* src_device, long long bytes)
{
	if (bytes > 0) HIP_CHECK(hipMemcpy(dst_device, src_device, static_cast<size_t>(bytes), hipMemcpyDeviceToDevice));
}

void synchronize()
{
	HIP_CHECK(hipDeviceSynchronize());
}

}  // namespace device_memory

int last_device_error()
{
	return static_cast<int>(hipGetLastError());
}

std::string print_cuda_device_props()
{
	std::stringstream ss;
	int num_devices = 0;
	HIP_CHECK(hipGetDeviceCount(&num_devices));
	hipDeviceProp_t p;
	HIP_CHECK(hipGetDeviceProperties(&p, 0));

	ss << "--- GPU device info (HIP) --- \n";
	ss << "  Device selection \n";
	ss << "    Num devices:                 " << num_devices << "\n";
	ss << "    Device id:                   " << 0 << "\n";
	ss << "    Device name:                 " << p.name << "\n";
	ss << "    Architecture:                " << p.gcnArchName << "\n";
	ss << "    integrated:                  " << p.integrated << "\n\n";
	ss << "  Memory info \n";
	ss << "    LDS per compute unit:        " << p.maxSharedMemoryPerMultiProcessor << "\n";
	ss << "    LDS per workgroup:           " << p.sharedMemPerBlock << "\n";
	ss << "    memoryBusWidth:              " << p.memoryBusWidth << "\n";
	ss << "    memoryClockRate (kHz):       " << p.memoryClockRate << "\n";
	ss << "    totalGlobalMem:              " << p.totalGlobalMem << "\n";
	ss << "    l2CacheSize:                 " << p.l2CacheSize << "\n\n";
	ss << "  Kernel launch info \n";
	ss << "    maxGridSize.x:               " << p.maxGridSize[0] << "\n";
	ss << "    maxGridSize.y:               " << p.maxGridSize[1] << "\n";
	ss << "    maxGridSize.z:               " << p.maxGridSize[2] << "\n";
	ss << "    compute units:               " << p.multiProcessorCount << "\n";
	ss << "    clockRate (kHz):             " << p.clockRate << "\n";
	ss << "    wavefront size:              " << p.warpSize << "\n";
	ss << "    maxThreadsPerMultiProcessor: " << p.maxThreadsPerMultiProcessor << "\n";
	ss << "    maxThreadsPerBlock:          " << p.maxThreadsPerBlock << "\n";
	ss << "    regsPerBlock:                " << p.regsPerBlock << "\n";
	ss << "    concurrentKernels:           " << p.concurrentKernels << "\n";
	return ss.str();
}
