// The only door from the host layer to GPU memory.  Implemented in device_memory.cpp on top of
// the HIP runtime (hipMalloc / hipMemset / hipMemcpy / hipFree on the current device); any
// runtime failure is fail-stop (message, exit(1)), like every other error in this layer.
#pragma once

#include <cstdint>

namespace device_memory {

// New zero-filled allocation of `bytes` bytes (bytes == 0 yields nullptr).
char* allocate_zeroed(long long bytes);
void release(char* ptr);

// Blocking copies; the *_from_device forms make all earlier kernel results visible to the host.
void copy_to_device(char* dst_device, const char* src_host, long long bytes);
void copy_from_device(char* dst_host, const char* src_device, long long bytes);
void copy_on_device(char* dst_device, const char* src_device, long long bytes);

// Waits for everything queued on the device.
void synchronize();

}  // namespace device_memory
