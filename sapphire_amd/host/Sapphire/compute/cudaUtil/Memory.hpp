// Throwing wrappers over the device-memory entry points of the C ABI.
//
// Same names and argument order as the reference's Sapphire::Compute::Cuda helpers
// (Includes/Sapphire/compute/cudaUtil/Memory.hpp:14-30); a failure becomes
// std::runtime_error("<Function> failed with <text>") as in
// Sources/Sapphire/compute/cudaUtil/Memory.cpp:14-98.  Byte counts are size_t: the
// reference's unsigned-int sizes convert implicitly, its 4 GiB cap is not inherited.
#ifndef SAPPHIRE_AMD_COMPUTE_CUDAUTIL_MEMORY_HPP
#define SAPPHIRE_AMD_COMPUTE_CUDAUTIL_MEMORY_HPP

#include <cstddef>

namespace Sapphire::Compute::Cuda
{
//! Opaque stream handle (a hipStream_t) for the one asynchronous entry point.
using StreamHandle = void*;

void CudaSetDevice(int deviceId);
void CudaMalloc(void** ptr, std::size_t byteSize);
void CudaFree(void* ptr);
//! Stream-ordered counterparts on the calling thread's stream: neither waits for the device,
//! freed blocks stay in the device's pool.
void CudaMallocAsync(void** ptr, std::size_t byteSize);
void CudaFreeAsync(void* ptr);
//! Returns idle pool memory to the driver.
void CudaTrimPool();
void CopyHostToDevice(void* devicePtr, const void* hostPtr, std::size_t byteSize);
void CopyDeviceToHost(void* hostPtr, const void* devicePtr, std::size_t byteSize);
void CopyDeviceToDevice(void* dst, const void* src, std::size_t byteSize);
//! Enqueues on `stream` (or on the calling thread's stream when null) and returns.
void CopyDeviceToDeviceAsync(void* dst, const void* src, std::size_t byteSize,
                             StreamHandle stream);
//! Fills dst with byteSize / srcStrideByteSize copies of the srcStrideByteSize bytes at src.
void CopyDeviceToDeviceBroadcast(void* dst, const void* src, std::size_t byteSize,
                                 std::size_t srcStrideByteSize);
//! Waits for everything the calling thread has enqueued on the current device.
void Synchronize();
//! Waits for everything any thread has enqueued on the current device.
void SynchronizeDevice();
//! The stream the calling thread's work on the current device is enqueued on.
StreamHandle CurrentStream();
//! Work the calling thread enqueues from now on waits for everything `stream` holds so far
//! (nothing happens when it is the calling thread's own stream).
void StreamWaitStream(StreamHandle stream);
}  // namespace Sapphire::Compute::Cuda

#endif
