#include <Sapphire/compute/cudaUtil/Memory.hpp>

#include <sapphire_hip.h>

#include <stdexcept>
#include <string>

namespace Sapphire::Compute::Cuda
{
namespace
{
void Check(int status, const char* function)
{
    if (status != SPH_OK)
        throw std::runtime_error(std::string(function) + " failed with " + sph_last_error());
}
}  // namespace

void CudaSetDevice(int deviceId)
{
    const int status = sph_set_device(deviceId);
    if (status == SPH_ERR_INVALID)
        throw std::runtime_error("CudaSetDevice - deviceId exceeds number of available devices");
    Check(status, "CudaSetDevice");
}

void CudaMalloc(void** ptr, std::size_t byteSize)
{
    Check(sph_malloc(ptr, byteSize), "CudaMalloc");
}

void CudaFree(void* ptr)
{
    Check(sph_free(ptr), "CudaFree");
}

void CudaMallocAsync(void** ptr, std::size_t byteSize)
{
    Check(sph_malloc_async(ptr, byteSize), "CudaMallocAsync");
}

void CudaFreeAsync(void* ptr)
{
    Check(sph_free_async(ptr), "CudaFreeAsync");
}

void CudaTrimPool()
{
    Check(sph_mem_pool_trim(), "CudaTrimPool");
}

void CopyHostToDevice(void* devicePtr, const void* hostPtr, std::size_t byteSize)
{
    Check(sph_memcpy_h2d(devicePtr, hostPtr, byteSize), "CopyHostToDevice");
}

void CopyDeviceToHost(void* hostPtr, const void* devicePtr, std::size_t byteSize)
{
    Check(sph_memcpy_d2h(hostPtr, devicePtr, byteSize), "CopyDeviceToHost");
}

void CopyDeviceToDevice(void* dst, const void* src, std::size_t byteSize)
{
    Check(sph_memcpy_d2d(dst, src, byteSize), "CopyDeviceToDevice");
}

void CopyDeviceToDeviceAsync(void* dst, const void* src, std::size_t byteSize, StreamHandle stream)
{
    if (stream == nullptr)
    {
        Check(sph_memcpy_d2d_async(dst, src, byteSize), "CopyDeviceToDeviceAsync");
        return;
    }
    void* previous = nullptr;
    Check(sph_get_stream(&previous), "CopyDeviceToDeviceAsync");
    Check(sph_set_stream(stream), "CopyDeviceToDeviceAsync");
    const int status = sph_memcpy_d2d_async(dst, src, byteSize);
    sph_set_stream(nullptr);
    Check(status, "CopyDeviceToDeviceAsync");
}

void CopyDeviceToDeviceBroadcast(void* dst, const void* src, std::size_t byteSize,
                                 std::size_t srcStrideByteSize)
{
    if (srcStrideByteSize == 0)
        throw std::runtime_error("CopyDeviceToDeviceBroadcast failed with zero stride");
    for (std::size_t done = 0; done < byteSize; done += srcStrideByteSize)
    {
        const int status =
            sph_memcpy_d2d_async(static_cast<char*>(dst) + done, src, srcStrideByteSize);
        if (status != SPH_OK)
            throw std::runtime_error("CopyDeviceToDeviceBroadcast failed in idx" +
                                     std::to_string(done) + " with " + sph_last_error());
    }
    Check(sph_stream_sync(), "CopyDeviceToDeviceBroadcast");
}

void Synchronize()
{
    Check(sph_stream_sync(), "Synchronize");
}

void SynchronizeDevice()
{
    Check(sph_device_sync(), "SynchronizeDevice");
}

StreamHandle CurrentStream()
{
    void* stream = nullptr;
    Check(sph_get_stream(&stream), "CurrentStream");
    return stream;
}

void StreamWaitStream(StreamHandle stream)
{
    Check(sph_stream_wait_stream(stream), "StreamWaitStream");
}
}  // namespace Sapphire::Compute::Cuda
