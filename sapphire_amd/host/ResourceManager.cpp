#include <Sapphire/util/ResourceManager.hpp>

#include <Sapphire/compute/cudaUtil/Memory.hpp>
#include <Sapphire/util/BlockPool.hpp>

#include <cstdlib>
#include <mutex>
#include <stdexcept>

namespace Sapphire::Util
{
namespace
{
void* AllocateHost(std::size_t size)
{
    void* ptr = std::aligned_alloc(64, size);
    if (ptr == nullptr)
        throw std::runtime_error("ResourceManager::GetMemoryHost - allocation failed");
    return ptr;
}

void ReleaseHost(void* ptr)
{
    std::free(ptr);
}

// Device blocks come from the stream-ordered allocator: a request that misses the exact-size
// free list costs no device synchronisation, and a released block goes back to the device's
// pool in stream order instead of waiting for the device like cudaFree.
void* AllocateCuda(std::size_t size)
{
    void* ptr = nullptr;
    Compute::Cuda::CudaMallocAsync(&ptr, size);
    return ptr;
}

void ReleaseCuda(void* ptr)
{
    Compute::Cuda::CudaFreeAsync(ptr);
}

void* NoStream()
{
    return nullptr;
}

void NoWait(void*) {}

void* CurrentCudaStream()
{
    return Compute::Cuda::CurrentStream();
}

void WaitForCudaStream(void* stream)
{
    Compute::Cuda::StreamWaitStream(stream);
}

std::mutex gMutex;
BlockPool gHost({ AllocateHost, ReleaseHost, NoStream, NoWait });
BlockPool gCuda({ AllocateCuda, ReleaseCuda, CurrentCudaStream, WaitForCudaStream });
}  // namespace

void* ResourceManager::GetMemoryCuda(std::size_t byteSize, bool preserve)
{
    std::lock_guard<std::mutex> lock(gMutex);
    return gCuda.Get(byteSize, preserve);
}

void* ResourceManager::GetMemoryHost(std::size_t byteSize, bool preserve)
{
    std::lock_guard<std::mutex> lock(gMutex);
    return gHost.Get(byteSize, preserve);
}

void ResourceManager::FreePreservedHost(void* ptr)
{
    std::lock_guard<std::mutex> lock(gMutex);
    gHost.FreePreserved(ptr, "FreePreservedHost");
}

void ResourceManager::FreePreservedCuda(void* ptr)
{
    std::lock_guard<std::mutex> lock(gMutex);
    gCuda.FreePreserved(ptr, "FreePreservedCuda");
}

void ResourceManager::MoveToPreservedHost(void* ptr)
{
    std::lock_guard<std::mutex> lock(gMutex);
    gHost.ToPreserved(ptr, "MoveToPreservedHost");
}

void ResourceManager::MoveToPreservedCuda(void* ptr)
{
    std::lock_guard<std::mutex> lock(gMutex);
    gCuda.ToPreserved(ptr, "MoveToPreservedCuda");
}

void ResourceManager::MoveToVolatileHost(void* ptr)
{
    std::lock_guard<std::mutex> lock(gMutex);
    gHost.ToVolatile(ptr, "MoveToVolatileHost");
}

void ResourceManager::MoveToVolatileCuda(void* ptr)
{
    std::lock_guard<std::mutex> lock(gMutex);
    gCuda.ToVolatile(ptr, "MoveToVolatileCuda");
}

void ResourceManager::MarkZeroPendingCuda(void* ptr)
{
    std::lock_guard<std::mutex> lock(gMutex);
    gCuda.MarkZeroPending(ptr);
}

bool ResourceManager::TakeZeroPendingCuda(void* ptr)
{
    std::lock_guard<std::mutex> lock(gMutex);
    return gCuda.TakeZeroPending(ptr);
}

void ResourceManager::Clean()
{
    std::lock_guard<std::mutex> lock(gMutex);
    gHost.Clean();
    gCuda.Clean();
}

void ResourceManager::ClearPreservedPool()
{
    std::lock_guard<std::mutex> lock(gMutex);
    gHost.ClearPreserved();
    gCuda.ClearPreserved();
}

void ResourceManager::ClearVolatilePool()
{
    std::lock_guard<std::mutex> lock(gMutex);
    gHost.ClearVolatile();
    gCuda.ClearVolatile();
}

void ResourceManager::ClearFreePool()
{
    std::lock_guard<std::mutex> lock(gMutex);
    gHost.ClearFree();
    gCuda.ClearFree();
}

void ResourceManager::ClearAll()
{
    // device work that may still use the blocks, on any thread's stream, has to finish first
    bool deviceBlocks = false;
    {
        std::lock_guard<std::mutex> lock(gMutex);
        deviceBlocks = gCuda.CountVolatile() + gCuda.CountPreserved() + gCuda.CountFree() > 0;
    }
    if (deviceBlocks)
        Compute::Cuda::SynchronizeDevice();
    ClearPreservedPool();
    ClearVolatilePool();
    ClearFreePool();
    if (deviceBlocks)
    {
        Compute::Cuda::Synchronize();  // the stream-ordered releases have to run first
        Compute::Cuda::CudaTrimPool();
    }
}

PoolStatistics ResourceManager::Statistics()
{
    std::lock_guard<std::mutex> lock(gMutex);
    return { gHost.CountVolatile(), gHost.CountPreserved(), gHost.CountFree(),
             gCuda.CountVolatile(), gCuda.CountPreserved(), gCuda.CountFree() };
}
}  // namespace Sapphire::Util
