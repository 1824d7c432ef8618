// Pooled host and device memory for TensorData.
//
// Same interface and life cycle as the memory half of the reference's
// Sapphire::Util::ResourceManager (Includes/Sapphire/util/ResourceManager.hpp:43-161,
// Sources/Sapphire/util/ResourceManager.cpp:38-323): requests are rounded up to 256 bytes;
// a volatile request reuses a block of exactly that size from the free pool when there is
// one; Clean() moves every volatile block to the free pool; the Clear*() calls release
// memory.  The cuBLAS / cuDNN handle maps of the reference have no counterpart: the stream
// that replaces the per-(device, thread) handle lives behind the C ABI.
// Unlike the reference's, these pools are guarded by a mutex.
#ifndef SAPPHIRE_AMD_UTIL_RESOURCEMANAGER_HPP
#define SAPPHIRE_AMD_UTIL_RESOURCEMANAGER_HPP

#include <cstddef>

namespace Sapphire::Util
{
struct PoolStatistics
{
    std::size_t hostVolatile, hostPreserved, hostFree;
    std::size_t cudaVolatile, cudaPreserved, cudaFree;
};

class ResourceManager
{
public:
    static void* GetMemoryCuda(std::size_t byteSize, bool preserve = false);
    static void* GetMemoryHost(std::size_t byteSize, bool preserve = false);

    //! Throw std::runtime_error when `ptr` is not in the named pool.
    static void FreePreservedHost(void* ptr);
    static void FreePreservedCuda(void* ptr);
    static void MoveToPreservedHost(void* ptr);
    static void MoveToPreservedCuda(void* ptr);
    static void MoveToVolatileHost(void* ptr);
    static void MoveToVolatileCuda(void* ptr);

    //! Deferred zero fill of a device block obtained from GetMemoryCuda: Mark says "this block
    //! is to be read as zeros, the fill has not been enqueued"; Take returns whether the mark
    //! was set and clears it (the caller then fills the block, or overwrites all of it).  The
    //! reference fills every fresh device buffer at once
    //! (Sources/Sapphire/tensor/TensorData.cpp:354); deferring it lets an operator whose first
    //! act is to write the whole buffer skip both the fill and the read of the zeros.
    static void MarkZeroPendingCuda(void* ptr);
    static bool TakeZeroPendingCuda(void* ptr);

    //! Volatile blocks become reusable; nothing is released.
    static void Clean();
    static void ClearPreservedPool();
    static void ClearVolatilePool();
    static void ClearFreePool();
    static void ClearAll();

    //! Number of blocks per pool (for tests and leak checks).
    static PoolStatistics Statistics();
};
}  // namespace Sapphire::Util

#endif
