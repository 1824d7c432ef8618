#include <Sapphire/util/ResourceManager.hpp>

#include <Sapphire/compute/cudaUtil/Memory.hpp>

#include <cstdlib>
#include <map>
#include <mutex>
#include <stdexcept>
#include <string>
#include <unordered_map>

namespace Sapphire::Util
{
namespace
{
constexpr std::size_t kGranule = 256;

std::size_t RoundUp(std::size_t bytes)
{
    return (bytes + kGranule - 1) / kGranule * kGranule;
}

// One memory space (host or device): live blocks by address, idle blocks by size.
class Space
{
public:
    using Allocate = void* (*)(std::size_t);
    using Release = void (*)(void*);

    Space(Allocate allocate, Release release) : m_allocate(allocate), m_release(release) {}

    void* Get(std::size_t byteSize, bool preserve)
    {
        const std::size_t size = RoundUp(byteSize);
        if (preserve)
        {
            void* ptr = m_allocate(size);
            m_preserved.emplace(ptr, size);
            return ptr;
        }
        void* ptr = nullptr;
        const auto idle = m_free.find(size);
        if (idle != m_free.end())
        {
            ptr = idle->second;
            m_free.erase(idle);
        }
        else
            ptr = m_allocate(size);
        m_volatile.emplace(ptr, size);
        return ptr;
    }

    void FreePreserved(void* ptr, const char* who)
    {
        const auto it = Find(m_preserved, ptr, who, "Given ptr to free was not found");
        m_release(ptr);
        m_preserved.erase(it);
    }

    void ToPreserved(void* ptr, const char* who)
    {
        const auto it = Find(m_volatile, ptr, who, "Cannot find given ptr");
        m_preserved.insert(*it);
        m_volatile.erase(it);
    }

    void ToVolatile(void* ptr, const char* who)
    {
        const auto it = Find(m_preserved, ptr, who, "Cannot find given ptr");
        m_volatile.insert(*it);
        m_preserved.erase(it);
    }

    void Clean()
    {
        for (const auto& [ptr, size] : m_volatile)
            m_free.emplace(size, ptr);
        m_volatile.clear();
    }

    void ClearPreserved() { ReleaseAll(m_preserved); }
    void ClearVolatile() { ReleaseAll(m_volatile); }
    void ClearFree()
    {
        for (const auto& [size, ptr] : m_free)
            m_release(ptr);
        m_free.clear();
    }

    std::size_t CountVolatile() const { return m_volatile.size(); }
    std::size_t CountPreserved() const { return m_preserved.size(); }
    std::size_t CountFree() const { return m_free.size(); }

private:
    using Live = std::unordered_map<void*, std::size_t>;

    static Live::iterator Find(Live& pool, void* ptr, const char* who, const char* what)
    {
        const auto it = pool.find(ptr);
        if (it == pool.end())
            throw std::runtime_error(std::string("ResourceManager::") + who + " - " + what);
        return it;
    }

    void ReleaseAll(Live& pool)
    {
        for (const auto& [ptr, size] : pool)
            m_release(ptr);
        pool.clear();
    }

    Allocate m_allocate;
    Release m_release;
    Live m_volatile;
    Live m_preserved;
    std::multimap<std::size_t, void*> m_free;
};

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

std::mutex gMutex;
Space gHost(AllocateHost, ReleaseHost);
Space gCuda(AllocateCuda, ReleaseCuda);
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
    // device work that may still use the blocks has to finish first
    bool deviceBlocks = false;
    {
        std::lock_guard<std::mutex> lock(gMutex);
        deviceBlocks = gCuda.CountVolatile() + gCuda.CountPreserved() + gCuda.CountFree() > 0;
    }
    if (deviceBlocks)
        Compute::Cuda::Synchronize();
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
