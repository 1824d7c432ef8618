// Bookkeeping of one memory space behind ResourceManager: live blocks by address (volatile and
// preserved), idle blocks by size.
//
// Same life cycle as the pools of the reference's Sapphire::Util::ResourceManager
// (Sources/Sapphire/util/ResourceManager.cpp:38-323): requests rounded up to 256 bytes, a
// volatile request reuses an idle block of exactly that size, Clean() makes every volatile
// block idle, the Clear*() calls release memory.
//
// Device blocks are stream-affine.  The reference releases with cudaFree, which waits for the
// device, so a block could never be handed on while work still used it.  Here every host
// thread enqueues on its own stream and blocks are released in stream order, so each block
// remembers the stream of the thread it was handed to, and whenever another stream takes it
// over -- reuse from the idle list, or release -- that stream is first made to wait for the work
// enqueued so far on the remembered one.  A block that several threads use at the same time
// is outside this rule (as it was outside the reference's unsynchronised pools): its users
// synchronise among themselves.
#ifndef SAPPHIRE_AMD_UTIL_BLOCKPOOL_HPP
#define SAPPHIRE_AMD_UTIL_BLOCKPOOL_HPP

#include <cstddef>
#include <map>
#include <stdexcept>
#include <string>
#include <unordered_map>

namespace Sapphire::Util
{
struct BlockPoolHooks
{
    void* (*allocate)(std::size_t);
    void (*release)(void*);
    //! Stream the calling thread enqueues on (nullptr for memory that has none).
    void* (*currentStream)();
    //! Work the calling thread enqueues from now on waits for what `stream` holds so far.
    void (*waitFor)(void* stream);
};

class BlockPool
{
public:
    static constexpr std::size_t kGranule = 256;

    explicit BlockPool(BlockPoolHooks hooks) : m_hooks(hooks) {}

    void* Get(std::size_t byteSize, bool preserve)
    {
        const std::size_t size = (byteSize + kGranule - 1) / kGranule * kGranule;
        void* const stream = m_hooks.currentStream();
        if (preserve)
        {
            void* ptr = m_hooks.allocate(size);
            m_preserved.emplace(ptr, Block{ size, stream, false });
            return ptr;
        }
        void* ptr = nullptr;
        const auto idle = m_free.find(size);
        if (idle != m_free.end())
        {
            ptr = idle->second.first;
            TakeOver(idle->second.second, stream);
            m_free.erase(idle);
        }
        else
            ptr = m_hooks.allocate(size);
        m_volatile.emplace(ptr, Block{ size, stream, false });
        return ptr;
    }

    void FreePreserved(void* ptr, const char* who)
    {
        const auto it = Find(m_preserved, ptr, who, "Given ptr to free was not found");
        Release(ptr, it->second.stream);
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
        for (const auto& [ptr, block] : m_volatile)
            m_free.emplace(block.size, std::make_pair(ptr, block.stream));
        m_volatile.clear();
    }

    void ClearPreserved() { ReleaseAll(m_preserved); }
    void ClearVolatile() { ReleaseAll(m_volatile); }
    void ClearFree()
    {
        for (const auto& [size, idle] : m_free)
            Release(idle.first, idle.second);
        m_free.clear();
    }

    //! Deferred zero fill.  A block handed out by Get() may be marked "holds zeros that have not
    //! been written yet"; whoever uses the block first takes the mark and either fills the
    //! block or, when it is about to write every byte anyway, does nothing.  The mark dies
    //! with the block's live entry (Clean, release), so a reused block starts unmarked.
    void MarkZeroPending(void* ptr)
    {
        if (Block* b = FindLive(ptr))
            b->zeroPending = true;
    }
    //! True when the mark was set; clears it.
    bool TakeZeroPending(void* ptr)
    {
        Block* b = FindLive(ptr);
        if (b == nullptr || !b->zeroPending)
            return false;
        b->zeroPending = false;
        return true;
    }

    std::size_t CountVolatile() const { return m_volatile.size(); }
    std::size_t CountPreserved() const { return m_preserved.size(); }
    std::size_t CountFree() const { return m_free.size(); }

private:
    struct Block
    {
        std::size_t size;
        void* stream;
        bool zeroPending = false;
    };
    using Live = std::unordered_map<void*, Block>;

    Block* FindLive(void* ptr)
    {
        auto it = m_volatile.find(ptr);
        if (it != m_volatile.end())
            return &it->second;
        it = m_preserved.find(ptr);
        return it != m_preserved.end() ? &it->second : nullptr;
    }

    static Live::iterator Find(Live& pool, void* ptr, const char* who, const char* what)
    {
        const auto it = pool.find(ptr);
        if (it == pool.end())
            throw std::runtime_error(std::string("ResourceManager::") + who + " - " + what);
        return it;
    }

    // the calling thread's stream is about to reuse or release a block that `owner` used
    void TakeOver(void* owner, void* current)
    {
        if (owner != nullptr && owner != current)
            m_hooks.waitFor(owner);
    }

    void Release(void* ptr, void* owner)
    {
        TakeOver(owner, m_hooks.currentStream());
        m_hooks.release(ptr);
    }

    void ReleaseAll(Live& pool)
    {
        for (const auto& [ptr, block] : pool)
            Release(ptr, block.stream);
        pool.clear();
    }

    BlockPoolHooks m_hooks;
    Live m_volatile;
    Live m_preserved;
    std::multimap<std::size_t, std::pair<void*, void*>> m_free;  // size -> (block, stream)
};
}  // namespace Sapphire::Util

#endif
