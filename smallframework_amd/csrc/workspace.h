// Bookkeeping of the library-owned device scratch blocks (host-only C++, no HIP types, so that it can be unit
// tested on a machine without a GPU with a fake allocator).
//
// One current block per (device, stream): work that uses a block is ordered by the stream it belongs to, so two
// streams never share a block and cannot overwrite each other's contents.  A pointer that was handed out stays valid
// until release_device(): a request larger than the current block allocates a NEW block and retires the old one,
// which stays allocated (a kernel already queued, or a captured graph that is replayed later, may still refer to it).
// Nothing is freed behind the caller's back: a full table refuses the request instead of evicting a block.
// Memory is given back only by release_device(), which the caller invokes when no queued or captured work of that
// device uses library scratch any more.  Every caller holds the pool's lock from acquire() until its last launch that
// uses the pointer has been enqueued, so release_device() on another thread cannot free a block in between.
#pragma once

#include <cstddef>
#include <cstdint>
#include <mutex>
#include <vector>

namespace shp
{

// Mem::alloc(void **p, size_t bytes) -> 0 on success, else an error code handed back to the caller;
// Mem::release(void *p) -> 0 or an error code; it must not return before every kernel queued on the block's device
// has finished.
template <class Mem>
class WorkspacePool
{
public:
    static constexpr size_t GRANULE = size_t(1) << 20;      // blocks are rounded up to 1 MiB
    static constexpr size_t MAX_BLOCKS = 64;                // (device, stream) pairs kept at once

    explicit WorkspacePool(size_t granule = GRANULE) : m_granule(granule) {}

    // Hold the returned lock until the work that uses the acquired pointer has been enqueued.
    std::unique_lock<std::mutex> lock() { return std::unique_lock<std::mutex>(m_mu); }

    // The block of (device, stream), at least `bytes` long.  The caller holds lock().
    int acquire(int device, const void *stream, size_t bytes, void **ptr)
    {
        *ptr = nullptr;
        Entry *e = find(device, stream);
        if (!e)
        {
            if (m_entries.size() >= MAX_BLOCKS) return m_full_code;
            m_entries.push_back(Entry{device, stream, nullptr, 0});
            e = &m_entries.back();
        }
        if (bytes > e->cap)
        {
            const size_t cap = (bytes + m_granule - 1) / m_granule * m_granule;
            void *p = nullptr;
            if (int rc = Mem::alloc(&p, cap)) return rc;    // the entry keeps its old block
            if (e->ptr) m_retired.push_back(Retired{device, e->ptr, e->cap});
            e->ptr = p;
            e->cap = cap;
        }
        *ptr = e->ptr;
        return 0;
    }

    // Frees every block of `device`, current and retired (e.g. before the caller destroys its streams, or after the
    // largest shapes have run and their graphs are gone).  The caller holds lock().  The first error is returned, all
    // blocks are dropped from the table either way.
    int release_device(int device)
    {
        int rc = 0;
        for (size_t i = 0; i < m_entries.size();)
        {
            if (m_entries[i].device != device) { ++i; continue; }
            if (m_entries[i].ptr)
                if (int r = Mem::release(m_entries[i].ptr)) rc = rc ? rc : r;
            m_entries.erase(m_entries.begin() + (long)i);
        }
        for (size_t i = 0; i < m_retired.size();)
        {
            if (m_retired[i].device != device) { ++i; continue; }
            if (int r = Mem::release(m_retired[i].ptr)) rc = rc ? rc : r;
            m_retired.erase(m_retired.begin() + (long)i);
        }
        return rc;
    }

    void set_full_code(int code) { m_full_code = code; }
    size_t blocks() const { return m_entries.size(); }
    size_t retired() const { return m_retired.size(); }
    size_t capacity(int device, const void *stream) const
    {
        for (auto const &e : m_entries)
            if (e.device == device && e.stream == stream) return e.cap;
        return 0;
    }
    // bytes held for `device`, retired blocks included
    size_t held(int device) const
    {
        size_t n = 0;
        for (auto const &e : m_entries)
            if (e.device == device) n += e.cap;
        for (auto const &r : m_retired)
            if (r.device == device) n += r.cap;
        return n;
    }

private:
    struct Entry
    {
        int device;
        const void *stream;
        void *ptr;
        size_t cap;
    };
    struct Retired
    {
        int device;
        void *ptr;
        size_t cap;
    };

    Entry *find(int device, const void *stream)
    {
        for (auto &e : m_entries)
            if (e.device == device && e.stream == stream) return &e;
        return nullptr;
    }

    std::mutex m_mu;
    std::vector<Entry> m_entries;
    std::vector<Retired> m_retired;
    size_t m_granule;
    int m_full_code = -1;
};

} // namespace shp
