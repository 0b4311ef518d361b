// Bookkeeping of the library-owned device scratch blocks (host-only C++, no HIP types, so that it can be unit
// tested on a machine without a GPU with a fake allocator).
//
// One block per (device, stream): work that uses a block is ordered by the stream it belongs to, so two streams
// never share a block and cannot overwrite each other's contents.  A block only grows; growing frees the old block
// with an allocator call that waits for the device (hipFree does), and every caller holds the pool's lock from
// acquire() until its last launch that uses the pointer has been enqueued, so no queued or about-to-be-queued
// kernel can refer to a freed block.
#pragma once

#include <cstddef>
#include <cstdint>
#include <mutex>
#include <vector>

namespace shp
{

// Mem::alloc(void **p, size_t bytes) -> 0 on success, else an error code handed back to the caller;
// Mem::release(void *p) must not return before every kernel queued on the block's device has finished.
template <class Mem>
class WorkspacePool
{
public:
    static constexpr size_t GRANULE = size_t(1) << 20;      // blocks are rounded up to 1 MiB
    static constexpr size_t MAX_BLOCKS = 64;                // (device, stream) pairs kept at once

    // Hold the returned lock until the work that uses the acquired pointer has been enqueued.
    std::unique_lock<std::mutex> lock() { return std::unique_lock<std::mutex>(m_mu); }

    // The block of (device, stream), at least `bytes` long.  The caller holds lock().
    int acquire(int device, const void *stream, size_t bytes, void **ptr)
    {
        *ptr = nullptr;
        Entry *e = find(device, stream);
        if (!e)
        {
            if (m_entries.size() >= MAX_BLOCKS && !evict(device)) return m_full_code;
            m_entries.push_back(Entry{device, stream, nullptr, 0, 0});
            e = &m_entries.back();
        }
        e->tick = ++m_clock;
        if (bytes > e->cap)
        {
            if (e->ptr)
            {
                void *old = e->ptr;
                e->ptr = nullptr;
                e->cap = 0;
                if (int rc = Mem::release(old)) return rc;
            }
            const size_t cap = (bytes + GRANULE - 1) / GRANULE * GRANULE;
            void *p = nullptr;
            if (int rc = Mem::alloc(&p, cap)) return rc;
            e->ptr = p;
            e->cap = cap;
        }
        *ptr = e->ptr;
        return 0;
    }

    // Frees every block of `device` (e.g. before the caller destroys its streams).  The caller holds lock().
    int release_device(int device)
    {
        int rc = 0;
        for (size_t i = 0; i < m_entries.size();)
        {
            if (m_entries[i].device != device) { ++i; continue; }
            if (m_entries[i].ptr)
                if (int r = Mem::release(m_entries[i].ptr)) rc = r;
            m_entries.erase(m_entries.begin() + (long)i);
        }
        return rc;
    }

    void set_full_code(int code) { m_full_code = code; }
    size_t blocks() const { return m_entries.size(); }
    size_t capacity(int device, const void *stream) const
    {
        for (auto const &e : m_entries)
            if (e.device == device && e.stream == stream) return e.cap;
        return 0;
    }

private:
    struct Entry
    {
        int device;
        const void *stream;
        void *ptr;
        size_t cap;
        uint64_t tick;
    };

    Entry *find(int device, const void *stream)
    {
        for (auto &e : m_entries)
            if (e.device == device && e.stream == stream) return &e;
        return nullptr;
    }

    // drops the least recently used block of `device` (only that device is current, and only its release waits for it)
    bool evict(int device)
    {
        long victim = -1;
        for (size_t i = 0; i < m_entries.size(); ++i)
            if (m_entries[i].device == device && (victim < 0 || m_entries[i].tick < m_entries[(size_t)victim].tick))
                victim = (long)i;
        if (victim < 0) return false;
        if (m_entries[(size_t)victim].ptr) Mem::release(m_entries[(size_t)victim].ptr);
        m_entries.erase(m_entries.begin() + victim);
        return true;
    }

    std::mutex m_mu;
    std::vector<Entry> m_entries;
    uint64_t m_clock = 0;
    int m_full_code = -1;
};

} // namespace shp
