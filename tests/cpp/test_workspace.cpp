// CPU unit test of the scratch-block bookkeeping (smallframework_amd/csrc/workspace.h) with a fake allocator:
// one current block per (device, stream); growth adds a block and keeps the old one allocated (a pointer handed out
// stays valid until release_device); a full table refuses instead of evicting; nothing is released twice; the lock
// serialises acquire-to-enqueue.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <set>
#include <thread>
#include <vector>

#include "../../smallframework_amd/csrc/workspace.h"

static int g_failures = 0;
#define CHECK(c)                                                                  \
    do                                                                            \
    {                                                                             \
        if (!(c))                                                                 \
        {                                                                         \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #c);            \
            ++g_failures;                                                         \
        }                                                                         \
    } while (0)

struct FakeMem
{
    static std::map<void *, size_t> live;
    static std::set<void *> released;
    static int fail_next_alloc, fail_next_release;
    static long allocs, releases;
    static int alloc(void **p, size_t bytes)
    {
        if (fail_next_alloc) { int rc = fail_next_alloc; fail_next_alloc = 0; return rc; }
        *p = std::malloc(16);                   // a unique address; the size is only recorded
        live[*p] = bytes;
        ++allocs;
        return 0;
    }
    static int release(void *p)
    {
        if (fail_next_release) { int rc = fail_next_release; fail_next_release = 0; return rc; }
        if (!live.count(p)) { std::printf("release of a block that is not live\n"); ++g_failures; return 0; }
        live.erase(p);
        released.insert(p);                     // kept allocated so that addresses are never re-used in the test
        ++releases;
        return 0;
    }
};
std::map<void *, size_t> FakeMem::live;
std::set<void *> FakeMem::released;
int FakeMem::fail_next_alloc = 0, FakeMem::fail_next_release = 0;
long FakeMem::allocs = 0, FakeMem::releases = 0;

using Pool = shp::WorkspacePool<FakeMem>;

static void test_per_stream_blocks()
{
    Pool pool;
    int s1, s2;           // two distinct stream handles
    void *a = nullptr, *b = nullptr, *c = nullptr;
    auto lk = pool.lock();
    CHECK(pool.acquire(0, &s1, 1000, &a) == 0 && a);
    CHECK(pool.acquire(0, &s2, 1000, &b) == 0 && b && b != a);      // another stream never shares a block
    CHECK(pool.acquire(1, &s1, 1000, &c) == 0 && c && c != a && c != b);   // nor another device
    CHECK(pool.blocks() == 3);
    CHECK(FakeMem::live[a] == Pool::GRANULE);                       // rounded up
    void *a2 = nullptr;
    CHECK(pool.acquire(0, &s1, 500, &a2) == 0 && a2 == a);          // smaller request: same block
    CHECK(pool.acquire(0, &s1, Pool::GRANULE, &a2) == 0 && a2 == a);
    CHECK(pool.release_device(0) == 0 && pool.blocks() == 1 && FakeMem::live.count(c) && !FakeMem::live.count(b));
    CHECK(pool.release_device(1) == 0 && FakeMem::live.empty());
}

static void test_a_pointer_handed_out_stays_valid_after_growth()
{
    // a kernel already queued, or a captured graph replayed later, may still use the smaller block: growth adds a
    // block and retires the old one, which stays allocated until release_device()
    Pool pool;
    int s1, s2;
    void *a = nullptr, *a2 = nullptr, *a3 = nullptr, *b = nullptr;
    auto lk = pool.lock();
    CHECK(pool.acquire(0, &s1, 1000, &a) == 0 && a);
    CHECK(pool.acquire(0, &s2, 1000, &b) == 0 && b);
    const long rel = FakeMem::releases;
    CHECK(pool.acquire(0, &s1, Pool::GRANULE + 1, &a2) == 0 && a2 && a2 != a);
    CHECK(FakeMem::releases == rel && FakeMem::live.count(a) && FakeMem::live.count(a2));   // nothing was freed
    CHECK(pool.capacity(0, &s1) == 2 * Pool::GRANULE && pool.retired() == 1);
    CHECK(pool.held(0) == 4 * Pool::GRANULE);                       // a, a2 (two granules), b
    CHECK(pool.acquire(0, &s1, 10 * Pool::GRANULE, &a3) == 0 && a3 != a2 && a3 != a);
    CHECK(FakeMem::releases == rel && FakeMem::live.count(a) && FakeMem::live.count(a2) && FakeMem::live.count(a3));
    CHECK(pool.retired() == 2 && pool.blocks() == 2);
    void *again = nullptr;
    CHECK(pool.acquire(0, &s1, 1000, &again) == 0 && again == a3);  // later small requests use the large block
    CHECK(FakeMem::live.count(b));                                  // the other stream's block is untouched
    // the explicit release frees current and retired blocks of that device, each exactly once
    CHECK(pool.release_device(0) == 0);
    CHECK(FakeMem::releases == rel + 4 && FakeMem::live.empty() && pool.blocks() == 0 && pool.retired() == 0);
    CHECK(pool.held(0) == 0);
}

static void test_failed_growth_leaves_a_consistent_entry()
{
    Pool pool;
    int s;
    void *a = nullptr, *b = nullptr;
    auto lk = pool.lock();
    CHECK(pool.acquire(0, &s, 10, &a) == 0);
    FakeMem::fail_next_alloc = 7;
    CHECK(pool.acquire(0, &s, 5 * Pool::GRANULE, &b) == 7 && b == nullptr);
    CHECK(pool.capacity(0, &s) == Pool::GRANULE && FakeMem::live.count(a));   // the old block is still the current one
    CHECK(pool.acquire(0, &s, 10, &b) == 0 && b == a && FakeMem::live.size() == 1);
    pool.release_device(0);
    CHECK(FakeMem::live.empty());
}

static void test_a_full_table_refuses_instead_of_evicting()
{
    Pool pool;
    pool.set_full_code(99);
    std::vector<int> streams(Pool::MAX_BLOCKS + 1);
    std::vector<void *> ptrs(Pool::MAX_BLOCKS);
    void *p = nullptr;
    auto lk = pool.lock();
    for (size_t i = 0; i < Pool::MAX_BLOCKS; ++i) CHECK(pool.acquire(0, &streams[i], 1, &ptrs[i]) == 0);
    const long rel = FakeMem::releases;
    CHECK(pool.acquire(0, &streams[Pool::MAX_BLOCKS], 1, &p) == 99 && p == nullptr);   // full: refused
    CHECK(FakeMem::releases == rel && pool.blocks() == Pool::MAX_BLOCKS);              // and nothing was freed
    for (size_t i = 0; i < Pool::MAX_BLOCKS; ++i) CHECK(FakeMem::live.count(ptrs[i]));
    CHECK(pool.acquire(0, &streams[3], 1, &p) == 0 && p == ptrs[3]);                   // known streams still served
    CHECK(pool.release_device(0) == 0);                                                // the way to make room
    CHECK(pool.acquire(0, &streams[Pool::MAX_BLOCKS], 1, &p) == 0 && p);
    pool.release_device(0);
    CHECK(FakeMem::live.empty());
}

static void test_release_reports_the_first_error()
{
    Pool pool;
    int s1, s2;
    void *a = nullptr, *b = nullptr;
    auto lk = pool.lock();
    CHECK(pool.acquire(0, &s1, 1, &a) == 0 && pool.acquire(0, &s2, 1, &b) == 0);
    FakeMem::fail_next_release = 5;
    CHECK(pool.release_device(0) == 5 && pool.blocks() == 0);
    FakeMem::live.clear();
}

static void test_lock_covers_acquire_to_enqueue()
{
    // Each thread acquires a growing block on ITS stream and "enqueues" (records the pointer as in use) under the
    // lease; a release of a pointer that some thread has in use between acquire and the end of its lease is the bug
    // the lock rules out.
    Pool pool;
    std::atomic<int> in_use_violations{0};
    std::vector<std::thread> th;
    int streams[4];
    for (int t = 0; t < 4; ++t)
        th.emplace_back([&, t] {
            for (int i = 1; i <= 200; ++i)
            {
                auto lk = pool.lock();
                void *p = nullptr;
                if (pool.acquire(0, &streams[t], (size_t)i * (Pool::GRANULE / 4), &p) != 0 || !p) { ++in_use_violations; continue; }
                if (!FakeMem::live.count(p)) ++in_use_violations;          // still live while the lease is held
            }
        });
    for (auto &x : th) x.join();
    CHECK(in_use_violations == 0);
    auto lk = pool.lock();
    CHECK(pool.blocks() == 4);
    pool.release_device(0);
    CHECK(FakeMem::live.empty());
}

int main()
{
    test_per_stream_blocks();
    test_a_pointer_handed_out_stays_valid_after_growth();
    test_failed_growth_leaves_a_consistent_entry();
    test_a_full_table_refuses_instead_of_evicting();
    test_release_reports_the_first_error();
    test_lock_covers_acquire_to_enqueue();
    std::printf(g_failures ? "%d CHECKS FAILED\n" : "ALL PASSED\n", g_failures);
    return g_failures ? 1 : 0;
}
