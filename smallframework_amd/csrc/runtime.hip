// Runtime helpers of the C ABI: error strings, device memory, copies.
#include "common.h"
#include "workspace.h"

#include <cstdlib>
#include <cstring>
#include <mutex>

namespace shp
{
static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

namespace
{
struct HipMem
{
    static int alloc(void **p, size_t bytes)
    {
        hipError_t e = hipMalloc(p, bytes);
        if (e == hipSuccess) return SMALL_HIP_OK;
        (void)hipGetLastError();
        set_error("workspace hipMalloc(%zu): %s", bytes, hipGetErrorString(e));
        return e == hipErrorOutOfMemory ? SMALL_HIP_ENOMEM : SMALL_HIP_EHIP;
    }
    // hipFree waits for the device, so no queued kernel still reads the block when it returns
    static int release(void *p)
    {
        hipError_t e = hipFree(p);
        return e == hipSuccess ? SMALL_HIP_OK : fail_hip(e, "workspace hipFree");
    }
};

// never destroyed: the blocks outlive static destruction order
WorkspacePool<HipMem> &pool()
{
    static WorkspacePool<HipMem> *p = [] {
        auto *q = new WorkspacePool<HipMem>();
        q->set_full_code(SMALL_HIP_ENOMEM);
        return q;
    }();
    return *p;
}
} // namespace

int lease_workspace(size_t bytes, hipStream_t stream, WorkspaceLease *lease)
{
    auto &pl = pool();
    int dev = 0;
    SHP_HIP(hipGetDevice(&dev));
    lease->lock = pl.lock();
    int rc = pl.acquire(dev, stream, bytes, &lease->ptr);
    if (rc != SMALL_HIP_OK)
    {
        if (rc == SMALL_HIP_ENOMEM && small_hip_last_error()[0] == 0)
            set_error("workspace: %zu streams hold a block already; small_hip_workspace_release() makes room", pl.blocks());
        lease->lock.unlock();
    }
    return rc;
}

// SMALL_HIP_TUNE="key=value,key=value": the value of `key`, or null
static const char *tune_find(const char *key)
{
    const char *env = std::getenv("SMALL_HIP_TUNE");     // call sites on launch paths keep the answer in a static
    if (!env) return nullptr;
    const size_t n = std::strlen(key);
    for (const char *p = env; *p;)
    {
        if (std::strncmp(p, key, n) == 0 && p[n] == '=') return p + n + 1;
        const char *c = std::strchr(p, ',');
        if (!c) break;
        p = c + 1;
    }
    return nullptr;
}

int tune_int(const char *key, int dflt)
{
    const char *v = tune_find(key);
    return v ? std::atoi(v) : dflt;
}

bool tune_pair(const char *key, int *a, int *b)
{
    const char *v = tune_find(key);
    return v && std::sscanf(v, "%dx%d", a, b) == 2;
}

} // namespace shp

using namespace shp;

extern "C" {

const char *small_hip_version(void) { return "small_hip 0.1 (gfx950)"; }

const char *small_hip_strerror(int status)
{
    switch (status)
    {
    case SMALL_HIP_OK: return "ok";
    case SMALL_HIP_ESTRIDE: return "stride unsupported";
    case SMALL_HIP_ECHANNELS: return "in_channels unsupported";
    case SMALL_HIP_ESCALE: return "scale factor unsupported (only 1 or 2)";
    case SMALL_HIP_EINVAL: return "invalid argument";
    case SMALL_HIP_EHIP: return "HIP runtime error";
    case SMALL_HIP_ENOMEM: return "out of memory";
    case SMALL_HIP_EUNSUPPORTED: return "not built for this shape: use the general path";
    default: return "unknown status";
    }
}

const char *small_hip_last_error(void) { return g_err; }

int small_hip_tune_int(const char *key, int default_value) { return key ? tune_int(key, default_value) : default_value; }

int small_hip_device_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int small_hip_set_device(int device)
{
    SHP_HIP(hipSetDevice(device));
    return SMALL_HIP_OK;
}

int small_hip_workspace_reserve(size_t bytes, small_hip_stream_t stream)
{
    g_err[0] = 0;
    WorkspaceLease lease;
    return lease_workspace(bytes, as_stream(stream), &lease);
}

int small_hip_workspace_release(void)
{
    int dev = 0;
    SHP_HIP(hipGetDevice(&dev));
    auto lk = pool().lock();
    return pool().release_device(dev);
}

size_t small_hip_workspace_held(void)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    auto lk = pool().lock();
    return pool().held(dev);
}

int small_hip_malloc(void **ptr, size_t bytes)
{
    if (!ptr) return einval("small_hip_malloc: null result pointer");
    *ptr = nullptr;
    if (bytes == 0) return SMALL_HIP_OK;
    hipError_t e = hipMalloc(ptr, bytes);
    if (e == hipErrorOutOfMemory)
    {
        set_error("hipMalloc(%zu): out of memory", bytes);
        (void)hipGetLastError();
        return SMALL_HIP_ENOMEM;
    }
    if (e != hipSuccess) return fail_hip(e, "hipMalloc");
    return SMALL_HIP_OK;
}

int small_hip_free(void *ptr)
{
    if (ptr) SHP_HIP(hipFree(ptr));
    return SMALL_HIP_OK;
}

int small_hip_host_malloc(void **ptr, size_t bytes)
{
    if (!ptr) return einval("small_hip_host_malloc: null result pointer");
    *ptr = nullptr;
    if (bytes == 0) return SMALL_HIP_OK;
    hipError_t e = hipHostMalloc(ptr, bytes, hipHostMallocDefault);
    if (e == hipErrorOutOfMemory)
    {
        set_error("hipHostMalloc(%zu): out of memory", bytes);
        (void)hipGetLastError();
        return SMALL_HIP_ENOMEM;
    }
    if (e != hipSuccess) return fail_hip(e, "hipHostMalloc");
    return SMALL_HIP_OK;
}

int small_hip_host_free(void *ptr)
{
    if (ptr) SHP_HIP(hipHostFree(ptr));
    return SMALL_HIP_OK;
}

int small_hip_memcpy_h2d(void *dst, const void *src, size_t bytes, small_hip_stream_t stream)
{
    if (bytes == 0) return SMALL_HIP_OK;
    SHP_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    return SMALL_HIP_OK;
}

int small_hip_memcpy_d2h(void *dst, const void *src, size_t bytes, small_hip_stream_t stream)
{
    if (bytes == 0) return SMALL_HIP_OK;
    SHP_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    return SMALL_HIP_OK;
}

int small_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, small_hip_stream_t stream)
{
    if (bytes == 0) return SMALL_HIP_OK;
    SHP_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return SMALL_HIP_OK;
}

int small_hip_memset(void *dst, int value, size_t bytes, small_hip_stream_t stream)
{
    if (bytes == 0) return SMALL_HIP_OK;
    SHP_HIP(hipMemsetAsync(dst, value, bytes, as_stream(stream)));
    return SMALL_HIP_OK;
}

int small_hip_stream_synchronize(small_hip_stream_t stream)
{
    SHP_HIP(hipStreamSynchronize(as_stream(stream)));
    return SMALL_HIP_OK;
}

// ---- uploads that overlap the compute stream -----------------------------------------------------------------
namespace
{
// one copy stream per device, created on first use (default priority, never destroyed)
int copy_stream(hipStream_t *out)
{
    constexpr int MAX_DEV = 64;
    static std::mutex mu;
    static hipStream_t streams[MAX_DEV] = {};
    int dev = 0;
    SHP_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEV) return einval("small_hip_upload_begin: device index out of range");
    std::lock_guard<std::mutex> lk(mu);
    if (!streams[dev]) SHP_HIP(hipStreamCreateWithFlags(&streams[dev], hipStreamNonBlocking));
    *out = streams[dev];
    return SMALL_HIP_OK;
}
} // namespace

int small_hip_upload_begin(void *dst, const void *src, size_t bytes, small_hip_stream_t after, small_hip_event_t *done)
{
    if (!done) return einval("small_hip_upload_begin: null event pointer");
    *done = nullptr;
    if (!dst || !src) return einval("small_hip_upload_begin: null pointer");
    hipStream_t cs = nullptr;
    if (int rc = copy_stream(&cs)) return rc;
    hipEvent_t ev = nullptr;
    SHP_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    // the copy must not overtake work already queued on `after` that still reads dst
    hipError_t e = hipEventRecord(ev, as_stream(after));
    if (e == hipSuccess) e = hipStreamWaitEvent(cs, ev, 0);
    if (e == hipSuccess && bytes) e = hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, cs);
    if (e == hipSuccess) e = hipEventRecord(ev, cs);          // re-recorded: now it marks the end of the copy
    if (e != hipSuccess)
    {
        (void)hipEventDestroy(ev);
        return fail_hip(e, "small_hip_upload_begin");
    }
    *done = ev;
    return SMALL_HIP_OK;
}

int small_hip_upload_wait(small_hip_event_t done, small_hip_stream_t stream)
{
    if (!done) return SMALL_HIP_OK;
    hipEvent_t ev = static_cast<hipEvent_t>(done);
    const hipError_t e = hipStreamWaitEvent(as_stream(stream), ev, 0);
    (void)hipEventDestroy(ev);                                  // released once the queued wait has seen it
    return e == hipSuccess ? SMALL_HIP_OK : fail_hip(e, "small_hip_upload_wait");
}

int small_hip_upload_finish(small_hip_event_t done)
{
    if (!done) return SMALL_HIP_OK;
    hipEvent_t ev = static_cast<hipEvent_t>(done);
    const hipError_t e = hipEventSynchronize(ev);
    (void)hipEventDestroy(ev);
    return e == hipSuccess ? SMALL_HIP_OK : fail_hip(e, "small_hip_upload_finish");
}

} // extern "C"
