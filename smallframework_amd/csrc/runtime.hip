// Runtime helpers of the C ABI: error strings, device memory, copies.
#include "common.h"
#include "workspace.h"

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

WorkspacePool<HipMem> &pool()
{
    static WorkspacePool<HipMem> *p = [] {
        auto *q = new WorkspacePool<HipMem>();       // never destroyed: blocks outlive static destruction order
        q->set_full_code(SMALL_HIP_ENOMEM);
        return q;
    }();
    return *p;
}
} // namespace

int lease_workspace(size_t bytes, hipStream_t stream, WorkspaceLease *lease)
{
    int dev = 0;
    SHP_HIP(hipGetDevice(&dev));
    lease->lock = pool().lock();
    int rc = pool().acquire(dev, stream, bytes, &lease->ptr);
    if (rc != SMALL_HIP_OK)
    {
        if (rc == SMALL_HIP_ENOMEM && small_hip_last_error()[0] == 0) set_error("workspace: too many streams hold a block");
        lease->lock.unlock();
    }
    return rc;
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
    default: return "unknown status";
    }
}

const char *small_hip_last_error(void) { return g_err; }

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

} // extern "C"
