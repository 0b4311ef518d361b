// Runtime helpers of the C ABI: error strings, device memory, copies.
#include "common.h"

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
constexpr int MAX_DEV = 16;
std::mutex g_ws_mu;
void *g_ws_ptr[MAX_DEV] = {};
size_t g_ws_cap[MAX_DEV] = {};
} // namespace

int get_workspace(size_t bytes, void **ptr)
{
    int dev = 0;
    SHP_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEV) return einval("get_workspace: device index out of range");
    std::lock_guard<std::mutex> lk(g_ws_mu);
    if (bytes > g_ws_cap[dev])
    {
        if (g_ws_ptr[dev])
        {
            // hipFree waits for the device, so no queued kernel still reads the old block
            SHP_HIP(hipFree(g_ws_ptr[dev]));
            g_ws_ptr[dev] = nullptr;
            g_ws_cap[dev] = 0;
        }
        size_t cap = (bytes + (1u << 20) - 1) & ~(size_t)((1u << 20) - 1);
        hipError_t e = hipMalloc(&g_ws_ptr[dev], cap);
        if (e != hipSuccess)
        {
            (void)hipGetLastError();
            set_error("workspace hipMalloc(%zu): %s", cap, hipGetErrorString(e));
            return e == hipErrorOutOfMemory ? SMALL_HIP_ENOMEM : SMALL_HIP_EHIP;
        }
        g_ws_cap[dev] = cap;
    }
    *ptr = g_ws_ptr[dev];
    return SMALL_HIP_OK;
}

} // namespace shp

using namespace shp;

namespace
{
typedef float probe_x16 __attribute__((ext_vector_type(16)));

// Measurement aid: every wave issues `iters` rounds of four independent v_mfma_f32_32x32x2_f32 on registers (no
// memory traffic inside the loop), i.e. what the matrix pipes sustain on this machine at its sustained clock.
__global__ __launch_bounds__(256) void mfma_f32_probe_kernel(int iters, float *sink)
{
    probe_x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    const float a = 1.0f + (float)(threadIdx.x & 3) * 0.25f, b = 0.5f;
    for (int it = 0; it < iters; ++it)
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
    }
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) t += acc[i][0] + acc[i][15];
    if (t == 12345.678f) sink[0] = t;      // keeps the loop alive; never true
}
} // namespace

extern "C" {

int small_hip_mfma_f32_probe(int workgroups, int iters, float *sink, small_hip_stream_t stream)
{
    if (workgroups <= 0 || iters <= 0 || !sink) return shp::einval("small_hip_mfma_f32_probe: bad argument");
    hipLaunchKernelGGL(mfma_f32_probe_kernel, dim3((unsigned)workgroups), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       iters, sink);
    SHP_LAUNCH_CHECK("small_hip_mfma_f32_probe");
    return SMALL_HIP_OK;
}

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
