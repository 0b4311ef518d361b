// Measurement aid, NOT part of the product library: built into libsmall_hip_probe.so, which only bench.py loads.
#include <hip/hip_runtime.h>

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

// Launches `workgroups` workgroups of 4 waves, each issuing 4 * iters MFMAs; returns 0 or the HIP error code.
int shp_probe_mfma_f32(int workgroups, int iters, float *sink, void *stream)
{
    if (workgroups <= 0 || iters <= 0 || !sink) return -1;
    hipLaunchKernelGGL(mfma_f32_probe_kernel, dim3((unsigned)workgroups), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       iters, sink);
    return (int)hipGetLastError();
}

} // extern "C"
