// Measurement aid, NOT part of the product library: built into libsmall_hip_probe.so, which only bench.py loads.
#include <hip/hip_runtime.h>

namespace
{
typedef float probe_x16 __attribute__((ext_vector_type(16)));

// Measurement aid: every wave issues `iters` rounds of four v_mfma_f32_32x32x2_f32 on registers (no memory traffic
// inside the loop), four rounds per loop iteration (a loop of four MFMAs spends a measurable part of its time in the
// loop's own branch: 138 TFLOP/s instead of 155), i.e. what the matrix pipes sustain on this machine.
__global__ __launch_bounds__(256) void mfma_f32_probe_kernel(int iters, float *sink)
{
    probe_x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    const float a = 1.0f + (float)(threadIdx.x & 3) * 0.25f, b = 0.5f;
    for (int it = 0; it < iters; it += 4)
    {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
    }
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) t += acc[i][0] + acc[i][15];
    if (t == 12345.678f) sink[0] = t;      // keeps the loop alive; never true
}

// Measurement aid: the memory traffic of a bandwidth-bound layer with nothing else in the kernel body.  Reads n_in 16-byte
// pieces and writes the first n_out of them (n_out <= n_in), four independent accesses per lane like the element-wise
// kernels of the library: the time a layer with those tensor sizes cannot beat on this machine in the same cache state.
__global__ __launch_bounds__(256) void stream_probe_kernel(const float4 *__restrict__ in, size_t n_in, float4 *__restrict__ out,
                                                           size_t n_out)
{
    // access k of a wave covers 1 KiB of consecutive memory
    const size_t base = (size_t)blockIdx.x * 1024 + threadIdx.x;
    float4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = base + k * 256 < n_in ? in[base + k * 256] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int k = 0; k < 4; ++k)
    {
        if (base + k * 256 < n_out) out[base + k * 256] = v[k];
        else if (v[k].x == 12345.678f && v[k].y == -8765.4321f) out[0] = v[k];      // keeps the read alive; never true
    }
}
} // namespace

extern "C" {

// in: n_in16 16-byte pieces read, out: the first n_out16 of them written; returns 0 or the HIP error code
int shp_probe_stream(const void *in, size_t n_in16, void *out, size_t n_out16, void *stream)
{
    if (!in || !out || n_in16 == 0 || n_out16 > n_in16) return -1;
    const size_t blocks = (n_in16 + 1023) / 1024;
    hipLaunchKernelGGL(stream_probe_kernel, dim3((unsigned)blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       static_cast<const float4 *>(in), n_in16, static_cast<float4 *>(out), n_out16);
    return (int)hipGetLastError();
}

// Launches `workgroups` workgroups of 4 waves, each issuing 4 * iters MFMAs (iters: a multiple of 4); returns 0 or the
// HIP error code.
int shp_probe_mfma_f32(int workgroups, int iters, float *sink, void *stream)
{
    if (workgroups <= 0 || iters <= 0 || iters % 4 != 0 || !sink) return -1;
    hipLaunchKernelGGL(mfma_f32_probe_kernel, dim3((unsigned)workgroups), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       iters, sink);
    return (int)hipGetLastError();
}

} // extern "C"
