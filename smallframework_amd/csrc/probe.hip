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
// Measurement aid: do the matrix instructions of one wave and the vector-ALU instructions of ANOTHER wave on the same SIMD
// overlap?  A workgroup is eight waves, two per SIMD.  Waves 0-3 issue 16 * iters v_mfma_f32_32x32x2_f32 on two accumulators
// (16 x 64 = 1024 cycles per iteration) when `mode` has bit 0; waves 4-7 issue 256 * iters independent vector FMAs
// (256 x 4 = 1024 cycles per iteration) when it has bit 1.  Timed one after the other and together.
__global__ __launch_bounds__(512) void issue_overlap_probe_kernel(int mode, int iters, float *sink)
{
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    float r = 0.f;
    if (wave < 4)
    {
        if (mode & 1)
        {
            probe_x16 a0, a1;
#pragma unroll
            for (int i = 0; i < 16; ++i) { a0[i] = 0.f; a1[i] = 0.f; }
            const float x = (float)lane, y = 1.0f;
            for (int i = 0; i < iters; ++i)
            {
#pragma unroll
                for (int k = 0; k < 8; ++k)
                {
                    a0 = __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, a0, 0, 0, 0);
                    a1 = __builtin_amdgcn_mfma_f32_32x32x2f32(y, x, a1, 0, 0, 0);
                }
            }
            r = a0[0] + a1[3];
        }
    }
    else if (mode & 2)
    {
        float f0 = (float)lane, f1 = 1.f, f2 = 2.f, f3 = 3.f, f4 = 4.f, f5 = 5.f, f6 = 6.f, f7 = 7.f;
        const float m = 1.0001f, c = 0.5f;
        for (int i = 0; i < iters; ++i)
        {
#pragma unroll
            for (int k = 0; k < 32; ++k)
            {
                f0 = fmaf(f0, m, c); f1 = fmaf(f1, m, c); f2 = fmaf(f2, m, c); f3 = fmaf(f3, m, c);
                f4 = fmaf(f4, m, c); f5 = fmaf(f5, m, c); f6 = fmaf(f6, m, c); f7 = fmaf(f7, m, c);
            }
        }
        r = f0 + f1 + f2 + f3 + f4 + f5 + f6 + f7;
    }
    if (r == 12345.678f) sink[0] = r;      // keeps the loops alive; never true
}
} // namespace

extern "C" {

// mode: 1 = matrix waves only, 2 = vector waves only, 3 = both in the same launch; one workgroup per CU is the intended use
int shp_probe_issue_overlap(int workgroups, int mode, int iters, float *sink, void *stream)
{
    if (workgroups <= 0 || iters <= 0 || mode < 1 || mode > 3 || !sink) return -1;
    hipLaunchKernelGGL(issue_overlap_probe_kernel, dim3((unsigned)workgroups), dim3(512), 0, reinterpret_cast<hipStream_t>(stream),
                       mode, iters, sink);
    return (int)hipGetLastError();
}

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
