// pack_buffer / unpack_buffer on the device: flat [d0][d1][d2][d3] tensors (NCHW activations,
// OIHW filters) <-> the packed channel-blocked layout, same index map as
// include/small/buffers.hpp:138-283 of the reference (convert_tensor2dc / convert_dc2tensor).
//
// Three kernels, all pure data movement (HBM bound, 1 read + 1 write per element):
//   repack_act16_kernel   activations with a 16-channel block: per block a [16][H*W] <-> [H*W][16]
//                         transpose through a wave-private LDS tile
//   repack_smallc_kernel  2 / 3 channel first-layer inputs, 16-byte accesses on both sides
//                         (1 channel: the two layouts are the same, a copy)
//   repack_generic_kernel any tensor type and blocking (filters once per model, ragged first-layer
//                         inputs): one element per lane, packed side contiguous.
#include "common.h"

using namespace shp;

namespace
{

constexpr int TPB = 256;

struct PackGeom
{
    uint32_t Ci, H, W;          // d1, d2, d3 after the type's adjustments
    uint32_t in_block, out_block;
    uint32_t ci_blocks;         // Ci / in_block
};

// packed offset -> flat offset inside one tensor (32-bit: a tensor has fewer than 2^32 elements)
__device__ __forceinline__ uint32_t flat_of_packed(uint32_t q, const PackGeom g)
{
    const uint32_t o = q % g.out_block; q /= g.out_block;
    const uint32_t i = q % g.in_block;  q /= g.in_block;
    const uint32_t w = q % g.W;         q /= g.W;
    const uint32_t h = q % g.H;         q /= g.H;
    const uint32_t i0 = q % g.ci_blocks;
    const uint32_t o0 = q / g.ci_blocks;
    return (((o0 * g.out_block + o) * g.Ci + i0 * g.in_block + i) * g.H + h) * g.W + w;
}

template <typename T, bool PACK>
__global__ __launch_bounds__(TPB) void repack_generic_kernel(const T *__restrict__ src, T *__restrict__ dst,
                                                             const PackGeom g, uint32_t per_tensor, size_t total)
{
    const size_t e = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (e >= total) return;
    uint32_t q;
    size_t base;
    if (e <= 0xffffffffull)
    {
        const uint32_t n = (uint32_t)e / per_tensor;
        q = (uint32_t)e - n * per_tensor;
        base = (size_t)n * per_tensor;
    }
    else
    {
        const size_t n = e / per_tensor;
        q = (uint32_t)(e - n * per_tensor);
        base = n * per_tensor;
    }
    const uint32_t f = flat_of_packed(q, g);
    if (PACK) dst[base + q] = src[base + f];
    else dst[base + f] = src[base + q];
}

// planes = tensors * channel blocks; both layouts of a plane start at plane * 16 * HW.
// The flat side moves one element per lane and channel row (coalesced over the wave); the packed side
// moves 16-byte vectors that are contiguous over the wave: the 64 pixels x 16 channels of a wave are
// turned round in a wave-private LDS tile (pixel rows padded by 16 bytes against bank conflicts).
// A lane-private turn in registers would leave 64-byte pieces per lane on the packed side, i.e.
// every store instruction writing a quarter of each cache line: measured a quarter slower.
template <typename T, bool PACK>
__global__ __launch_bounds__(TPB) void repack_act16_kernel(const T *__restrict__ src, T *__restrict__ dst,
                                                           uint32_t HW, uint32_t px_blocks)
{
    constexpr int NV = (int)(CB * sizeof(T) / 16);      // 16-byte vectors per pixel: 4 (float) or 1 (uint8)
    constexpr int ROW = NV + 1;                         // padded pixel row in vectors
    __shared__ uint4 tile[TPB / WAVE][WAVE * ROW];
    const uint32_t plane = blockIdx.x / px_blocks;
    const uint32_t lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const uint32_t px0 = (blockIdx.x - plane * px_blocks) * TPB + wave * WAVE;   // first pixel of this wave
    const uint32_t px = px0 + lane;
    const size_t base = (size_t)plane * CB * HW;
    uint4 *mine = &tile[wave][lane * ROW];              // this lane's pixel row
    if (PACK)
    {
        __align__(16) T e[CB] = {};
        if (px < HW)
        {
#pragma unroll
            for (int c = 0; c < CB; ++c) e[c] = src[base + (size_t)c * HW + px];
        }
#pragma unroll
        for (int j = 0; j < NV; ++j) mine[j] = reinterpret_cast<const uint4 *>(e)[j];
        __syncthreads();
        // vector v of the wave's packed block: pixel v / NV, part v % NV
        uint4 *o = reinterpret_cast<uint4 *>(dst + base + (size_t)px0 * CB);
#pragma unroll
        for (int j = 0; j < NV; ++j)
        {
            const uint32_t v = j * WAVE + lane;
            if (px0 + v / NV < HW) o[v] = tile[wave][(v / NV) * ROW + (v % NV)];
        }
    }
    else
    {
        const uint4 *i = reinterpret_cast<const uint4 *>(src + base + (size_t)px0 * CB);
#pragma unroll
        for (int j = 0; j < NV; ++j)
        {
            const uint32_t v = j * WAVE + lane;
            if (px0 + v / NV < HW) tile[wave][(v / NV) * ROW + (v % NV)] = i[v];
        }
        __syncthreads();
        __align__(16) T e[CB];
#pragma unroll
        for (int j = 0; j < NV; ++j) reinterpret_cast<uint4 *>(e)[j] = mine[j];
        if (px < HW)
        {
#pragma unroll
            for (int c = 0; c < CB; ++c) dst[base + (size_t)c * HW + px] = e[c];
        }
    }
}

// First-layer inputs: C in {2, 3} channels, [C][HW] <-> [HW][C].  A lane owns VE = 16 / sizeof(T)
// consecutive pixels: C vector accesses on the flat side (one per channel plane) and C on the packed
// side (its VE * C consecutive elements).  Needs HW % VE == 0 (planes stay 16-byte aligned).
template <typename T, int C, bool PACK>
__global__ __launch_bounds__(TPB) void repack_smallc_kernel(const T *__restrict__ src, T *__restrict__ dst,
                                                            uint32_t HW, uint32_t groups_per_tensor, size_t total_groups)
{
    constexpr int VE = 16 / (int)sizeof(T);
    const size_t gidx = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (gidx >= total_groups) return;
    const size_t n = gidx / groups_per_tensor;
    const uint32_t g = (uint32_t)(gidx - n * groups_per_tensor);
    const size_t base = n * (size_t)C * HW;
    __align__(16) T planar[C][VE];
    __align__(16) T inter[VE * C];
    if (PACK)
    {
#pragma unroll
        for (int c = 0; c < C; ++c)
            *reinterpret_cast<uint4 *>(planar[c]) = *reinterpret_cast<const uint4 *>(src + base + (size_t)c * HW + (size_t)g * VE);
#pragma unroll
        for (int i = 0; i < VE; ++i)
#pragma unroll
            for (int c = 0; c < C; ++c) inter[i * C + c] = planar[c][i];
#pragma unroll
        for (int c = 0; c < C; ++c)
            reinterpret_cast<uint4 *>(dst + base + (size_t)g * VE * C)[c] = reinterpret_cast<const uint4 *>(inter)[c];
    }
    else
    {
#pragma unroll
        for (int c = 0; c < C; ++c)
            reinterpret_cast<uint4 *>(inter)[c] = reinterpret_cast<const uint4 *>(src + base + (size_t)g * VE * C)[c];
#pragma unroll
        for (int i = 0; i < VE; ++i)
#pragma unroll
            for (int c = 0; c < C; ++c) planar[c][i] = inter[i * C + c];
#pragma unroll
        for (int c = 0; c < C; ++c)
            *reinterpret_cast<uint4 *>(dst + base + (size_t)c * HW + (size_t)g * VE) = *reinterpret_cast<const uint4 *>(planar[c]);
    }
}

template <typename T, int C, bool PACK>
int launch_smallc(size_t tensors, uint32_t HW, const T *src, T *dst, hipStream_t st, const char *who)
{
    constexpr uint32_t VE = 16 / sizeof(T);
    const uint32_t groups = HW / VE;
    const size_t total = tensors * groups;
    hipLaunchKernelGGL((repack_smallc_kernel<T, C, PACK>), dim3((uint32_t)((total + TPB - 1) / TPB)), dim3(TPB), 0, st,
                       src, dst, HW, groups, total);
    SHP_LAUNCH_CHECK(who);
    return SMALL_HIP_OK;
}

template <typename T, bool PACK>
int repack_t(int batch, uint32_t Co, const PackGeom &g, const T *src, T *dst, hipStream_t st, const char *who)
{
    const uint64_t per = (uint64_t)Co * g.Ci * g.H * g.W;
    if (per == 0) return SMALL_HIP_OK;
    if (per > 0xffffffffull) return einval("small_hip_pack/unpack: a tensor must have fewer than 2^32 elements");
    const size_t total = (size_t)per * batch;
    const uint32_t HW = g.H * g.W;
    if (g.out_block == 1 && g.in_block == CB && aligned16(PACK ? (const void *)dst : (const void *)src))
    {
        const uint32_t px_blocks = (HW + TPB - 1) / TPB;
        const uint64_t planes = (uint64_t)batch * Co * g.ci_blocks;
        if (planes * px_blocks <= 0x7fffffffull)
        {
            hipLaunchKernelGGL((repack_act16_kernel<T, PACK>), dim3((uint32_t)(planes * px_blocks)), dim3(TPB), 0, st,
                               src, dst, HW, px_blocks);
            SHP_LAUNCH_CHECK(who);
            return SMALL_HIP_OK;
        }
    }
    // one block of 1, 2 or 3 channels (first-layer inputs): [C][HW] <-> [HW][C]
    if (g.out_block == 1 && g.ci_blocks == 1 && g.in_block <= 3 && total / TPB < 0x7fffffffull)
    {
        if (g.in_block == 1)
        {
            SHP_HIP(hipMemcpyAsync(dst, src, total * sizeof(T), hipMemcpyDeviceToDevice, st));
            return SMALL_HIP_OK;
        }
        if (HW % (16 / sizeof(T)) == 0 && aligned16(src) && aligned16(dst))
        {
            const size_t tensors = (size_t)batch * Co;
            if (g.in_block == 2) return launch_smallc<T, 2, PACK>(tensors, HW, src, dst, st, who);
            return launch_smallc<T, 3, PACK>(tensors, HW, src, dst, st, who);
        }
    }
    const size_t blocks = (total + TPB - 1) / TPB;
    if (blocks > 0x7fffffffull) return einval("small_hip_pack/unpack: too many elements for one launch");
    hipLaunchKernelGGL((repack_generic_kernel<T, PACK>), dim3((uint32_t)blocks), dim3(TPB), 0, st, src, dst, g,
                       (uint32_t)per, total);
    SHP_LAUNCH_CHECK(who);
    return SMALL_HIP_OK;
}

// the reference's adjustments of blocking and extents per tensor type (buffers.hpp:150-198)
int make_geom(int type, uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3, uint32_t cib, uint32_t cob,
              PackGeom *g, uint32_t *Co)
{
    if (cib == 0 || cob == 0) return einval("small_hip_pack/unpack: zero channel block");
    if (type == SMALL_HIP_FILTER_FC) d2 = d3 = 1;
    if (type == SMALL_HIP_FILTER_DW) cib = 1;
    if ((type == SMALL_HIP_FILTER_CONV || type == SMALL_HIP_INPUT) && d1 < cib) cib = d1;
    uint32_t ib, ob;
    switch (type)
    {
    case SMALL_HIP_INPUT: ib = cib; ob = 1; break;
    case SMALL_HIP_OUTPUT: ib = cob; ob = 1; break;
    case SMALL_HIP_FILTER_DW:
    case SMALL_HIP_FILTER_CONV:
    case SMALL_HIP_FILTER_FC: ib = cib; ob = cob; break;
    default: return einval("small_hip_pack/unpack: unsupported tensor buffer type");
    }
    if (ib == 0 || d1 % ib != 0 || d0 % ob != 0)
        return einval("small_hip_pack/unpack: extents are not multiples of the channel blocks");
    g->Ci = d1; g->H = d2; g->W = d3;
    g->in_block = ib; g->out_block = ob; g->ci_blocks = d1 / ib;
    *Co = d0;
    return SMALL_HIP_OK;
}

template <bool PACK>
int repack(const char *who, int type, int batch, uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3, uint32_t cib,
           uint32_t cob, const void *src, void *dst, size_t esize, small_hip_stream_t stream)
{
    if (batch <= 0 || !src || !dst || (esize != 1 && esize != 4)) return einval("small_hip_pack/unpack: bad argument");
    if (src == dst) return einval("small_hip_pack/unpack: in-place conversion is not possible");
    PackGeom g;
    uint32_t Co;
    if (int rc = make_geom(type, d0, d1, d2, d3, cib, cob, &g, &Co)) return rc;
    if (esize == 4)
        return repack_t<float, PACK>(batch, Co, g, static_cast<const float *>(src), static_cast<float *>(dst),
                                     as_stream(stream), who);
    return repack_t<uint8_t, PACK>(batch, Co, g, static_cast<const uint8_t *>(src), static_cast<uint8_t *>(dst),
                                   as_stream(stream), who);
}

} // namespace

extern "C"
{

int small_hip_pack(int type, int batch, uint32_t dim0, uint32_t dim1, uint32_t dim2, uint32_t dim3, uint32_t c_ib,
                   uint32_t c_ob, const void *flat, void *packed, size_t element_size, small_hip_stream_t stream)
{
    return repack<true>("small_hip_pack", type, batch, dim0, dim1, dim2, dim3, c_ib, c_ob, flat, packed,
                        element_size, stream);
}

int small_hip_unpack(int type, int batch, uint32_t dim0, uint32_t dim1, uint32_t dim2, uint32_t dim3, uint32_t c_ib,
                     uint32_t c_ob, const void *packed, void *flat, size_t element_size, small_hip_stream_t stream)
{
    return repack<false>("small_hip_unpack", type, batch, dim0, dim1, dim2, dim3, c_ib, c_ob, packed, flat,
                         element_size, stream);
}

} // extern "C"
