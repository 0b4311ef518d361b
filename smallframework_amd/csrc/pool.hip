// MaxPool2D / AveragePool2D, float32 and uint8.  Bandwidth-bound: one lane produces four
// channels (16 bytes of float, or 4 bytes of uint8) of one output pixel; the four lanes of a
// pixel-block read one 64-byte line per tap, neighbouring lanes read neighbouring pixels.
//
// Reference semantics kept bit-for-bit:
//   - max-pool windows that touch padding include the value 0 in the maximum
//     (abstract_layer.hpp:514-521, 718-728 zero the tile and only max valid taps)
//   - average-pool multiplies the sum of the valid taps by float(1.0 / (kh*kw))
//     (abstract_layer.hpp:565-569), i.e. padded positions count in the divisor
#include "common.h"
#include "quant.h"

using namespace shp;

namespace
{

constexpr int TPB = 256;

template <bool IS_MAX>
__global__ __launch_bounds__(TPB) void pool_f32_kernel(const float4 *__restrict__ in,
                                                       float4 *__restrict__ out, size_t total4,
                                                       Geom g, float norm)
{
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= total4) return;
    const int q = (int)(i & 3);
    const PixelPos pp = split_pixel(i >> 2, g.Wo, g.Ho);
    const int ow = pp.ow, oh = pp.oh;
    const size_t plane = pp.plane;                        // n * cblocks + cb
    const float4 *src = in + plane * (size_t)g.H * g.W * 4 + q;
    const int ih0 = oh * g.stride_h - g.pt, iw0 = ow * g.stride - g.pl;
    const bool full = ih0 >= 0 && iw0 >= 0 && ih0 + g.kh <= g.H && iw0 + g.kw <= g.W;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (IS_MAX && full) acc = src[((size_t)ih0 * g.W + iw0) * 4];
    for (int a = 0; a < g.kh; ++a)
    {
        const int ih = ih0 + a;
        if (ih < 0 || ih >= g.H) continue;
        for (int b = 0; b < g.kw; ++b)
        {
            const int iw = iw0 + b;
            if (iw < 0 || iw >= g.W) continue;
            const float4 v = src[((size_t)ih * g.W + iw) * 4];
            if (IS_MAX)
            {
                acc.x = v.x > acc.x ? v.x : acc.x; acc.y = v.y > acc.y ? v.y : acc.y;
                acc.z = v.z > acc.z ? v.z : acc.z; acc.w = v.w > acc.w ? v.w : acc.w;
            }
            else
            {
                acc.x = acc.x + v.x; acc.y = acc.y + v.y; acc.z = acc.z + v.z; acc.w = acc.w + v.w;
            }
        }
    }
    if (!IS_MAX) { acc.x *= norm; acc.y *= norm; acc.z *= norm; acc.w *= norm; }
    out[i] = acc;
}

// Fixed-window variant (2x2 and 3x3 cover the networks in use): the taps are unrolled and every
// load is issued before the first use, out-of-image taps read a clamped address and are replaced
// by 0.  For max that is the reference rule itself (a window that touches padding includes 0, an
// interior window has no replaced tap); for average, adding +0 leaves the running sum unchanged.
template <bool IS_MAX, int KH, int KW>
__global__ __launch_bounds__(TPB) void pool_win_f32_kernel(const float4 *__restrict__ in,
                                                           float4 *__restrict__ out, size_t total4,
                                                           Geom g, float norm)
{
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= total4) return;
    const int q = (int)(i & 3);
    const PixelPos pp = split_pixel(i >> 2, g.Wo, g.Ho);
    const int ow = pp.ow, oh = pp.oh;
    const size_t plane = pp.plane;
    const float4 *src = in + plane * (size_t)g.H * g.W * 4 + q;
    const int ih0 = oh * g.stride_h - g.pt, iw0 = ow * g.stride - g.pl;
    float4 v[KH * KW];
#pragma unroll
    for (int a = 0; a < KH; ++a)
#pragma unroll
        for (int b = 0; b < KW; ++b)
        {
            const int ih = ih0 + a, iw = iw0 + b;
            const int ihc = min(max(ih, 0), g.H - 1), iwc = min(max(iw, 0), g.W - 1);
            v[a * KW + b] = src[((size_t)ihc * g.W + iwc) * 4];
        }
    const bool full = ih0 >= 0 && iw0 >= 0 && ih0 + KH <= g.H && iw0 + KW <= g.W;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (IS_MAX && full) acc = v[0];
#pragma unroll
    for (int a = 0; a < KH; ++a)
#pragma unroll
        for (int b = 0; b < KW; ++b)
        {
            const int ih = ih0 + a, iw = iw0 + b;
            const bool ok = ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
            float4 t = v[a * KW + b];
            if (!ok) t = make_float4(0.f, 0.f, 0.f, 0.f);
            if (IS_MAX)
            {
                acc.x = t.x > acc.x ? t.x : acc.x; acc.y = t.y > acc.y ? t.y : acc.y;
                acc.z = t.z > acc.z ? t.z : acc.z; acc.w = t.w > acc.w ? t.w : acc.w;
            }
            else
            {
                acc.x = acc.x + t.x; acc.y = acc.y + t.y; acc.z = acc.z + t.z; acc.w = acc.w + t.w;
            }
        }
    if (!IS_MAX) { acc.x *= norm; acc.y *= norm; acc.z *= norm; acc.w *= norm; }
    out[i] = acc;
}

// uint8: a lane owns 4 channels (one dword) of one output pixel
template <bool IS_MAX>
__global__ __launch_bounds__(TPB) void pool_u8_kernel(const uint32_t *__restrict__ in,
                                                      uint32_t *__restrict__ out, size_t total,
                                                      Geom g, int32_t zi, QOut qo)
{
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= total) return;
    const int q = (int)(i & 3);
    const PixelPos pp = split_pixel(i >> 2, g.Wo, g.Ho);
    const int ow = pp.ow, oh = pp.oh;
    const size_t plane = pp.plane;
    const uint32_t *src = in + plane * (size_t)g.H * g.W * 4 + q;
    const int ih0 = oh * g.stride_h - g.pt, iw0 = ow * g.stride - g.pl;
    const bool full = ih0 >= 0 && iw0 >= 0 && ih0 + g.kh <= g.H && iw0 + g.kw <= g.W;
    int32_t acc[4] = {0, 0, 0, 0};
    if (IS_MAX && full)
    {
        // q_abstract_layer.hpp:286-293: un-padded windows start from the first RAW byte
        const uint32_t v = src[((size_t)ih0 * g.W + iw0) * 4];
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[b] = (int32_t)((v >> (8 * b)) & 0xffu);
    }
    for (int a = 0; a < g.kh; ++a)
    {
        const int ih = ih0 + a;
        if (ih < 0 || ih >= g.H) continue;
        for (int c = 0; c < g.kw; ++c)
        {
            const int iw = iw0 + c;
            if (iw < 0 || iw >= g.W) continue;
            const uint32_t v = src[((size_t)ih * g.W + iw) * 4];
#pragma unroll
            for (int b = 0; b < 4; ++b)
            {
                const int32_t x = (int32_t)((v >> (8 * b)) & 0xffu) + zi;
                if (IS_MAX) acc[b] = x > acc[b] ? x : acc[b];
                else acc[b] = (int32_t)((uint32_t)acc[b] + (uint32_t)x);
            }
        }
    }
    uint32_t packed = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) packed |= requant_u8(acc[b], qo) << (8 * b);
    out[i] = packed;
}

// Global pooling (the window is the whole un-padded image, one output pixel per channel): one wave
// per (image, channel block).  Lane = (pixel slot, channel quad): the 16 slots stride over the
// pixels with 16-byte (float) / 4-byte (uint8) accesses, i.e. the wave reads whole kilobytes /
// 256-byte runs, then the slots are combined with a wavefront xor-shuffle reduction.
template <bool IS_MAX>
__global__ __launch_bounds__(TPB) void global_pool_f32_kernel(const float4 *__restrict__ in,
                                                              float4 *__restrict__ out, int planes, int hw,
                                                              float norm)
{
    const int plane = blockIdx.x * (TPB / 64) + (threadIdx.x >> 6);
    if (plane >= planes) return;                     // whole waves leave together
    const int lane = threadIdx.x & 63, q = lane & 3, slot = lane >> 2;
    const float4 *src = in + (size_t)plane * hw * 4 + q;
    // every slot starts from pixel 0 for max (any element of the window is a valid start value)
    float4 acc = IS_MAX ? src[0] : make_float4(0.f, 0.f, 0.f, 0.f);
    for (int p = slot; p < hw; p += 16)
    {
        const float4 v = src[(size_t)p * 4];
        if (IS_MAX)
        {
            acc.x = v.x > acc.x ? v.x : acc.x; acc.y = v.y > acc.y ? v.y : acc.y;
            acc.z = v.z > acc.z ? v.z : acc.z; acc.w = v.w > acc.w ? v.w : acc.w;
        }
        else { acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w; }
    }
#pragma unroll
    for (int m = 4; m < 64; m <<= 1)
    {
        const float ox = __shfl_xor(acc.x, m), oy = __shfl_xor(acc.y, m);
        const float oz = __shfl_xor(acc.z, m), ow = __shfl_xor(acc.w, m);
        if (IS_MAX)
        {
            acc.x = ox > acc.x ? ox : acc.x; acc.y = oy > acc.y ? oy : acc.y;
            acc.z = oz > acc.z ? oz : acc.z; acc.w = ow > acc.w ? ow : acc.w;
        }
        else { acc.x += ox; acc.y += oy; acc.z += oz; acc.w += ow; }
    }
    if (!IS_MAX) { acc.x *= norm; acc.y *= norm; acc.z *= norm; acc.w *= norm; }
    if (slot == 0) out[(size_t)plane * 4 + q] = acc;
}

template <bool IS_MAX>
__global__ __launch_bounds__(TPB) void global_pool_u8_kernel(const uint32_t *__restrict__ in,
                                                             uint32_t *__restrict__ out, int planes, int hw,
                                                             int32_t zi, QOut qo)
{
    const int plane = blockIdx.x * (TPB / 64) + (threadIdx.x >> 6);
    if (plane >= planes) return;
    const int lane = threadIdx.x & 63, q = lane & 3, slot = lane >> 2;
    const uint32_t *src = in + (size_t)plane * hw * 4 + q;
    int32_t acc[4];
    {
        // un-padded max windows start from the first RAW byte (q_abstract_layer.hpp:286-293)
        const uint32_t v0 = src[0];
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[b] = IS_MAX ? (int32_t)((v0 >> (8 * b)) & 0xffu) : 0;
    }
    for (int p = slot; p < hw; p += 16)
    {
        const uint32_t v = src[(size_t)p * 4];
#pragma unroll
        for (int b = 0; b < 4; ++b)
        {
            const int32_t x = (int32_t)((v >> (8 * b)) & 0xffu) + zi;
            if (IS_MAX) acc[b] = x > acc[b] ? x : acc[b];
            else acc[b] = (int32_t)((uint32_t)acc[b] + (uint32_t)x);
        }
    }
#pragma unroll
    for (int m = 4; m < 64; m <<= 1)
#pragma unroll
        for (int b = 0; b < 4; ++b)
        {
            const int32_t o = __shfl_xor(acc[b], m);
            if (IS_MAX) acc[b] = o > acc[b] ? o : acc[b];
            else acc[b] = (int32_t)((uint32_t)acc[b] + (uint32_t)o);
        }
    if (slot == 0)
    {
        uint32_t packed = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) packed |= requant_u8(acc[b], qo) << (8 * b);
        out[(size_t)plane * 4 + q] = packed;
    }
}

inline bool is_global(const Geom &g, int pt, int pb, int pl, int pr)
{
    return g.kh == g.H && g.kw == g.W && pt == 0 && pb == 0 && pl == 0 && pr == 0 && g.H * g.W >= 16;
}

int pool_check(const char *op, bool avg, int batch, int kh, int kw, int stride, int stride_h, int pt, int pb, int pl,
               int pr, int C, int H, int W, const void *in, const void *out, Geom *g)
{
    // interface_abstract.hpp:797-833 / 929-977: channel test first, then stride
    if (C <= 0 || C % CB != 0) return SMALL_HIP_ECHANNELS;
    if (avg ? (stride < 1 || stride > 3) : (stride != 1 && stride != 2)) return SMALL_HIP_ESTRIDE;
    if (batch <= 0 || kh <= 0 || kw <= 0 || H <= 0 || W <= 0 || !pads_ok(pt, pb, pl, pr))
    { set_error("%s: bad size", op); return SMALL_HIP_EINVAL; }
    if (!in || !out || !aligned16(in) || !aligned16(out)) { set_error("%s: null or misaligned pointer", op); return SMALL_HIP_EINVAL; }
    if (in == out) { set_error("%s: in-place pooling is not supported", op); return SMALL_HIP_EINVAL; }
    if ((long)batch * (C / CB) > 0x7fffffffL || (long)H * W > 0x7fffffffL)
    { set_error("%s: batch * C / 16 or H * W too large", op); return SMALL_HIP_EINVAL; }
    g->H = H; g->W = W; g->kh = kh; g->kw = kw; g->stride = stride; g->pt = pt; g->pl = pl;
    g->stride_h = stride_h ? stride_h : stride;
    g->Ho = out_dim(H, pt, pb, kh, g->stride_h);
    g->Wo = out_dim(W, pl, pr, kw, stride);
    return SMALL_HIP_OK;
}

template <bool IS_MAX>
int pool_f32(const char *op, int batch, int kh, int kw, int stride, int stride_h, int pt, int pb, int pl, int pr, int C,
             int H, int W, const float *in, float *out, small_hip_stream_t stream)
{
    Geom g;
    if (int rc = pool_check(op, !IS_MAX, batch, kh, kw, stride, stride_h, pt, pb, pl, pr, C, H, W, in, out, &g)) return rc;
    const size_t total4 = (size_t)batch * C * g.Ho * g.Wo / 4;
    if (total4 == 0) return SMALL_HIP_OK;
    const float norm = (float)(1.0 / (1.0 * kh * kw));
    if (is_global(g, pt, pb, pl, pr))
    {
        const int planes = batch * (C / CB);
        hipLaunchKernelGGL(global_pool_f32_kernel<IS_MAX>, dim3((planes + TPB / 64 - 1) / (TPB / 64)), dim3(TPB), 0,
                           as_stream(stream), reinterpret_cast<const float4 *>(in), reinterpret_cast<float4 *>(out),
                           planes, H * W, norm);
        SHP_LAUNCH_CHECK(op);
        return SMALL_HIP_OK;
    }
    auto kern = pool_f32_kernel<IS_MAX>;
    if (kh == 2 && kw == 2) kern = pool_win_f32_kernel<IS_MAX, 2, 2>;
    if (kh == 3 && kw == 3) kern = pool_win_f32_kernel<IS_MAX, 3, 3>;
    hipLaunchKernelGGL(kern, dim3((unsigned)((total4 + TPB - 1) / TPB)), dim3(TPB), 0,
                       as_stream(stream), reinterpret_cast<const float4 *>(in),
                       reinterpret_cast<float4 *>(out), total4, g, norm);
    SHP_LAUNCH_CHECK(op);
    return SMALL_HIP_OK;
}

template <bool IS_MAX>
int pool_u8(const char *op, int batch, int kh, int kw, int stride, int stride_h, int pt, int pb, int pl, int pr, int C,
            int H, int W, const uint8_t *in, const small_hip_quant *iq, uint8_t *out,
            const small_hip_quant *oq, small_hip_stream_t stream)
{
    if (!iq || !oq) { set_error("%s: null quantisation parameters", op); return SMALL_HIP_EINVAL; }
    Geom g;
    if (int rc = pool_check(op, !IS_MAX, batch, kh, kw, stride, stride_h, pt, pb, pl, pr, C, H, W, in, out, &g)) return rc;
    const size_t total = (size_t)batch * C * g.Ho * g.Wo / 4;
    if (total == 0) return SMALL_HIP_OK;
    const QOut q = make_qout(oq->multiplier, oq->lshift, oq->rshift);
    if (is_global(g, pt, pb, pl, pr))
    {
        const int planes = batch * (C / CB);
        hipLaunchKernelGGL(global_pool_u8_kernel<IS_MAX>, dim3((planes + TPB / 64 - 1) / (TPB / 64)), dim3(TPB), 0,
                           as_stream(stream), reinterpret_cast<const uint32_t *>(in),
                           reinterpret_cast<uint32_t *>(out), planes, H * W, iq->zero, q);
        SHP_LAUNCH_CHECK(op);
        return SMALL_HIP_OK;
    }
    hipLaunchKernelGGL(pool_u8_kernel<IS_MAX>, dim3((unsigned)((total + TPB - 1) / TPB)), dim3(TPB), 0,
                       as_stream(stream), reinterpret_cast<const uint32_t *>(in),
                       reinterpret_cast<uint32_t *>(out), total, g, iq->zero, q);
    SHP_LAUNCH_CHECK(op);
    return SMALL_HIP_OK;
}

} // namespace

extern "C" {

int small_hip_maxpool2d_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int C,
                            int H, int W, const float *in, float *out, small_hip_stream_t stream)
{
    return pool_f32<true>("small_hip_maxpool2d_f32", batch, kh, kw, stride, 0, pt, pb, pl, pr, C, H, W, in, out, stream);
}

int small_hip_avgpool2d_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int C,
                            int H, int W, const float *in, float *out, small_hip_stream_t stream)
{
    return pool_f32<false>("small_hip_avgpool2d_f32", batch, kh, kw, stride, 0, pt, pb, pl, pr, C, H, W, in, out, stream);
}

int small_hip_maxpool2d_u8(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int C,
                           int H, int W, const uint8_t *in, const small_hip_quant *iq, uint8_t *out,
                           const small_hip_quant *oq, small_hip_stream_t stream)
{
    return pool_u8<true>("small_hip_maxpool2d_u8", batch, kh, kw, stride, 0, pt, pb, pl, pr, C, H, W, in, iq, out, oq, stream);
}

int small_hip_avgpool2d_u8(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int C,
                           int H, int W, const uint8_t *in, const small_hip_quant *iq, uint8_t *out,
                           const small_hip_quant *oq, small_hip_stream_t stream)
{
    return pool_u8<false>("small_hip_avgpool2d_u8", batch, kh, kw, stride, 0, pt, pb, pl, pr, C, H, W, in, iq, out, oq, stream);
}

// The 1-D pooling layers (interface_abstract_1D.hpp:776-1100): `rows` independent signals of `width` samples in one
// [C/16][rows][width][16] tensor, a 1 x k window moved by `stride` along the width only.
int small_hip_pool1d_f32(int is_max, int batch, int k, int stride, int l_pad, int r_pad, int C, int rows, int width,
                         const float *in, float *out, small_hip_stream_t stream)
{
    return is_max ? pool_f32<true>("small_hip_pool1d_f32", batch, 1, k, stride, 1, 0, 0, l_pad, r_pad, C, rows, width, in, out, stream)
                  : pool_f32<false>("small_hip_pool1d_f32", batch, 1, k, stride, 1, 0, 0, l_pad, r_pad, C, rows, width, in, out, stream);
}

int small_hip_pool1d_u8(int is_max, int batch, int k, int stride, int l_pad, int r_pad, int C, int rows, int width,
                        const uint8_t *in, const small_hip_quant *iq, uint8_t *out, const small_hip_quant *oq,
                        small_hip_stream_t stream)
{
    return is_max ? pool_u8<true>("small_hip_pool1d_u8", batch, 1, k, stride, 1, 0, 0, l_pad, r_pad, C, rows, width, in, iq, out, oq, stream)
                  : pool_u8<false>("small_hip_pool1d_u8", batch, 1, k, stride, 1, 0, 0, l_pad, r_pad, C, rows, width, in, iq, out, oq, stream);
}

} // extern "C"
