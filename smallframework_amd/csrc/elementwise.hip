// Bandwidth-bound element-wise layers: ReLU, LeakyReLU, Accum, Bias, UpSample2D, Concat
// (float32) and ReLU / Accum (uint8).  One 16-byte vector per lane and access, four
// independent accesses per lane so that every wave keeps 4 KiB of loads in flight.
#include "common.h"
#include "quant.h"

using namespace shp;

namespace
{

constexpr int TPB = 256;
constexpr int UNROLL = 4;

enum EwOp { EW_RELU, EW_LEAKY, EW_ACCUM, EW_SCALE };

template <int OP>
__device__ __forceinline__ float4 ew_apply(float4 x, float4 o, float slope)
{
    float4 r;
    if (OP == EW_RELU)
    {
        r.x = x.x > 0.f ? x.x : 0.f; r.y = x.y > 0.f ? x.y : 0.f;
        r.z = x.z > 0.f ? x.z : 0.f; r.w = x.w > 0.f ? x.w : 0.f;
    }
    else if (OP == EW_LEAKY)
    {
        r.x = x.x > 0.f ? x.x : x.x * slope; r.y = x.y > 0.f ? x.y : x.y * slope;
        r.z = x.z > 0.f ? x.z : x.z * slope; r.w = x.w > 0.f ? x.w : x.w * slope;
    }
    else if (OP == EW_SCALE)
    {
        r.x = x.x * slope; r.y = x.y * slope; r.z = x.z * slope; r.w = x.w * slope;
    }
    else
    {
        r.x = o.x + x.x; r.y = o.y + x.y; r.z = o.z + x.z; r.w = o.w + x.w;
    }
    return r;
}

// n4 = number of float4 elements
template <int OP>
__global__ __launch_bounds__(TPB) void ew_f32_kernel(const float4 *in, float4 *out,
                                                     size_t n4, float slope)
{
    const size_t base = (size_t)blockIdx.x * (TPB * UNROLL) + threadIdx.x;
    float4 x[UNROLL], o[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
    {
        const size_t i = base + (size_t)u * TPB;
        if (i < n4)
        {
            x[u] = in[i];
            if (OP == EW_ACCUM) o[u] = out[i];
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
    {
        const size_t i = base + (size_t)u * TPB;
        if (i < n4) out[i] = ew_apply<OP>(x[u], o[u], slope);
    }
}

// in == out is allowed (every activation of every model runs in place), so neither pointer above is __restrict__:
// every lane reads its own elements before writing them.

// bias: out[n][cb][p][16] = (accumulate ? out : 0) + bias[cb*16 + c]
template <bool ACC>
__global__ __launch_bounds__(TPB) void bias_f32_kernel(const float4 *__restrict__ bias, float4 *out,
                                                       size_t n4, int hw, int cblocks)
{
    const size_t base = (size_t)blockIdx.x * (TPB * UNROLL) + threadIdx.x;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
    {
        const size_t i = base + (size_t)u * TPB;
        if (i < n4)
        {
            const size_t pix = i >> 2;                        // 4 float4 per (pixel, block)
            const int cbk = (int)((pix / (size_t)hw) % (size_t)cblocks);
            const float4 b = bias[cbk * 4 + (int)(i & 3)];
            float4 r = b;
            if (ACC)
            {
                const float4 o = out[i];
                r.x = o.x + b.x; r.y = o.y + b.y; r.z = o.z + b.z; r.w = o.w + b.w;
            }
            out[i] = r;
        }
    }
}

// nearest-neighbour x2 (along the width, and along the height too when hshift is 1): one lane per output float4
__global__ __launch_bounds__(TPB) void upsample2_f32_kernel(const float4 *__restrict__ in,
                                                            float4 *__restrict__ out, size_t n4out,
                                                            int H, int W, int hshift)
{
    const size_t base = (size_t)blockIdx.x * (TPB * UNROLL) + threadIdx.x;
    const int Wo = 2 * W, Ho = H << hshift;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
    {
        const size_t i = base + (size_t)u * TPB;
        if (i < n4out)
        {
            const int q = (int)(i & 3);
            const PixelPos pp = split_pixel(i >> 2, Wo, Ho);
            const int ow = pp.ow, oh = pp.oh;
            const size_t plane = pp.plane;                    // n * cblocks + cb
            out[i] = in[((plane * H + (oh >> hshift)) * W + (ow >> 1)) * 4 + q];
        }
    }
}

// YOLO head decode (include/small/YOLOLayer.hpp:150-222): packed [C/16][H][W][16] scores -> [anchor][h][w][5 + classes]
// box records.  One lane per output element; consecutive lanes write consecutive floats of a record.
struct YoloAnchors
{
    float w[8], h[8];
};

__global__ __launch_bounds__(TPB) void yolo_decode_f32_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                              size_t n_out, int C, int H, int W, int na, int nrec,
                                                              float stride, YoloAnchors anchors)
{
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n_out) return;
    const int field = (int)(i % (size_t)nrec);
    size_t pred = i / (size_t)nrec;
    const int ow = (int)(pred % (size_t)W);
    pred /= (size_t)W;
    const int oh = (int)(pred % (size_t)H);
    pred /= (size_t)H;                       // n * anchors + anchor
    const int a = (int)(pred % (size_t)na);
    const size_t n = pred / (size_t)na;
    const int c = a * nrec + field;
    const float x = in[((n * (size_t)(C / CB) + (size_t)(c / CB)) * H + oh) * (size_t)W * CB + (size_t)ow * CB + (c % CB)];
    float r;
    if (field == 2) r = expf(x) * anchors.w[a];
    else if (field == 3) r = expf(x) * anchors.h[a];
    else
    {
        r = (float)(1.0 / (1.0 + (double)expf(-x)));
        if (field == 0) r = stride * (r + (float)ow);
        else if (field == 1) r = stride * (r + (float)oh);
    }
    out[i] = r;
}

// concat: per image two contiguous copies, 16-byte granules
__global__ __launch_bounds__(TPB) void concat_kernel(const uint4 *__restrict__ in0,
                                                     const uint4 *__restrict__ in1,
                                                     uint4 *__restrict__ out, size_t v0, size_t v1,
                                                     size_t total)
{
    const size_t base = (size_t)blockIdx.x * (TPB * UNROLL) + threadIdx.x;
    const size_t per = v0 + v1;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
    {
        const size_t i = base + (size_t)u * TPB;
        if (i < total)
        {
            const size_t n = i / per, r = i % per;
            out[i] = (r < v0) ? in0[n * v0 + r] : in1[n * v1 + (r - v0)];
        }
    }
}

// uint8 ReLU / Accum: 16 bytes per lane and access
template <bool ACCUM>
__global__ __launch_bounds__(TPB) void ew_u8_kernel(const uint4 *in, uint4 *out, size_t n16,
                                                    int32_t zi, int32_t zo, QOut q)
{
    const size_t base = (size_t)blockIdx.x * (TPB * UNROLL) + threadIdx.x;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
    {
        const size_t i = base + (size_t)u * TPB;
        if (i < n16)
        {
            const uint4 x = in[i];
            uint4 o = ACCUM ? out[i] : make_uint4(0, 0, 0, 0);
            const uint32_t xs[4] = {x.x, x.y, x.z, x.w};
            const uint32_t os[4] = {o.x, o.y, o.z, o.w};
            uint32_t rs[4];
#pragma unroll
            for (int w = 0; w < 4; ++w)
            {
                uint32_t packed = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b)
                {
                    int32_t v = (int32_t)((xs[w] >> (8 * b)) & 0xffu) + zi;
                    if (ACCUM) v = (int32_t)((uint32_t)v + ((os[w] >> (8 * b)) & 0xffu) + (uint32_t)zo);
                    else v = v > 0 ? v : 0;
                    packed |= requant_u8(v, q) << (8 * b);
                }
                rs[w] = packed;
            }
            out[i] = make_uint4(rs[0], rs[1], rs[2], rs[3]);
        }
    }
}

// SoftMax over the whole tensor of an image: out = exp(in) * float(1 / sum(exp(in))), no maximum
// subtracted (interface_abstract.hpp:1778-1832).  One workgroup per image: pass 1 writes exp(in) and
// reduces the sum (per lane, then wave shuffles, then LDS), pass 2 scales what pass 1 wrote (it is
// still in cache for the class-score sized tensors this layer sees).  In place is allowed.
__global__ __launch_bounds__(TPB) void softmax_f32_kernel(const float4 *in, float4 *out, size_t per4)
{
    __shared__ float part[TPB / WAVE];
    __shared__ float inv_s;
    const float4 *a = in + (size_t)blockIdx.x * per4;
    float4 *c = out + (size_t)blockIdx.x * per4;
    float sum = 0.f;
    for (size_t i = threadIdx.x; i < per4; i += TPB)
    {
        const float4 x = a[i];
        const float4 e = make_float4(expf(x.x), expf(x.y), expf(x.z), expf(x.w));
        c[i] = e;
        sum += (e.x + e.y) + (e.z + e.w);
    }
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, WAVE);
    if ((threadIdx.x & (WAVE - 1)) == 0) part[threadIdx.x / WAVE] = sum;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < TPB / WAVE; ++w) t += part[w];
        inv_s = (float)(1.0 / (double)t);
    }
    __syncthreads();
    const float inv = inv_s;
    for (size_t i = threadIdx.x; i < per4; i += TPB)
    {
        float4 e = c[i];
        e.x *= inv; e.y *= inv; e.z *= inv; e.w *= inv;
        c[i] = e;
    }
}

inline unsigned blocks_for(size_t nvec) { return (unsigned)((nvec + TPB * UNROLL - 1) / (TPB * UNROLL)); }

int check_act_args(const char *op, int batch, int C, int H, int W, const void *in, const void *out)
{
    if (C <= 0 || C % CB != 0) return SMALL_HIP_ECHANNELS;
    if (batch <= 0 || H <= 0 || W <= 0) { set_error("%s: non-positive size", op); return SMALL_HIP_EINVAL; }
    if (!in || !out || !aligned16(in) || !aligned16(out)) { set_error("%s: null or misaligned pointer", op); return SMALL_HIP_EINVAL; }
    return SMALL_HIP_OK;
}

template <int OP>
int launch_ew(const char *op, int batch, int C, int H, int W, const float *in, float *out, float slope,
              small_hip_stream_t stream)
{
    if (int rc = check_act_args(op, batch, C, H, W, in, out)) return rc;
    const size_t n4 = (size_t)batch * C * H * W / 4;
    hipLaunchKernelGGL(ew_f32_kernel<OP>, dim3(blocks_for(n4)), dim3(TPB), 0, as_stream(stream),
                       reinterpret_cast<const float4 *>(in), reinterpret_cast<float4 *>(out), n4, slope);
    SHP_LAUNCH_CHECK(op);
    return SMALL_HIP_OK;
}

} // namespace

extern "C" {

int small_hip_relu_f32(int batch, int C, int H, int W, const float *in, float *out,
                       small_hip_stream_t stream)
{
    return launch_ew<EW_RELU>("small_hip_relu_f32", batch, C, H, W, in, out, 0.f, stream);
}

int small_hip_leaky_relu_f32(int batch, int C, int H, int W, const float *in, float slope, float *out,
                             small_hip_stream_t stream)
{
    return launch_ew<EW_LEAKY>("small_hip_leaky_relu_f32", batch, C, H, W, in, out, slope, stream);
}

int small_hip_dropout_f32(int batch, int C, int H, int W, const float *in, float scale, float *out,
                          small_hip_stream_t stream)
{
    return launch_ew<EW_SCALE>("small_hip_dropout_f32", batch, C, H, W, in, out, scale, stream);
}

int small_hip_softmax_f32(int batch, int C, int H, int W, const float *in, float *out, small_hip_stream_t stream)
{
    if (int rc = check_act_args("small_hip_softmax_f32", batch, C, H, W, in, out)) return rc;
    const size_t per4 = (size_t)C * H * W / 4;
    hipLaunchKernelGGL(softmax_f32_kernel, dim3((unsigned)batch), dim3(TPB), 0, as_stream(stream),
                       reinterpret_cast<const float4 *>(in), reinterpret_cast<float4 *>(out), per4);
    SHP_LAUNCH_CHECK("small_hip_softmax_f32");
    return SMALL_HIP_OK;
}

int small_hip_accum_f32(int batch, int C, int H, int W, const float *in, float *out,
                        small_hip_stream_t stream)
{
    return launch_ew<EW_ACCUM>("small_hip_accum_f32", batch, C, H, W, in, out, 0.f, stream);
}

static int bias_impl(bool acc, int batch, int C, int H, int W, const float *bias, float *out,
                     small_hip_stream_t stream)
{
    if (int rc = check_act_args("small_hip_bias_f32", batch, C, H, W, bias, out)) return rc;
    const size_t n4 = (size_t)batch * C * H * W / 4;
    auto k = acc ? bias_f32_kernel<true> : bias_f32_kernel<false>;
    hipLaunchKernelGGL(k, dim3(blocks_for(n4)), dim3(TPB), 0, as_stream(stream),
                       reinterpret_cast<const float4 *>(bias), reinterpret_cast<float4 *>(out), n4,
                       H * W, C / CB);
    SHP_LAUNCH_CHECK("small_hip_bias_f32");
    return SMALL_HIP_OK;
}

int small_hip_bias_f32(int batch, int C, int H, int W, const float *bias, float *out,
                       small_hip_stream_t stream)
{
    return bias_impl(false, batch, C, H, W, bias, out, stream);
}

int small_hip_partial_bias_f32(int batch, int C, int H, int W, const float *bias, float *out,
                               small_hip_stream_t stream)
{
    return bias_impl(true, batch, C, H, W, bias, out, stream);
}

static int upsample_impl(const char *name, int hshift, int batch, int scale, int C, int H, int W, const float *in,
                         float *out, small_hip_stream_t stream);

int small_hip_upsample2d_f32(int batch, int scale, int C, int H, int W, const float *in, float *out,
                             small_hip_stream_t stream)
{
    return upsample_impl("small_hip_upsample2d_f32", 1, batch, scale, C, H, W, in, out, stream);
}

int small_hip_upsample1d_f32(int batch, int scale, int C, int rows, int W, const float *in, float *out,
                             small_hip_stream_t stream)
{
    return upsample_impl("small_hip_upsample1d_f32", 0, batch, scale, C, rows, W, in, out, stream);
}

static int upsample_impl(const char *name, int hshift, int batch, int scale, int C, int H, int W, const float *in,
                         float *out, small_hip_stream_t stream)
{
    // interface_abstract.hpp:1858-1886: scale 1 copies whatever the channel count is, scale 2
    // checks the channel count, anything else is a scale error
    if (scale == 1)
    {
        if (batch <= 0 || C <= 0 || H <= 0 || W <= 0 || !in || !out) { set_error("%s: bad argument", name); return SMALL_HIP_EINVAL; }
        if (in != out)
            SHP_HIP(hipMemcpyAsync(out, in, (size_t)batch * C * H * W * sizeof(float),
                                   hipMemcpyDeviceToDevice, as_stream(stream)));
        return SMALL_HIP_OK;
    }
    if (scale != 2) return SMALL_HIP_ESCALE;
    if (int rc = check_act_args(name, batch, C, H, W, in, out)) return rc;
    if (in == out) { set_error("%s: in-place upsampling is not possible", name); return SMALL_HIP_EINVAL; }
    const size_t n4 = ((size_t)batch * C * H * W) << hshift >> 1;  // 2x or 4x the elements, /4 per vector
    hipLaunchKernelGGL(upsample2_f32_kernel, dim3(blocks_for(n4)), dim3(TPB), 0, as_stream(stream),
                       reinterpret_cast<const float4 *>(in), reinterpret_cast<float4 *>(out), n4, H, W, hshift);
    SHP_LAUNCH_CHECK(name);
    return SMALL_HIP_OK;
}

int small_hip_yolo_decode_f32(int batch, int padded_channels, int H, int W, int num_anchors,
                              const uint32_t *anchors_wh, int num_classes, int image_size, const float *in,
                              float *out, small_hip_stream_t stream)
{
    const char *name = "small_hip_yolo_decode_f32";
    if (int rc = check_act_args(name, batch, padded_channels, H, W, in, out)) return rc;
    if (num_anchors <= 0 || num_anchors > 8 || num_classes < 0 || !anchors_wh || image_size < H)
    {
        set_error("%s: 1..8 anchors, a class count >= 0 and an image at least as high as the map are needed", name);
        return SMALL_HIP_EINVAL;
    }
    const int nrec = num_classes + 5;
    if ((long)num_anchors * nrec > padded_channels)
    {
        set_error("%s: %d anchors x %d fields do not fit %d channels", name, num_anchors, nrec, padded_channels);
        return SMALL_HIP_EINVAL;
    }
    if (in == out) { set_error("%s: in-place decode is not possible", name); return SMALL_HIP_EINVAL; }
    YoloAnchors an{};
    for (int a = 0; a < num_anchors; ++a) { an.w[a] = (float)anchors_wh[2 * a]; an.h[a] = (float)anchors_wh[2 * a + 1]; }
    const size_t n_out = (size_t)batch * num_anchors * H * W * nrec;
    hipLaunchKernelGGL(yolo_decode_f32_kernel, dim3((unsigned)((n_out + TPB - 1) / TPB)), dim3(TPB), 0, as_stream(stream),
                       in, out, n_out, padded_channels, H, W, num_anchors, nrec, (float)(image_size / H), an);
    SHP_LAUNCH_CHECK(name);
    return SMALL_HIP_OK;
}

int small_hip_concat(int batch, uint32_t C0, uint32_t C1, uint32_t H, uint32_t W, const void *in0,
                     const void *in1, void *out, size_t esize, small_hip_stream_t stream)
{
    if (batch <= 0 || !in0 || !in1 || !out || (esize != 1 && esize != 4))
        return einval("small_hip_concat: bad argument");
    const size_t b0 = (size_t)C0 * H * W * esize, b1 = (size_t)C1 * H * W * esize;
    if (b0 + b1 == 0) return SMALL_HIP_OK;
    if (b0 % 16 || b1 % 16 || !aligned16(in0) || !aligned16(in1) || !aligned16(out))
    {
        // odd sizes: plain copies, image by image (the reference does two std::copy calls)
        for (int n = 0; n < batch; ++n)
        {
            char *o = static_cast<char *>(out) + (size_t)n * (b0 + b1);
            if (b0) SHP_HIP(hipMemcpyAsync(o, static_cast<const char *>(in0) + (size_t)n * b0, b0, hipMemcpyDeviceToDevice, as_stream(stream)));
            if (b1) SHP_HIP(hipMemcpyAsync(o + b0, static_cast<const char *>(in1) + (size_t)n * b1, b1, hipMemcpyDeviceToDevice, as_stream(stream)));
        }
        return SMALL_HIP_OK;
    }
    const size_t v0 = b0 / 16, v1 = b1 / 16, total = (v0 + v1) * (size_t)batch;
    hipLaunchKernelGGL(concat_kernel, dim3(blocks_for(total)), dim3(TPB), 0, as_stream(stream),
                       static_cast<const uint4 *>(in0), static_cast<const uint4 *>(in1),
                       static_cast<uint4 *>(out), v0, v1, total);
    SHP_LAUNCH_CHECK("small_hip_concat");
    return SMALL_HIP_OK;
}

int small_hip_relu_u8(int batch, int C, int H, int W, const uint8_t *in, const small_hip_quant *iq,
                      uint8_t *out, const small_hip_quant *oq, small_hip_stream_t stream)
{
    if (!iq || !oq) return einval("small_hip_relu_u8: null quantisation parameters");
    if (int rc = check_act_args("small_hip_relu_u8", batch, C, H, W, in, out)) return rc;
    const size_t n16 = (size_t)batch * C * H * W / 16;
    const QOut q = make_qout(oq->multiplier, oq->lshift, oq->rshift);
    hipLaunchKernelGGL(ew_u8_kernel<false>, dim3(blocks_for(n16)), dim3(TPB), 0, as_stream(stream),
                       reinterpret_cast<const uint4 *>(in), reinterpret_cast<uint4 *>(out), n16,
                       iq->zero, 0, q);
    SHP_LAUNCH_CHECK("small_hip_relu_u8");
    return SMALL_HIP_OK;
}

int small_hip_accum_u8(int batch, int C, int H, int W, const uint8_t *in, const small_hip_quant *iq,
                       uint8_t *out, const small_hip_quant *oq, small_hip_stream_t stream)
{
    if (!iq || !oq) return einval("small_hip_accum_u8: null quantisation parameters");
    if (int rc = check_act_args("small_hip_accum_u8", batch, C, H, W, in, out)) return rc;
    const size_t n16 = (size_t)batch * C * H * W / 16;
    const QOut q = make_qout(oq->multiplier, oq->lshift, oq->rshift);
    hipLaunchKernelGGL(ew_u8_kernel<true>, dim3(blocks_for(n16)), dim3(TPB), 0, as_stream(stream),
                       reinterpret_cast<const uint4 *>(in), reinterpret_cast<uint4 *>(out), n16,
                       iq->zero, oq->zero, q);
    SHP_LAUNCH_CHECK("small_hip_accum_u8");
    return SMALL_HIP_OK;
}

} // extern "C"
