/* TEST INFRASTRUCTURE ONLY -- see small_oracle.h.
 *
 * CPU restatement of the SMaLL layer hot path, written from the semantics of
 * the reference (paths relative to the reference tree):
 *
 *   shapes      include/small/utils.hpp:43-64 (calc_padding), :159-165 (output_dim)
 *   index maps  include/small/buffers.hpp:33-79, 83-120, 138-263, 287-394
 *   loop nest   include/small/abstract_layer.hpp:1358-1823 (+ kernel*: 193-1352)
 *   dispatch    include/small/interface_abstract.hpp (per-op stride / channel checks)
 *   quantised   include/small/q_abstract_layer.hpp:894-1567,
 *               include/small/platforms/reference/intrinsics_quint8.h:191-310, 481-531
 *
 * Pinning status (what each function has been checked against; the checks live
 * in tests/):
 *   so_calc_padding, so_output_dim, so_packed_*_index, so_pack, so_unpack
 *        reference build (every index of several shapes), closed-form cases
 *   so_conv2d_f32, so_dwconv2d_f32 (<= 1 padded output row/col per side)
 *        reference regression fixtures (PyTorch generated), REF and ZEN2 builds of the
 *        reference on seeded inputs, float64 brute force, 1x1 case against a plain matmul
 *   so_conv2d_f32 with >= 2 padded output rows/cols on a side (e.g. 10x4 stride 2 "same")
 *        float64 brute-force zero-padded convolution and a library float64 conv2d on every row
 *        (tests/test_oracle_pins.py); the reference's scalar build, bit-identical, on the rows
 *        its edge code handles (rows 2..21 of the 10x4 stem): elsewhere its edge code is not
 *        usable (abstract_layer.hpp:1269-1349), so this is the textbook result
 *   so_maxpool2d_f32 (incl. "padding counts as 0" quirk), so_avgpool2d_f32 (count_include_pad)
 *        reference fixtures, REF/ZEN2 builds with negative inputs on padded borders
 *   so_relu_f32, so_leaky_relu_f32, so_accum_f32, so_bias_f32, so_upsample2d_f32, so_upsample1d_f32, so_concat
 *        closed forms (exact), reference fixtures (relu), REF/ZEN2 builds
 *   so_dropout_f32, so_softmax_f32   REF/ZEN2 builds (dropout exact; softmax within 1e-6 relative:
 *        the reduction order of the global sum differs), closed form sum(out) == 1
 *   so_dense_f32   REF build's Conv2D on a 1x1 image, plain matmul
 *   so_dense_literal_f32   REF build's small::Dense
 *   so_requant, so_conv2d_u8, so_dwconv2d_u8, so_maxpool2d_u8, so_relu_u8, so_dense_u8
 *        REF build (bit exact) on seeded inputs with positive and negative zero points;
 *        RNDRSHIFT/VQRDMULH against brute force on small ranges
 *   so_avgpool2d_u8   the reference has no uint8 AveragePool2D (interface_abstract.hpp:983); the
 *        definition here is a depthwise convolution with a filter of ones and filter zero point 0,
 *        and is pinned as such: bit-identical to the REF build's DepthwiseConv2D<QUInt8Buffer> on
 *        that filter, to so_dwconv2d_u8, and to int64 window sums (tests/test_oracle_pins.py)
 *   so_accum_u8   the reference has no uint8 Accum (interface_abstract.hpp:1981); the definition
 *        here equals a two-input-channel 1x1 Conv2D<QUInt8Buffer> with a filter of ones, and is
 *        pinned as such against the REF build over all 256 x 256 byte pairs (zI == zO; the
 *        reachable pairs otherwise) and against an evaluation in unbounded integers
 *   uint8 functions at channel block 16: equal to channel block 1 (what REF pins) after unpacking
 *   so_conv2d_bias_act_f32   equals the reference's Bias + PartialConv2D + activation sequence
 *        (Conv2DLayer.hpp:827-879), which the REF build pins
 *   quantised 1-D forms (the 2-D functions on a 1 x k window): PARITY UNPINNED as 1-D calls; the
 *        reference's quantised 1-D functions write unrelated bytes on its scalar build
 */
#include "small_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------- */
/* shapes: utils.hpp:43-64, 159-165                                           */
/* ------------------------------------------------------------------------- */
void so_calc_padding(size_t I_dim, uint32_t K_dim, uint32_t stride, uint8_t *front, uint8_t *back)
{
    uint32_t padding;
    size_t rem = I_dim % stride;
    if (rem == 0)
        padding = (K_dim > stride) ? K_dim - stride : 0;
    else
        padding = (K_dim > rem) ? (uint32_t)(K_dim - rem) : 0;
    *front = (uint8_t)(padding / 2);
    *back = (uint8_t)(padding - padding / 2);
}

uint32_t so_output_dim(uint32_t in_dim, uint32_t stride, uint32_t k_dim)
{
    /* "valid" output count; 0 when the kernel does not fit */
    if (k_dim > in_dim || stride == 0) return 0;
    return (in_dim - k_dim) / stride + 1;
}

/* ------------------------------------------------------------------------- */
/* index maps: buffers.hpp:33-120                                             */
/* ------------------------------------------------------------------------- */
static int eff_block(uint32_t C, uint32_t cb, uint32_t *out)
{
    if (C < cb)
    {
        if (C == 1 || C == 2 || C == 3) { *out = C; return 0; }
        return -1;
    }
    if (C % cb != 0) return -1;
    *out = cb;
    return 0;
}

long so_packed_weight_index(uint32_t Co, uint32_t Ci, uint32_t Fh, uint32_t Fw, uint32_t cob,
                            uint32_t cib, size_t o, size_t c, size_t h, size_t w)
{
    (void)Co;
    uint32_t ib;
    if (eff_block(Ci, cib, &ib)) return -1;
    size_t blk = (size_t)Fh * Fw * ib * cob;
    return (long)((o / cob) * ((size_t)(Ci / ib) * blk) + (c / ib) * blk +
                  h * ((size_t)Fw * ib * cob) + w * ((size_t)ib * cob) + (c % ib) * cob +
                  (o % cob));
}

long so_packed_buffer_index(uint32_t C, uint32_t H, uint32_t W, uint32_t cb, size_t c, size_t h,
                            size_t w)
{
    uint32_t b;
    if (eff_block(C, cb, &b)) return -1;
    return (long)((c / b) * ((size_t)H * W * b) + h * ((size_t)W * b) + w * b + (c % b));
}

/* buffers.hpp:138-263 / 287-394: flat [d0][d1][d2][d3] (OIHW or 1CHW) <-> packed */
static long pack_generic(const uint8_t *src, uint8_t *dst, int type, uint32_t Co, uint32_t Ci,
                         uint32_t H, uint32_t W, uint32_t cib, uint32_t cob, size_t es, int unpack)
{
    uint32_t ipb, opb;
    if (type == 4) { H = 1; W = 1; }
    if (type == 2) cib = 1;
    if ((type == 3 || type == 0) && Ci < cib)
    {
        if (!(Ci == 1 || Ci == 2 || Ci == 3)) return -1;
        cib = Ci;
    }
    if (type == 0) { ipb = cib; opb = 1; }
    else if (type == 1) { ipb = cob; opb = 1; }
    else if (type == 2 || type == 3 || type == 4) { ipb = cib; opb = cob; }
    else return -1;
    if (Ci % ipb != 0 || Co % opb != 0) return -1;

    size_t off = 0;
    for (uint32_t g = 0; g < Co; g += opb)
        for (uint32_t h = 0; h < Ci; h += ipb)
            for (uint32_t i = 0; i < H; i++)
                for (uint32_t j = 0; j < W; j++)
                    for (uint32_t k = 0; k < ipb; k++)
                        for (uint32_t l = 0; l < opb; l++)
                        {
                            size_t flat = ((size_t)(g + l) * Ci + (h + k)) * H * W + (size_t)i * W + j;
                            if (unpack)
                                memcpy(dst + flat * es, src + off * es, es);
                            else
                                memcpy(dst + off * es, src + flat * es, es);
                            off++;
                        }
    return (long)((size_t)Co * Ci * H * W);
}

long so_pack(const void *flat, int type, uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3,
             uint32_t cib, uint32_t cob, void *packed, size_t esize)
{
    return pack_generic((const uint8_t *)flat, (uint8_t *)packed, type, d0, d1, d2, d3, cib, cob,
                        esize, 0);
}

long so_unpack(const void *packed, int type, uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3,
               uint32_t cib, uint32_t cob, void *flat, size_t esize)
{
    return pack_generic((const uint8_t *)packed, (uint8_t *)flat, type, d0, d1, d2, d3, cib, cob,
                        esize, 1);
}

/* ------------------------------------------------------------------------- */
/* common window geometry                                                     */
/* ------------------------------------------------------------------------- */
typedef struct geom
{
    int Ho, Wo;
} geom;

static geom out_geom(int kh, int kw, int stride, int pt, int pb, int pl, int pr, int H, int W)
{
    geom g;
    g.Ho = (int)so_output_dim((uint32_t)(H + pt + pb), (uint32_t)stride, (uint32_t)kh);
    g.Wo = (int)so_output_dim((uint32_t)(W + pl + pr), (uint32_t)stride, (uint32_t)kw);
    return g;
}

/* conv channel rule: interface_abstract.hpp:70-220 */
static int conv_in_block(int Ci, int cb, int *cib)
{
    if (Ci <= 0) return SO_ECHANNELS;
    if (Ci % cb == 0) { *cib = cb; return 0; }
    if ((Ci == 3 || Ci == 2 || Ci == 1) && Ci < cb) { *cib = Ci; return 0; }
    return SO_ECHANNELS;
}

#define MAXCB 64

/* ------------------------------------------------------------------------- */
/* float conv: abstract_layer.hpp:491-575 (tile init, n/m/ii loop order),     */
/* :1630-1632 (first = rewrite && i == 0)                                     */
/* ------------------------------------------------------------------------- */
static int conv_f32_impl(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl,
                         int pr, int Co, int Ci, int H, int W, const float *in, const float *filt,
                         const float *bias, int act, float slope, float *out, int accumulate,
                         int acc64)
{
    int cib;
    int rc = conv_in_block(Ci, cb, &cib);
    if (rc) return rc;
    if (stride != 1 && stride != 2) return SO_ESTRIDE;
    if (cb > MAXCB || Co % cb != 0 || kh <= 0 || kw <= 0) return SO_EINVAL;
    geom g = out_geom(kh, kw, stride, pt, pb, pl, pr, H, W);
    const int Ho = g.Ho, Wo = g.Wo;
    const int nci = Ci / cib;
    const size_t in_img = (size_t)Ci * H * W, out_img = (size_t)Co * Ho * Wo;

    for (int n = 0; n < batch; n++)
    {
        const float *I = in + n * in_img;
        float *O = out + n * out_img;
        for (int kb = 0; kb < Co / cb; kb++)
        {
            const float *Fk = filt + (size_t)kb * nci * kh * kw * cib * cb;
            for (int oh = 0; oh < Ho; oh++)
                for (int ow = 0; ow < Wo; ow++)
                {
                    float *o = O + (((size_t)kb * Ho + oh) * Wo + ow) * cb;
                    float acc[MAXCB];
                    double dacc[MAXCB];
                    for (int j = 0; j < cb; j++)
                    {
                        float init = accumulate ? o[j] : (bias ? bias[kb * cb + j] : 0.0f);
                        acc[j] = init;
                        dacc[j] = init;
                    }
                    for (int ib = 0; ib < nci; ib++)
                        for (int a = 0; a < kh; a++)
                        {
                            int ih = oh * stride + a - pt;
                            if (ih < 0 || ih >= H) continue;
                            for (int b = 0; b < kw; b++)
                            {
                                int iw = ow * stride + b - pl;
                                if (iw < 0 || iw >= W) continue;
                                const float *ip = I + (((size_t)ib * H + ih) * W + iw) * cib;
                                const float *fp =
                                    Fk + ((((size_t)ib * kh + a) * kw + b) * cib) * cb;
                                for (int ii = 0; ii < cib; ii++)
                                {
                                    float av = ip[ii];
                                    const float *f = fp + (size_t)ii * cb;
                                    if (acc64)
                                        for (int j = 0; j < cb; j++) dacc[j] += (double)av * (double)f[j];
                                    else
                                        for (int j = 0; j < cb; j++)
                                        {
                                            float p = av * f[j];
                                            acc[j] = acc[j] + p;
                                        }
                                }
                            }
                        }
                    for (int j = 0; j < cb; j++)
                    {
                        float v = acc64 ? (float)dacc[j] : acc[j];
                        if (act == SO_ACT_RELU) v = (v > 0.0f) ? v : 0.0f;
                        else if (act == SO_ACT_LEAKY) v = (v > 0.0f) ? v : v * slope;
                        o[j] = v;
                    }
                }
        }
    }
    return SO_OK;
}

int so_conv2d_f32(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                  int Co, int Ci, int H, int W, const float *in, const float *filt, float *out,
                  int accumulate, int acc64)
{
    return conv_f32_impl(batch, cb, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, filt, NULL,
                         SO_ACT_NONE, 0.0f, out, accumulate, acc64);
}

int so_conv2d_bias_act_f32(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl,
                           int pr, int Co, int Ci, int H, int W, const float *in,
                           const float *filt, const float *bias, int act, float slope, float *out)
{
    return conv_f32_impl(batch, cb, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, filt, bias,
                         act, slope, out, 0, 0);
}

/* ------------------------------------------------------------------------- */
/* depthwise / pooling share one window walker.                               */
/* interface_abstract.hpp:778-834 (max), 910-978 (avg), 994-1051 (dw)         */
/* ------------------------------------------------------------------------- */
enum { W_DW, W_MAX, W_AVG };

static int window_f32(int op, int batch, int cb, int kh, int kw, int stride, int pt, int pb,
                      int pl, int pr, int C, int H, int W, const float *in, const float *filt,
                      float *out, int accumulate, int acc64)
{
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    if (op == W_AVG) { if (stride < 1 || stride > 3) return SO_ESTRIDE; }
    else if (stride != 1 && stride != 2) return SO_ESTRIDE;
    if (kh <= 0 || kw <= 0) return SO_EINVAL;
    geom g = out_geom(kh, kw, stride, pt, pb, pl, pr, H, W);
    const int Ho = g.Ho, Wo = g.Wo;
    /* abstract_layer.hpp:565-569: float norm = 1.0 / (1.0 * F_h * F_w) */
    const float norm = (float)(1.0 / (1.0 * kh * kw));
    for (int n = 0; n < batch; n++)
        for (int cbk = 0; cbk < C / cb; cbk++)
        {
            const float *I = in + ((size_t)n * (C / cb) + cbk) * H * W * cb;
            float *O = out + ((size_t)n * (C / cb) + cbk) * Ho * Wo * cb;
            const float *Fk = filt ? filt + (size_t)cbk * kh * kw * cb : NULL;
            for (int oh = 0; oh < Ho; oh++)
                for (int ow = 0; ow < Wo; ow++)
                    for (int j = 0; j < cb; j++)
                    {
                        float *o = O + ((size_t)oh * Wo + ow) * cb + j;
                        int all_valid = (oh * stride - pt >= 0) && (oh * stride - pt + kh <= H) &&
                                        (ow * stride - pl >= 0) && (ow * stride - pl + kw <= W);
                        float acc = 0.0f;
                        double dacc = 0.0;
                        if (op == W_DW && accumulate) { acc = *o; dacc = *o; }
                        /* abstract_layer.hpp:514-521: an un-padded max-pool window starts from
                         * its first input element; a padded one starts from the zeroed tile */
                        if (op == W_MAX && all_valid)
                            acc = I[((size_t)(oh * stride - pt) * W + (ow * stride - pl)) * cb + j];
                        for (int a = 0; a < kh; a++)
                        {
                            int ih = oh * stride + a - pt;
                            if (ih < 0 || ih >= H) continue;
                            for (int b = 0; b < kw; b++)
                            {
                                int iw = ow * stride + b - pl;
                                if (iw < 0 || iw >= W) continue;
                                float v = I[((size_t)ih * W + iw) * cb + j];
                                if (op == W_DW)
                                {
                                    float f = Fk[((size_t)a * kw + b) * cb + j];
                                    if (acc64) dacc += (double)v * (double)f;
                                    else { float p = v * f; acc = acc + p; }
                                }
                                else if (op == W_MAX) acc = (v > acc) ? v : acc;
                                else acc = acc + v;
                            }
                        }
                        if (op == W_AVG) acc = acc * norm;
                        if (op == W_DW && acc64) acc = (float)dacc;
                        *o = acc;
                    }
        }
    return SO_OK;
}

int so_dwconv2d_f32(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                    int C, int H, int W, const float *in, const float *filt, float *out,
                    int accumulate, int acc64)
{
    return window_f32(W_DW, batch, cb, kh, kw, stride, pt, pb, pl, pr, C, H, W, in, filt, out,
                      accumulate, acc64);
}

int so_maxpool2d_f32(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                     int C, int H, int W, const float *in, float *out)
{
    return window_f32(W_MAX, batch, cb, kh, kw, stride, pt, pb, pl, pr, C, H, W, in, NULL, out, 0,
                      0);
}

int so_avgpool2d_f32(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                     int C, int H, int W, const float *in, float *out)
{
    return window_f32(W_AVG, batch, cb, kh, kw, stride, pt, pb, pl, pr, C, H, W, in, NULL, out, 0,
                      0);
}

/* ------------------------------------------------------------------------- */
/* elementwise: interface_abstract.hpp:1541-1566, 1616-1646, 1950-1978,       */
/* 1992-2064, 1845-1889, 2072-2105                                            */
/* intrinsics_float.h:306-338 (c = a > c ? a : c), :423-457 (a > 0 ? a : a*s) */
/* ------------------------------------------------------------------------- */
int so_relu_f32(int batch, int cb, int C, int H, int W, const float *in, float *out)
{
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    size_t n = (size_t)batch * C * H * W;
    for (size_t i = 0; i < n; i++) { float v = in[i]; out[i] = (v > 0.0f) ? v : 0.0f; }
    return SO_OK;
}

int so_leaky_relu_f32(int batch, int cb, int C, int H, int W, const float *in, float slope,
                      float *out)
{
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    size_t n = (size_t)batch * C * H * W;
    for (size_t i = 0; i < n; i++) { float v = in[i]; out[i] = (v > 0.0f) ? v : v * slope; }
    return SO_OK;
}

/* Dropout at inference: c = a * filter[0] (abstract_layer.hpp:82-86 "drop_out_rate = b_cur[0]",
 * intrinsics_float.h:534-545 FLOAT_DIV_TILE_C multiplies), interface_abstract.hpp:1697-1726 */
int so_dropout_f32(int batch, int cb, int C, int H, int W, const float *in, float scale, float *out)
{
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    size_t n = (size_t)batch * C * H * W;
    for (size_t i = 0; i < n; i++) out[i] = in[i] * scale;
    return SO_OK;
}

/* SoftMax over the WHOLE tensor of an image (interface_abstract.hpp:1778-1832): element-wise exp
 * (intrinsics_float.h:671-686, std::exp on float, no maximum subtracted), one global sum of all
 * C*H*W values, then a multiplication by float(1.0 / sum) (the reciprocal is taken in double and
 * stored in a float buffer).  The sum here is accumulated in double and rounded to float once: the
 * reference adds floats in its tile order, which differs from this by float rounding only (about 1e-7
 * relative at class-score sizes, checked; it grows with the element count, so a float restatement in
 * any other order would be no closer to it). */
int so_softmax_f32(int batch, int cb, int C, int H, int W, const float *in, float *out)
{
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    size_t per = (size_t)C * H * W;
    for (int n = 0; n < batch; n++)
    {
        const float *a = in + (size_t)n * per;
        float *c = out + (size_t)n * per;
        double sum = 0.0;
        for (size_t i = 0; i < per; i++) { c[i] = expf(a[i]); sum += (double)c[i]; }
        const float inv = (float)(1.0 / (double)(float)sum);
        for (size_t i = 0; i < per; i++) c[i] *= inv;
    }
    return SO_OK;
}

int so_accum_f32(int batch, int cb, int C, int H, int W, const float *in, float *out)
{
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    size_t n = (size_t)batch * C * H * W;
    for (size_t i = 0; i < n; i++) out[i] = out[i] + in[i];
    return SO_OK;
}

int so_bias_f32(int batch, int cb, int C, int H, int W, const float *bias, float *out,
                int accumulate)
{
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    for (int n = 0; n < batch; n++)
        for (int k = 0; k < C / cb; k++)
            for (size_t p = 0; p < (size_t)H * W; p++)
                for (int j = 0; j < cb; j++)
                {
                    float *o = out + (((size_t)n * (C / cb) + k) * H * W + p) * cb + j;
                    *o = accumulate ? (*o + bias[k * cb + j]) : bias[k * cb + j];
                }
    return SO_OK;
}

int so_upsample2d_f32(int batch, int cb, int scale, int C, int H, int W, const float *in,
                      float *out)
{
    if (scale == 1)
    {
        memmove(out, in, (size_t)batch * C * H * W * sizeof(float));
        return SO_OK;
    }
    if (scale != 2) return SO_ESCALE;
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    const int Ho = H * 2, Wo = W * 2;
    for (int n = 0; n < batch; n++)
        for (int k = 0; k < C / cb; k++)
        {
            const float *I = in + ((size_t)n * (C / cb) + k) * H * W * cb;
            float *O = out + ((size_t)n * (C / cb) + k) * Ho * Wo * cb;
            for (int i = 0; i < Ho; i++)
                for (int j = 0; j < Wo; j++)
                    for (int c = 0; c < cb; c++)
                        O[((size_t)i * Wo + j) * cb + c] = I[((size_t)(i / 2) * W + (j / 2)) * cb + c];
        }
    return SO_OK;
}

/* YOLOLayer::compute_output (YOLOLayer.hpp:150-222; sigmoid :21-24 is evaluated in double around a float exp) */
int so_yolo_decode_f32(int batch, int cb, int C, int H, int W, int num_anchors, const uint32_t *anchors_wh,
                       int num_classes, int image_size, const float *in, float *out)
{
    const int nrec = num_classes + 5;
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    if (num_anchors * nrec > C) return SO_EINVAL;
    const float stride = (float)(image_size / H);
    size_t o = 0;
    for (int n = 0; n < batch; n++)
        for (int a = 0; a < num_anchors; a++)
            for (int i = 0; i < H; i++)
                for (int j = 0; j < W; j++)
                    for (int f = 0; f < nrec; f++)
                    {
                        const int c = a * nrec + f;
                        const float x = in[((((size_t)n * (C / cb) + c / cb) * H + i) * W + j) * cb + c % cb];
                        float r;
                        if (f == 2) r = expf(x) * (float)anchors_wh[2 * a];
                        else if (f == 3) r = expf(x) * (float)anchors_wh[2 * a + 1];
                        else
                        {
                            r = (float)(1.0 / (1.0 + expf(-x)));
                            if (f == 0) r = stride * (r + (float)j);
                            else if (f == 1) r = stride * (r + (float)i);
                        }
                        out[o++] = r;
                    }
    return SO_OK;
}

/* UpSample1D (interface_abstract_1D.hpp:1614-1655): x2 along the width only; rows = its batch_size argument */
int so_upsample1d_f32(int batch, int cb, int scale, int C, int rows, int W, const float *in, float *out)
{
    if (scale == 1)
    {
        memmove(out, in, (size_t)batch * C * rows * W * sizeof(float));
        return SO_OK;
    }
    if (scale != 2) return SO_ESCALE;
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    const size_t planes = (size_t)batch * (C / cb) * rows;
    for (size_t p = 0; p < planes; p++)
        for (int j = 0; j < 2 * W; j++)
            for (int c = 0; c < cb; c++)
                out[(p * 2 * W + j) * cb + c] = in[(p * W + j / 2) * cb + c];
    return SO_OK;
}

int so_concat(int batch, uint32_t C0, uint32_t C1, uint32_t H, uint32_t W, const void *in0,
              const void *in1, void *out, size_t esize)
{
    size_t s0 = (size_t)C0 * H * W * esize, s1 = (size_t)C1 * H * W * esize;
    for (int n = 0; n < batch; n++)
    {
        memcpy((uint8_t *)out + n * (s0 + s1), (const uint8_t *)in0 + n * s0, s0);
        memcpy((uint8_t *)out + n * (s0 + s1) + s0, (const uint8_t *)in1 + n * s1, s1);
    }
    return SO_OK;
}

int so_dense_f32(int batch, int cb, int No, int Ni, const float *in, const float *filt, float *out)
{
    return so_conv2d_f32(batch, cb, 1, 1, 1, 0, 0, 0, 0, No, Ni, 1, 1, in, filt, out, 0, 0);
}

/* interface_abstract.hpp:2113-2132: a 1x1 depthwise over a 1 x Ni image with No channels */
int so_dense_literal_f32(int cb, int No, int Ni, const float *in, const float *filt, float *out)
{
    return so_dwconv2d_f32(1, cb, 1, 1, 1, 0, 0, 0, 0, No, 1, Ni, in, filt, out, 0, 0);
}

/* ------------------------------------------------------------------------- */
/* quantised uint8                                                            */
/* intrinsics_quint8.h:481-497 (VQRDMULH, RNDRSHIFT), :500-531 (quantize+clamp)*/
/* ------------------------------------------------------------------------- */
uint8_t so_requant(int32_t acc, const so_quant *oq)
{
    /* val * (1 << lshift) in 32-bit wrap-around arithmetic, then widened */
    int32_t shifted = (int32_t)((uint32_t)acc * ((uint32_t)1 << (oq->lshift & 31)));
    int64_t a = (int64_t)shifted;
    int64_t b = (int64_t)oq->multiplier;
    int overflow = (a == b) && (a == -2147483648LL);
    int64_t prod = a * b;
    int64_t nudge = prod >= 0 ? (1 << 30) : (1 - (1 << 30));
    int32_t v = overflow ? 2147483647 : (int32_t)((prod + nudge) / (1LL << 31)); /* truncating */
    int rs = oq->rshift;
    int32_t mask = (int32_t)((1LL << rs) - 1);
    int32_t mod = v & mask;
    int32_t threshold = (mask >> 1) + ((v < 0) ? -1 : 0);
    /* "one" is ~0 in the reference, so the rounding term is -1, not +1 */
    int32_t r = (v >> rs) + ((mod > threshold) ? -1 : 0);
    return (uint8_t)(r > 0 ? (r < 255 ? r : 255) : 0);
}

static int conv_u8_impl(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl,
                        int pr, int Co, int Ci, int H, int W, const uint8_t *in, int32_t zi,
                        const uint8_t *filt, int32_t zf, uint8_t *out, const so_quant *oq)
{
    int cib;
    int rc = conv_in_block(Ci, cb, &cib);
    if (rc) return rc;
    if (stride != 1 && stride != 2) return SO_ESTRIDE;
    if (cb > MAXCB || Co % cb != 0 || kh <= 0 || kw <= 0) return SO_EINVAL;
    geom g = out_geom(kh, kw, stride, pt, pb, pl, pr, H, W);
    const int Ho = g.Ho, Wo = g.Wo;
    const int nci = Ci / cib;
    for (int n = 0; n < batch; n++)
    {
        const uint8_t *I = in + (size_t)n * Ci * H * W;
        uint8_t *O = out + (size_t)n * Co * Ho * Wo;
        for (int kb = 0; kb < Co / cb; kb++)
        {
            const uint8_t *Fk = filt + (size_t)kb * nci * kh * kw * cib * cb;
            for (int oh = 0; oh < Ho; oh++)
                for (int ow = 0; ow < Wo; ow++)
                {
                    uint32_t acc[MAXCB];
                    for (int j = 0; j < cb; j++) acc[j] = 0;
                    for (int ib = 0; ib < nci; ib++)
                        for (int a = 0; a < kh; a++)
                        {
                            int ih = oh * stride + a - pt;
                            if (ih < 0 || ih >= H) continue;
                            for (int b = 0; b < kw; b++)
                            {
                                int iw = ow * stride + b - pl;
                                if (iw < 0 || iw >= W) continue;
                                const uint8_t *ip = I + (((size_t)ib * H + ih) * W + iw) * cib;
                                const uint8_t *fp =
                                    Fk + ((((size_t)ib * kh + a) * kw + b) * cib) * cb;
                                for (int ii = 0; ii < cib; ii++)
                                {
                                    uint32_t av = (uint32_t)((int32_t)ip[ii] + zi);
                                    for (int j = 0; j < cb; j++)
                                        acc[j] += av * (uint32_t)((int32_t)fp[ii * cb + j] + zf);
                                }
                            }
                        }
                    uint8_t *o = O + (((size_t)kb * Ho + oh) * Wo + ow) * cb;
                    for (int j = 0; j < cb; j++) o[j] = so_requant((int32_t)acc[j], oq);
                }
        }
    }
    return SO_OK;
}

int so_conv2d_u8(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                 int Co, int Ci, int H, int W, const uint8_t *in, const so_quant *iq,
                 const uint8_t *filt, const so_quant *fq, uint8_t *out, const so_quant *oq)
{
    return conv_u8_impl(batch, cb, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, iq->zero,
                        filt, fq->zero, out, oq);
}

int so_dense_u8(int batch, int cb, int No, int Ni, const uint8_t *in, const so_quant *iq,
                const uint8_t *filt, const so_quant *fq, uint8_t *out, const so_quant *oq)
{
    return conv_u8_impl(batch, cb, 1, 1, 1, 0, 0, 0, 0, No, Ni, 1, 1, in, iq->zero, filt,
                        fq->zero, out, oq);
}

enum { Q_DW, Q_MAX, Q_AVG };

static int window_u8(int op, int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl,
                     int pr, int C, int H, int W, const uint8_t *in, int32_t zi,
                     const uint8_t *filt, int32_t zf, uint8_t *out, const so_quant *oq)
{
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    if (op == Q_AVG) { if (stride < 1 || stride > 3) return SO_ESTRIDE; }
    else if (stride != 1 && stride != 2) return SO_ESTRIDE;
    if (kh <= 0 || kw <= 0) return SO_EINVAL;
    geom g = out_geom(kh, kw, stride, pt, pb, pl, pr, H, W);
    const int Ho = g.Ho, Wo = g.Wo;
    for (int n = 0; n < batch; n++)
        for (int k = 0; k < C / cb; k++)
        {
            const uint8_t *I = in + ((size_t)n * (C / cb) + k) * H * W * cb;
            uint8_t *O = out + ((size_t)n * (C / cb) + k) * Ho * Wo * cb;
            const uint8_t *Fk = filt ? filt + (size_t)k * kh * kw * cb : NULL;
            for (int oh = 0; oh < Ho; oh++)
                for (int ow = 0; ow < Wo; ow++)
                    for (int j = 0; j < cb; j++)
                    {
                        int all_valid = (oh * stride - pt >= 0) && (oh * stride - pt + kh <= H) &&
                                        (ow * stride - pl >= 0) && (ow * stride - pl + kw <= W);
                        int32_t acc = 0;
                        /* q_abstract_layer.hpp:286-293: un-padded max windows start from the
                         * first RAW input byte (no zero point added) */
                        if (op == Q_MAX && all_valid)
                            acc = I[((size_t)(oh * stride - pt) * W + (ow * stride - pl)) * cb + j];
                        for (int a = 0; a < kh; a++)
                        {
                            int ih = oh * stride + a - pt;
                            if (ih < 0 || ih >= H) continue;
                            for (int b = 0; b < kw; b++)
                            {
                                int iw = ow * stride + b - pl;
                                if (iw < 0 || iw >= W) continue;
                                int32_t v = (int32_t)I[((size_t)ih * W + iw) * cb + j] + zi;
                                if (op == Q_DW)
                                    acc = (int32_t)((uint32_t)acc +
                                                    (uint32_t)v * (uint32_t)((int32_t)Fk[((size_t)a * kw + b) * cb + j] + zf));
                                else if (op == Q_MAX) acc = (v > acc) ? v : acc;
                                else acc = (int32_t)((uint32_t)acc + (uint32_t)v);
                            }
                        }
                        O[((size_t)oh * Wo + ow) * cb + j] = so_requant(acc, oq);
                    }
        }
    return SO_OK;
}

int so_dwconv2d_u8(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                   int C, int H, int W, const uint8_t *in, const so_quant *iq, const uint8_t *filt,
                   const so_quant *fq, uint8_t *out, const so_quant *oq)
{
    return window_u8(Q_DW, batch, cb, kh, kw, stride, pt, pb, pl, pr, C, H, W, in, iq->zero, filt,
                     fq->zero, out, oq);
}

int so_maxpool2d_u8(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                    int C, int H, int W, const uint8_t *in, const so_quant *iq, uint8_t *out,
                    const so_quant *oq)
{
    return window_u8(Q_MAX, batch, cb, kh, kw, stride, pt, pb, pl, pr, C, H, W, in, iq->zero, NULL,
                     0, out, oq);
}

/* No reference counterpart.  Sum of (x + zI) over the valid taps, requantised with the output
 * buffer's multiplier/shift (the caller folds 1/(kh*kw) into them) == the reference's quantised
 * depthwise convolution with a filter of ones and filter zero point 0, which pins it. */
int so_avgpool2d_u8(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                    int C, int H, int W, const uint8_t *in, const so_quant *iq, uint8_t *out,
                    const so_quant *oq)
{
    return window_u8(Q_AVG, batch, cb, kh, kw, stride, pt, pb, pl, pr, C, H, W, in, iq->zero, NULL,
                     0, out, oq);
}

/* q_abstract_layer.hpp:950 + intrinsics_quint8.h:219-237: max(x + zI, 0) then requantise */
int so_relu_u8(int batch, int cb, int C, int H, int W, const uint8_t *in, const so_quant *iq,
               uint8_t *out, const so_quant *oq)
{
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    size_t n = (size_t)batch * C * H * W;
    for (size_t i = 0; i < n; i++)
    {
        int32_t v = (int32_t)in[i] + iq->zero;
        out[i] = so_requant(v > 0 ? v : 0, oq);
    }
    return SO_OK;
}

/* No reference counterpart.  out = requant_out((in + zI) + (out + zO)) == the reference's quantised
 * Conv2D over two input channels with a 1x1 filter of ones, which pins it. */
int so_accum_u8(int batch, int cb, int C, int H, int W, const uint8_t *in, const so_quant *iq,
                uint8_t *out, const so_quant *oq)
{
    if (C <= 0 || C % cb != 0) return SO_ECHANNELS;
    size_t n = (size_t)batch * C * H * W;
    for (size_t i = 0; i < n; i++)
    {
        int32_t v = (int32_t)in[i] + iq->zero + (int32_t)out[i] + oq->zero;
        out[i] = so_requant(v, oq);
    }
    return SO_OK;
}
