// TEST INFRASTRUCTURE ONLY -- never linked into, loaded by or called from the
// shipped HIP library.
//
// Thin extern "C" shim around the *unmodified* SMaLL headers, which are
// compiled from where they lie (the include path is given on the compiler
// command line by build_ref.sh; no reference source is copied).  One shim
// source builds two shared objects:
//
//   -DUARCH_REF + platforms/reference  -> libsmall_ref_REF.so   (float + quint8,
//                                         C_ob = C_ib = 1, scalar C)
//   platforms/zen2 + -mavx2 -mfma      -> libsmall_ref_ZEN2.so  (float only,
//                                         C_ob = C_ib = 16, AVX2 micro-kernels)
//
// Buffers are handle based so that a timing loop can call a layer repeatedly
// without copying tensors: sref_*buf_new() returns an opaque small::FloatBuffer*
// / small::QUInt8Buffer*, sref_*buf_data() its host pointer.
//
// Every entry point returns 0 on success, 1 for std::invalid_argument,
// 2 for any other exception; sref_last_error() returns the message.

#include <cstring>
#include <string>
#include <stdexcept>
#include <limits>
#include <omp.h>

#include <small.h>
#include <small/Conv1DLayer.hpp>
#include <small/Conv2DLayer.hpp>
#include <small/PartialConv2DLayer.hpp>
#include <small/DepthwiseConv2DLayer.hpp>
#include <small/MaxPool2DLayer.hpp>
#include <small/AveragePool2DLayer.hpp>
#include <small/ReLULayer.hpp>
#include <small/LeakyReLULayer.hpp>
#include <small/UpSample2DLayer.hpp>
#include <small/AddLayer.hpp>
#include <small/RouteLayer.hpp>
#include <small/SoftMaxLayer.hpp>
#include <small/models/MobileNetTiny.hpp>
#include <small/models/Resnet8Tiny.hpp>
#include <small/models/DSCNNTiny.hpp>
#include <small/models/TinyYoloV2.hpp>
#include <small/models/Darknet.hpp>
#include <small/models/AutoencoderTiny.hpp>
#include <small/models/DSCNNSquareTiny.hpp>

#include <memory>
#include <vector>

namespace {
thread_local std::string g_err;

template <class Fn>
int guarded(Fn &&fn)
{
    try { fn(); return 0; }
    catch (std::invalid_argument const &e) { g_err = e.what(); return 1; }
    catch (std::exception const &e) { g_err = e.what(); return 2; }
    catch (...) { g_err = "unknown exception"; return 2; }
}
} // namespace

#if defined(SMALL_HAS_FLOAT_SUPPORT)
using FB = small::FloatBuffer;
#define F(h) (*static_cast<FB *>(h))
#endif
#if defined(SMALL_HAS_QUINT8_SUPPORT)
using QB = small::QUInt8Buffer;
#define Q(h) (*static_cast<QB *>(h))
#endif

extern "C" {

const char *sref_last_error(void) { return g_err.c_str(); }

// out[0..2] = float C_ob, C_ib, W_ob ; out[3..5] = quint8 C_ob, C_ib, W_ob (0 if absent)
void sref_params(int *out)
{
    for (int i = 0; i < 6; ++i) out[i] = 0;
#if defined(SMALL_HAS_FLOAT_SUPPORT)
    out[0] = FB::C_ob; out[1] = FB::C_ib; out[2] = FB::W_ob;
#endif
#if defined(SMALL_HAS_QUINT8_SUPPORT)
    out[3] = QB::C_ob; out[4] = QB::C_ib; out[5] = QB::W_ob;
#endif
}

// ---- shape helpers (small/utils.hpp) ---------------------------------------
void sref_calc_padding(size_t I_dim, uint32_t K_dim, uint16_t stride,
                       uint8_t *front, uint8_t *back)
{
    small::calc_padding(I_dim, K_dim, stride, *front, *back);
}

uint32_t sref_output_dim(uint32_t in_dim, uint32_t stride, uint32_t k_dim)
{
    return small::output_dim(in_dim, stride, k_dim);
}

// ---- index maps (small/buffers.hpp) ----------------------------------------
long sref_packed_weight_index(uint32_t Co, uint32_t Ci, uint32_t H, uint32_t W,
                              uint32_t cob, uint32_t cib,
                              size_t o, size_t c, size_t h, size_t w)
{
    try { return (long)small::packed_weight_index(Co, Ci, H, W, cob, cib, o, c, h, w); }
    catch (std::exception const &e) { g_err = e.what(); return -1; }
}

long sref_packed_buffer_index(uint32_t C, uint32_t H, uint32_t W, uint32_t cb,
                              size_t c, size_t h, size_t w)
{
    try { return (long)small::packed_buffer_index(C, H, W, cb, c, h, w); }
    catch (std::exception const &e) { g_err = e.what(); return -1; }
}

#if defined(SMALL_HAS_FLOAT_SUPPORT)
// type: 0 INPUT, 1 OUTPUT, 2 FILTER_DW, 3 FILTER_CONV, 4 FILTER_FC
uint32_t sref_pack_f32(const float *flat, int type, uint32_t d0, uint32_t d1,
                       uint32_t d2, uint32_t d3, uint32_t cib, uint32_t cob,
                       float *packed)
{
    return small::convert_tensor2dc<float>(flat, (small::BufferTypeEnum)type,
                                           d0, d1, d2, d3, cib, cob, packed);
}
uint32_t sref_unpack_f32(const float *packed, int type, uint32_t d0, uint32_t d1,
                         uint32_t d2, uint32_t d3, uint32_t cib, uint32_t cob,
                         float *flat)
{
    return small::convert_dc2tensor<float>(packed, (small::BufferTypeEnum)type,
                                           d0, d1, d2, d3, cib, cob, flat);
}

// ---- FloatBuffer handles ----------------------------------------------------
void *sref_fbuf_new(size_t n) { try { return new FB(n); } catch (...) { return nullptr; } }
void sref_fbuf_free(void *h) { delete static_cast<FB *>(h); }
float *sref_fbuf_data(void *h) { return F(h).data(); }
size_t sref_fbuf_size(void *h) { return F(h).size(); }

int sref_conv2d_f32(int kh, int kw, int s, int t, int b, int l, int r,
                    int Co, int Ci, int H, int W, void *in, void *filt, void *out)
{
    return guarded([&] { small::Conv2D(kh, kw, s, t, b, l, r, Co, Ci, H, W,
                                       F(in), F(filt), F(out)); });
}
int sref_partial_conv2d_f32(int kh, int kw, int s, int t, int b, int l, int r,
                            int Co, int Ci, int H, int W, void *in, void *filt, void *out)
{
    return guarded([&] { small::PartialConv2D(kh, kw, s, t, b, l, r, Co, Ci, H, W,
                                              F(in), F(filt), F(out)); });
}
// small::GroupConv2D / small::PartialGroupConv2D (interface_abstract.hpp:1265-1533); C = channels per group
int sref_group_conv2d_f32(int partial, int kh, int kw, int s, int G, int t, int b, int l, int r,
                          int C, int H, int W, void *in, void *filt, void *out)
{
    return guarded([&] {
        if (partial) small::PartialGroupConv2D(kh, kw, s, G, t, b, l, r, C, H, W, F(in), F(filt), F(out));
        else small::GroupConv2D(kh, kw, s, G, t, b, l, r, C, H, W, F(in), F(filt), F(out));
    });
}
int sref_dwconv2d_f32(int kh, int kw, int s, int t, int b, int l, int r,
                      int C, int H, int W, void *in, void *filt, void *out)
{
    return guarded([&] { small::DepthwiseConv2D(kh, kw, s, t, b, l, r, C, H, W,
                                                F(in), F(filt), F(out)); });
}
int sref_partial_dwconv2d_f32(int kh, int kw, int s, int t, int b, int l, int r,
                              int C, int H, int W, void *in, void *filt, void *out)
{
    return guarded([&] { small::PartialDepthwiseConv2D(kh, kw, s, t, b, l, r, C, H, W,
                                                       F(in), F(filt), F(out)); });
}
int sref_maxpool2d_f32(int kh, int kw, int s, int t, int b, int l, int r,
                       int C, int H, int W, void *in, void *out)
{
    return guarded([&] { small::MaxPool2D(kh, kw, s, t, b, l, r, C, H, W, F(in), F(out)); });
}
int sref_avgpool2d_f32(int kh, int kw, int s, int t, int b, int l, int r,
                       int C, int H, int W, void *in, void *out)
{
    return guarded([&] { small::AveragePool2D(kh, kw, s, t, b, l, r, C, H, W, F(in), F(out)); });
}
int sref_relu_f32(int C, int H, int W, void *in, void *out)
{
    return guarded([&] { small::ReLUActivation(C, H, W, F(in), F(out)); });
}
int sref_leaky_relu_f32(int C, int H, int W, void *in, void *slope, void *out)
{
    return guarded([&] { small::LeakyReLUActivation(C, H, W, F(in), F(slope), F(out)); });
}
int sref_dropout_f32(int C, int H, int W, void *in, void *scale, void *out)
{
    return guarded([&] { small::Dropout(C, H, W, F(in), F(scale), F(out)); });
}
int sref_softmax_f32(int C, int H, int W, void *in, void *out)
{
    return guarded([&] { small::SoftMax(C, H, W, F(in), F(out)); });
}
int sref_accum_f32(int C, int H, int W, void *in, void *out)
{
    return guarded([&] { small::Accum(C, H, W, F(in), F(out)); });
}
int sref_bias_f32(int C, int H, int W, void *in, void *out)
{
    return guarded([&] { small::Bias(C, H, W, F(in), F(out)); });
}
int sref_partial_bias_f32(int C, int H, int W, void *in, void *out)
{
    return guarded([&] { small::PartialBias(C, H, W, F(in), F(out)); });
}
int sref_upsample2d_f32(int scale, int C, int H, int W, void *in, void *out)
{
    return guarded([&] { small::UpSample2D(scale, C, H, W, F(in), F(out)); });
}
int sref_concat_f32(uint32_t C0, uint32_t C1, uint32_t H, uint32_t W,
                    void *in0, void *in1, void *out)
{
    return guarded([&] { small::Concat(C0, C1, H, W, F(in0), F(in1), F(out)); });
}
int sref_dense_f32(int No, int Ni, void *in, void *filt, void *out)
{
    return guarded([&] { small::Dense(No, Ni, F(in), F(filt), F(out)); });
}

// ---- 1-D functions, include/small/interface_abstract_1D.hpp (rows = their batch_size argument) -----------------
// kind 0 Conv1D, 1 PartialConv1D, 2 MaxPool1D, 3 AveragePool1D, 4 ReLUActivation1D, 5 UpSample1D (k = scale),
// 6 GroupConv1D, 7 PartialGroupConv1D (Co = groups, Ci = channels per group)
int sref_1d_f32(int kind, int k, int s, int l, int r, int Co, int Ci, int rows, int W, void *in, void *filt, void *out)
{
    return guarded([&] {
        switch (kind)
        {
        case 0: small::Conv1D(k, s, l, r, Co, Ci, rows, W, F(in), F(filt), F(out)); break;
        case 1: small::PartialConv1D(k, s, l, r, Co, Ci, rows, W, F(in), F(filt), F(out)); break;
        case 2: small::MaxPool1D(k, s, l, r, Ci, rows, W, F(in), F(out)); break;
        case 3: small::AveragePool1D(k, s, l, r, Ci, rows, W, F(in), F(out)); break;
        case 4: small::ReLUActivation1D(Ci, rows, W, F(in), F(out)); break;
        case 6: small::GroupConv1D(k, s, Co, l, r, Ci, rows, W, F(in), F(filt), F(out)); break;        // Co = groups
        case 7: small::PartialGroupConv1D(k, s, Co, l, r, Ci, rows, W, F(in), F(filt), F(out)); break;
        default: small::UpSample1D(k, Ci, rows, W, F(in), F(out)); break;
        }
    });
}

// ---- the reference's two-layer ("fused") functions, include/small/fused_interface_abstract.hpp ------------
// variant 0: Conv2D_Maxpool2D, 1: Conv2D_ReLU_Maxpool2D, 2: Conv2D_Bias_ReLU_Maxpool2D
int sref_fused_conv_pool_f32(int variant, int ck, int cs, int ct, int cb, int cl, int cr, int pk, int ps, int pt,
                             int pb, int pl, int pr, int Co, int Ci, int H, int W, void *in, void *filt, void *bias,
                             void *inter, void *out)
{
    return guarded([&] {
        if (variant == 0)
            small::Conv2D_Maxpool2D(ck, ck, cs, ct, cb, cl, cr, pk, pk, ps, pt, pb, pl, pr, Co, Ci, H, W, F(in),
                                    F(filt), F(inter), F(out));
        else if (variant == 1)
            small::Conv2D_ReLU_Maxpool2D(ck, ck, cs, ct, cb, cl, cr, pk, pk, ps, pt, pb, pl, pr, Co, Ci, H, W, F(in),
                                         F(filt), F(inter), F(out));
        else
            small::Conv2D_Bias_ReLU_Maxpool2D(ck, ck, cs, ct, cb, cl, cr, pk, pk, ps, pt, pb, pl, pr, Co, Ci, H, W,
                                              F(in), F(filt), F(bias), F(inter), F(out));
    });
}
// variant 0: Conv2D_DepthwiseConv2D, 1: Conv2D_ReLU_DepthwiseConv2D_ReLU,
//         2: Conv2D_Bias_ReLU_DepthwiseConv2D_Bias_ReLU
int sref_fused_conv_dw_f32(int variant, int ck, int cs, int ct, int cb, int cl, int cr, int dk, int ds, int dt,
                           int db, int dl, int dr, int Co, int Ci, int H, int W, void *in, void *filt, void *bias,
                           void *inter, void *dwfilt, void *dwbias, void *out)
{
    return guarded([&] {
        if (variant == 0)
            small::Conv2D_DepthwiseConv2D(ck, ck, cs, ct, cb, cl, cr, dk, dk, ds, dt, db, dl, dr, Co, Ci, H, W,
                                          F(in), F(filt), F(inter), F(dwfilt), F(out));
        else if (variant == 1)
            small::Conv2D_ReLU_DepthwiseConv2D_ReLU(ck, ck, cs, ct, cb, cl, cr, dk, dk, ds, dt, db, dl, dr, Co, Ci,
                                                    H, W, F(in), F(filt), F(inter), F(dwfilt), F(out));
        else
            small::Conv2D_Bias_ReLU_DepthwiseConv2D_Bias_ReLU(ck, ck, cs, ct, cb, cl, cr, dk, dk, ds, dt, db, dl, dr,
                                                              Co, Ci, H, W, F(in), F(filt), F(bias), F(inter),
                                                              F(dwfilt), F(dwbias), F(out));
    });
}
// variant 0: DepthwiseConv2D_ReLU, 1: DepthwiseConv2D_Bias_ReLU, 2: Conv2D_ReLU, 3: Conv2D_Bias_ReLU
// (Co is ignored by the depthwise variants)
int sref_fused_single_f32(int variant, int k, int s, int t, int b, int l, int r, int Co, int Ci, int H, int W,
                          void *in, void *filt, void *bias, void *out)
{
    return guarded([&] {
        if (variant == 0)
            small::DepthwiseConv2D_ReLU(k, k, s, t, b, l, r, Ci, H, W, F(in), F(filt), F(out));
        else if (variant == 1)
            small::DepthwiseConv2D_Bias_ReLU(k, k, s, t, b, l, r, Ci, H, W, F(in), F(filt), F(bias), F(out));
        else if (variant == 2)
            small::Conv2D_ReLU(k, k, s, t, b, l, r, Co, Ci, H, W, F(in), F(filt), F(out));
        else
            small::Conv2D_Bias_ReLU(k, k, s, t, b, l, r, Co, Ci, H, W, F(in), F(filt), F(bias), F(out));
    });
}
#endif // float

#if defined(SMALL_HAS_QUINT8_SUPPORT)
// ---- QUInt8Buffer handles ---------------------------------------------------
void *sref_qbuf_new(size_t n) { try { return new QB(n); } catch (...) { return nullptr; } }
void sref_qbuf_free(void *h) { delete static_cast<QB *>(h); }
uint8_t *sref_qbuf_data(void *h) { return Q(h).data(); }
size_t sref_qbuf_size(void *h) { return Q(h).size(); }
void sref_qbuf_set_quant(void *h, int32_t zero, int32_t multiplier, int lshift, int rshift)
{
    Q(h).m_zero = zero; Q(h).multiplier = multiplier; Q(h).lshift = lshift; Q(h).rshift = rshift;
}
// out[0..6] = zero, multiplier, lshift, rshift, min_val, max_val, b ; *scale = scale
void sref_qbuf_get_quant(void *h, int32_t *out, float *scale)
{
    out[0] = Q(h).m_zero; out[1] = Q(h).multiplier; out[2] = Q(h).lshift; out[3] = Q(h).rshift;
    out[4] = Q(h).min_val; out[5] = Q(h).max_val; out[6] = Q(h).b; *scale = Q(h).scale;
}

int sref_conv2d_u8(int kh, int kw, int s, int t, int b, int l, int r,
                   int Co, int Ci, int H, int W, void *in, void *filt, void *out)
{
    return guarded([&] { small::Conv2D(kh, kw, s, t, b, l, r, Co, Ci, H, W,
                                       Q(in), Q(filt), Q(out)); });
}
int sref_group_conv2d_u8(int kh, int kw, int s, int G, int t, int b, int l, int r,
                         int C, int H, int W, void *in, void *filt, void *out)
{
    return guarded([&] { small::GroupConv2D(kh, kw, s, G, t, b, l, r, C, H, W, Q(in), Q(filt), Q(out)); });
}
int sref_dwconv2d_u8(int kh, int kw, int s, int t, int b, int l, int r,
                     int C, int H, int W, void *in, void *filt, void *out)
{
    return guarded([&] { small::DepthwiseConv2D(kh, kw, s, t, b, l, r, C, H, W,
                                                Q(in), Q(filt), Q(out)); });
}
int sref_maxpool2d_u8(int kh, int kw, int s, int t, int b, int l, int r,
                      int C, int H, int W, void *in, void *out)
{
    return guarded([&] { small::MaxPool2D(kh, kw, s, t, b, l, r, C, H, W, Q(in), Q(out)); });
}
int sref_relu_u8(int C, int H, int W, void *in, void *out)
{
    return guarded([&] { small::ReLUActivation(C, H, W, Q(in), Q(out)); });
}
int sref_concat_u8(uint32_t C0, uint32_t C1, uint32_t H, uint32_t W,
                   void *in0, void *in1, void *out)
{
    return guarded([&] { small::Concat(C0, C1, H, W, Q(in0), Q(in1), Q(out)); });
}
int sref_dense_u8(int No, int Ni, void *in, void *filt, void *out)
{
    return guarded([&] { small::Dense(No, Ni, Q(in), Q(filt), Q(out)); });
}
#endif // quint8

// ---- Layer and Model classes (float) -----------------------------------------
// The reference's own Layer / Model objects on flat (NCHW / OIHW, unpacked) data: the shim packs the
// input for this platform's blocking, runs compute_output() / inference() and unpacks the result, so
// the REF and ZEN2 builds can be compared with each other and with other implementations.
#if defined(SMALL_HAS_FLOAT_SUPPORT)
} // extern "C"
namespace {
FB fb_from(const float *p, size_t n)
{
    FB b(n);
    if (n) std::memcpy(b.data(), p, n * sizeof(float));
    return b;
}
small::Tensor<FB> packed_tensor(const float *flat, small::shape_type const &shape)
{
    const size_t n = small::compute_size(shape);
    FB f = fb_from(flat, n), p(n);
    small::pack_buffer(f, small::INPUT, 1U, shape[1], shape[2], shape[3], FB::C_ib, FB::C_ob, p);
    return small::Tensor<FB>(shape, std::move(p));
}
void unpack_tensor(small::Tensor<FB> const &t, float *flat, int *out_shape)
{
    auto const &s = t.shape();
    for (int i = 0; i < 4; ++i) out_shape[i] = (int)s[i];
    const size_t n = small::compute_size(s);
    FB p(n), f(n);
    std::memcpy(p.data(), t.buffer().data(), n * sizeof(float));
    small::unpack_buffer(p, small::OUTPUT, 1U, s[1], s[2], s[3], FB::C_ib, FB::C_ob, f);
    std::memcpy(flat, f.data(), n * sizeof(float));
}
} // namespace
extern "C" {

// kind: 0 Conv2DLayer, 1 PartialConv2DLayer, 2 DepthwiseConv2DLayer, 3 Conv1DLayer; batch 1 (the reference computes one
// image).  filters [Co][Ci][kh][kw] (depthwise [C][kh][kw]); bias Co or NULL; bn 4 x Co (gamma, beta, mean,
// variance) or NULL; out is in/out, flat [Co_padded][Ho][Wo].
int sref_conv_layer_f32(int kind, int C, int H, int W, int kh, int kw, int stride, int padding, int Co,
                        const float *filters, const float *bias, const float *bn, float eps, int act, float slope,
                        const float *in, float *out, int *out_shape)
{
    return guarded([&] {
        const small::shape_type is{1UL, (size_t)C, (size_t)H, (size_t)W};
        const size_t nf = (kind == 2 ? (size_t)C : (size_t)Co * C) * kh * kw;
        const size_t nb = kind == 2 ? C : Co;
        FB f = fb_from(filters, nf), b = bias ? fb_from(bias, nb) : FB();
        FB g, be, mu, var;
        if (bn) { g = fb_from(bn, nb); be = fb_from(bn + nb, nb); mu = fb_from(bn + 2 * nb, nb); var = fb_from(bn + 3 * nb, nb); }
        const auto pad = padding ? small::PADDING_F : small::PADDING_V;
        const auto a = (small::ActivationType)act;
        std::unique_ptr<small::Layer<FB>> layer;
        if (kind == 3)      // Conv1DLayer: kh is ignored; it has no constructor taking bias and batch normalisation
        {
            if (bn) layer.reset(new small::Conv1DLayer<FB>(is, kw, stride, pad, Co, f, g, be, mu, var, eps, false, a, slope));
            else if (bias) layer.reset(new small::Conv1DLayer<FB>(is, kw, stride, pad, Co, f, b, false, a, slope));
            else layer.reset(new small::Conv1DLayer<FB>(is, kw, stride, pad, Co, f, false, a, slope));
        }
        else if (kind == 2)
        {
            if (bn) layer.reset(new small::DepthwiseConv2DLayer<FB>(is, kh, kw, stride, pad, f, b, g, be, mu, var, eps, false, a, slope));
            else if (bias) layer.reset(new small::DepthwiseConv2DLayer<FB>(is, kh, kw, stride, pad, f, b, false, a, slope));
            else layer.reset(new small::DepthwiseConv2DLayer<FB>(is, kh, kw, stride, pad, f, false, a, slope));
        }
        else if (kind == 1)
        {
            if (bn) layer.reset(new small::PartialConv2DLayer<FB>(is, kh, kw, stride, pad, Co, f, b, g, be, mu, var, eps, false, a, slope));
            else if (bias) layer.reset(new small::PartialConv2DLayer<FB>(is, kh, kw, stride, pad, Co, f, b, false, a, slope));
            else layer.reset(new small::PartialConv2DLayer<FB>(is, kh, kw, stride, pad, Co, f, false, a, slope));
        }
        else
        {
            if (bn) layer.reset(new small::Conv2DLayer<FB>(is, kh, kw, stride, pad, Co, f, b, g, be, mu, var, eps, false, a, slope));
            else if (bias) layer.reset(new small::Conv2DLayer<FB>(is, kh, kw, stride, pad, Co, f, b, false, a, slope));
            else layer.reset(new small::Conv2DLayer<FB>(is, kh, kw, stride, pad, Co, f, false, a, slope));
        }
        auto x = packed_tensor(in, is);
        auto y = packed_tensor(out, layer->output_shape());
        layer->compute_output({&x}, &y);
        unpack_tensor(y, out, out_shape);
    });
}

// kind: 0 MaxPool2DLayer, 1 AveragePool2DLayer, 2 ReLULayer, 3 LeakyReLULayer(slope), 4 UpSample2DLayer(k = scale),
// 5 AddLayer (out += in), 6 RouteLayer(one input), 7 RouteLayer(in, in2 with C2 channels), 8 SoftMaxLayer
int sref_simple_layer_f32(int kind, int C, int H, int W, int k, int kw, int stride, int padding, float slope,
                          const float *in, const float *in2, int C2, float *out, int *out_shape)
{
    return guarded([&] {
        const small::shape_type is{1UL, (size_t)C, (size_t)H, (size_t)W};
        const small::shape_type is2{1UL, (size_t)C2, (size_t)H, (size_t)W};
        const auto pad = padding ? small::PADDING_F : small::PADDING_V;
        std::unique_ptr<small::Layer<FB>> layer;
        switch (kind)
        {
        case 0: layer.reset(new small::MaxPool2DLayer<FB>(is, k, kw, stride, pad)); break;
        case 1: layer.reset(new small::AveragePool2DLayer<FB>(is, k, kw, stride, pad)); break;
        case 2: layer.reset(new small::ReLULayer<FB>(is)); break;
        case 3: layer.reset(new small::LeakyReLULayer<FB>(is, slope)); break;
        case 4: layer.reset(new small::UpSample2DLayer<FB>(is, k)); break;
        case 5: layer.reset(new small::AddLayer<FB>(is, is)); break;
        case 6: layer.reset(new small::RouteLayer<FB>(is)); break;
        case 7: layer.reset(new small::RouteLayer<FB>(is, is2)); break;
        case 8: layer.reset(new small::SoftMaxLayer<FB>(is)); break;
        default: throw std::invalid_argument("sref_simple_layer_f32: unknown kind");
        }
        auto x = packed_tensor(in, is);
        auto y = packed_tensor(out, layer->output_shape());
        if (kind == 7)
        {
            auto x2 = packed_tensor(in2, is2);
            layer->compute_output({&x, &x2}, &y);
        }
        else
            layer->compute_output({&x}, &y);
        unpack_tensor(y, out, out_shape);
    });
}

// which: 0 MobileNetTiny, 1 Resnet8Tiny, 2 DSCNNTiny, 3 TinyYoloV2 as the reference defines them;
// filters unpacked, in the model's own filter order.
int sref_model_f32(int which, int C, int H, int W, const float *const *filters, const size_t *sizes, int nfilters,
                   const float *in, float *out, int *out_shape)
{
    return guarded([&] {
        const small::shape_type is{1UL, (size_t)C, (size_t)H, (size_t)W};
        std::vector<std::unique_ptr<FB>> own;
        std::vector<FB *> fl;
        for (int i = 0; i < nfilters; ++i)
        {
            own.emplace_back(new FB(fb_from(filters[i], sizes[i])));
            fl.push_back(own.back().get());
        }
        std::unique_ptr<small::Model<FB>> m;
        switch (which)
        {
        case 0: m.reset(new small::MobileNetTiny<FB>(is, fl, false)); break;
        case 1: m.reset(new small::Resnet8Tiny<FB>(is, fl, false)); break;
        case 2: m.reset(new small::DSCNNTiny<FB>(is, fl, false)); break;
        case 3: m.reset(new small::TinyYoloV2<FB>(is, fl, false)); break;
        case 4: m.reset(new small::AutoencoderTiny<FB>(is, 16, fl, false)); break;
        case 5: m.reset(new small::DSCNNSquareTiny<FB>(is, fl, false)); break;
        default: throw std::invalid_argument("sref_model_f32: unknown model");
        }
        auto x = packed_tensor(in, is);
        auto outs = m->inference(&x);
        unpack_tensor(*outs[0], out, out_shape);
    });
}

// ---- Darknet cfg / weights model, YOLO decode, non-maximum suppression -------------------------------------------
// Runs the model the two files describe on one flat [C][H][W] image.  out receives the YOLO heads' records one
// after the other (each head is [predictions][5 + classes]); out_preds[i] = predictions of head i.
// det (may be NULL): detections after process_outputs(conf, iou), 7 floats each {x, y, w, h, objectness, class
// score, class id}; *n_det in: capacity, out: count.
int sref_darknet_f32(const char *cfg, const char *weights, const float *in, size_t n_in, float *out, size_t out_cap,
                       int *out_preds, int *n_heads, int *record_len, float conf, float iou, float *det, int *n_det)
{
    return guarded([&] {
        small::Darknet<FB> model(cfg, weights);
        auto const &is = model.get_input_shape();
        if (small::compute_size(is) != n_in) throw std::invalid_argument("darknet shim: input size mismatch");
        auto x = packed_tensor(in, is);
        model.inference(&x);                     // the second pass runs on recycled pool tensors
        auto outs = model.inference(&x);
        size_t at = 0;
        *n_heads = (int)outs.size();
        for (size_t i = 0; i < outs.size(); ++i)
        {
            auto const &s = outs[i]->shape();
            out_preds[i] = (int)s[2];
            *record_len = (int)s[3];
            const size_t n = s[2] * s[3];
            if (at + n > out_cap) throw std::invalid_argument("darknet shim: output capacity");
            for (size_t k = 0; k < n; ++k) out[at + k] = outs[i]->buffer()[k];
            at += n;
        }
        if (det)
        {
            auto d = model.process_outputs(outs, conf, iou);
            const int cap = *n_det;
            *n_det = (int)d.size();
            for (int i = 0; i < (int)d.size() && i < cap; ++i)
            {
                float *r = det + 7 * i;
                r[0] = d[i].bbox.x; r[1] = d[i].bbox.y; r[2] = d[i].bbox.w; r[3] = d[i].bbox.h;
                r[4] = d[i].objectness; r[5] = d[i].class_score; r[6] = (float)d[i].class_id;
            }
        }
    });
}

// basic_nms on n records of 7 floats (layout as above); kept records are written to out, their count returned in *n_out
int sref_nms(const float *pred, int n, float iou, float *out, int *n_out)
{
    return guarded([&] {
        std::vector<small::Detection> p;
        for (int i = 0; i < n; ++i)
        {
            const float *r = pred + 7 * i;
            p.push_back(small::Detection{{r[0], r[1], r[2], r[3]}, r[4], r[5], (size_t)r[6]});
        }
        auto k = small::basic_nms(p, iou);
        *n_out = (int)k.size();
        for (size_t i = 0; i < k.size(); ++i)
        {
            float *r = out + 7 * i;
            r[0] = k[i].bbox.x; r[1] = k[i].bbox.y; r[2] = k[i].bbox.w; r[3] = k[i].bbox.h;
            r[4] = k[i].objectness; r[5] = k[i].class_score; r[6] = (float)k[i].class_id;
        }
    });
}

// YOLOLayer on a flat [C][H][W] input (C is padded to the channel block with zeros by the caller)
int sref_yolo_layer_f32(int C, int H, int W, const uint32_t *anchors_wh, int num_anchors, int classes, int image_size,
                          const float *in, float *out)
{
    return guarded([&] {
        const small::shape_type is{1UL, (size_t)C, (size_t)H, (size_t)W};
        std::vector<std::pair<uint32_t, uint32_t>> an;
        for (int a = 0; a < num_anchors; ++a) an.emplace_back(anchors_wh[2 * a], anchors_wh[2 * a + 1]);
        small::YOLOLayer<FB> layer(is, an, classes, image_size);
        auto x = packed_tensor(in, is);
        small::Tensor<FB> y(layer.output_shape());
        layer.compute_output({&x}, &y);
        for (size_t k = 0; k < layer.output_size(); ++k) out[k] = y.buffer()[k];
    });
}
#endif // float layers

} // extern "C"
