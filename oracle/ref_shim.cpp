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

} // extern "C"
