/* TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C CPU restatement of the SMaLL layer hot path.  It exists to check the
 * HIP library; nothing in the shipped library or its host headers includes,
 * links, loads or calls it.  Only tests, the smoke check and the cpu_baseline
 * leg of the benchmark use it.
 *
 * Layout contract (reference: include/small/abstract_layer.hpp:1419-1432,
 * include/small/buffers.hpp:33-120):
 *   activations  [N][C/cb][H][W][cb]
 *   conv filter  [Co/cb][Ci/cib][Fh][Fw][cib][cb]     (cib = Ci when Ci in {1,2,3} and Ci < cb)
 *   dw filter    [C/cb][Fh][Fw][cb]
 * "cb" is the channel block (C_ob == C_ib of the platform): 1 for the reference's
 * REF build, 16 for its ZEN2 build and for the HIP library.
 * Every function returns 0, or one of the SO_E* codes where the reference
 * throws std::invalid_argument.
 *
 * Pinning status per function is listed at the top of small_oracle.c.
 */
#ifndef SMALL_ORACLE_H
#define SMALL_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SO_OK 0
#define SO_ESTRIDE 1   /* "<op> ERROR: stride unsupported."      */
#define SO_ECHANNELS 2 /* "<op> ERROR: in_channels unsupported." */
#define SO_ESCALE 3    /* "Upsample ERROR: scale factor unsupported (only 1 or 2)." */
#define SO_EINVAL 4

#define SO_ACT_NONE 0
#define SO_ACT_RELU 1
#define SO_ACT_LEAKY 2

/* quantisation parameters as carried by the reference's QUInt8Buffer objects */
typedef struct so_quant
{
    int32_t zero;       /* m_zero  */
    int32_t multiplier; /* q_mul   */
    int32_t lshift;
    int32_t rshift;
} so_quant;

/* ---- shape + index contract --------------------------------------------- */
void so_calc_padding(size_t I_dim, uint32_t K_dim, uint32_t stride, uint8_t *front, uint8_t *back);
uint32_t so_output_dim(uint32_t in_dim, uint32_t stride, uint32_t k_dim);
long so_packed_weight_index(uint32_t Co, uint32_t Ci, uint32_t Fh, uint32_t Fw, uint32_t cob,
                            uint32_t cib, size_t o, size_t c, size_t h, size_t w);
long so_packed_buffer_index(uint32_t C, uint32_t H, uint32_t W, uint32_t cb, size_t c, size_t h,
                            size_t w);
/* type: 0 INPUT, 1 OUTPUT, 2 FILTER_DW, 3 FILTER_CONV, 4 FILTER_FC; esize = bytes per element */
long so_pack(const void *flat, int type, uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3,
             uint32_t cib, uint32_t cob, void *packed, size_t esize);
long so_unpack(const void *packed, int type, uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3,
               uint32_t cib, uint32_t cob, void *flat, size_t esize);

/* ---- float32 ------------------------------------------------------------- */
/* acc64 != 0: accumulate in double (error attribution), else float in the reference's order */
int so_conv2d_f32(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                  int Co, int Ci, int H, int W, const float *in, const float *filt, float *out,
                  int accumulate, int acc64);
/* bias (packed, Co floats, may be NULL) is broadcast first, the convolution accumulates on
 * top of it, then the activation is applied: the reference's Conv2DLayer sequence. */
int so_conv2d_bias_act_f32(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl,
                           int pr, int Co, int Ci, int H, int W, const float *in,
                           const float *filt, const float *bias, int act, float slope,
                           float *out);
int so_dwconv2d_f32(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                    int C, int H, int W, const float *in, const float *filt, float *out,
                    int accumulate, int acc64);
int so_maxpool2d_f32(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                     int C, int H, int W, const float *in, float *out);
int so_avgpool2d_f32(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                     int C, int H, int W, const float *in, float *out);
int so_relu_f32(int batch, int cb, int C, int H, int W, const float *in, float *out);
int so_dropout_f32(int batch, int cb, int C, int H, int W, const float *in, float scale, float *out);
int so_softmax_f32(int batch, int cb, int C, int H, int W, const float *in, float *out);
int so_leaky_relu_f32(int batch, int cb, int C, int H, int W, const float *in, float slope,
                      float *out);
int so_accum_f32(int batch, int cb, int C, int H, int W, const float *in, float *out);
int so_bias_f32(int batch, int cb, int C, int H, int W, const float *bias, float *out,
                int accumulate);
int so_upsample2d_f32(int batch, int cb, int scale, int C, int H, int W, const float *in,
                      float *out);
int so_yolo_decode_f32(int batch, int cb, int C, int H, int W, int num_anchors, const uint32_t *anchors_wh,
                       int num_classes, int image_size, const float *in, float *out);
int so_upsample1d_f32(int batch, int cb, int scale, int C, int rows, int W, const float *in, float *out);
int so_concat(int batch, uint32_t C0, uint32_t C1, uint32_t H, uint32_t W, const void *in0,
              const void *in1, void *out, size_t esize);
/* y = W x : Conv2D(1,1,...) on a 1x1 image (how every reference model spells a
 * fully-connected layer); NOT the reference's literal small::Dense formula. */
int so_dense_f32(int batch, int cb, int No, int Ni, const float *in, const float *filt,
                 float *out);
/* the literal reference small::Dense: out[o*Ni+i] = in[o*Ni+i]*filt[o] (a 1x1 depthwise) */
int so_dense_literal_f32(int cb, int No, int Ni, const float *in, const float *filt, float *out);

/* ---- quantised uint8 ------------------------------------------------------ */
uint8_t so_requant(int32_t acc, const so_quant *oq);
int so_conv2d_u8(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                 int Co, int Ci, int H, int W, const uint8_t *in, const so_quant *iq,
                 const uint8_t *filt, const so_quant *fq, uint8_t *out, const so_quant *oq);
int so_dwconv2d_u8(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                   int C, int H, int W, const uint8_t *in, const so_quant *iq, const uint8_t *filt,
                   const so_quant *fq, uint8_t *out, const so_quant *oq);
int so_maxpool2d_u8(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                    int C, int H, int W, const uint8_t *in, const so_quant *iq, uint8_t *out,
                    const so_quant *oq);
int so_relu_u8(int batch, int cb, int C, int H, int W, const uint8_t *in, const so_quant *iq,
               uint8_t *out, const so_quant *oq);
int so_dense_u8(int batch, int cb, int No, int Ni, const uint8_t *in, const so_quant *iq,
                const uint8_t *filt, const so_quant *fq, uint8_t *out, const so_quant *oq);
/* no reference counterpart; each equals a reference uint8 call on a filter of ones, which pins it (small_oracle.c) */
int so_accum_u8(int batch, int cb, int C, int H, int W, const uint8_t *in, const so_quant *iq,
                uint8_t *out, const so_quant *oq);
int so_avgpool2d_u8(int batch, int cb, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                    int C, int H, int W, const uint8_t *in, const so_quant *iq, uint8_t *out,
                    const so_quant *oq);

#ifdef __cplusplus
}
#endif
#endif
