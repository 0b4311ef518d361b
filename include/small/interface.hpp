// The `small::` layer functions on the MI355X library.
//
// Same names, argument order and error behaviour as the reference's public API
// (include/small/interface.hpp:49-497, definitions in include/small/interface_abstract.hpp):
// buffers by reference, pads as uint8_t in the order top, bottom, left, right, and
// std::invalid_argument with the reference's messages for unsupported strides / channel counts.
// Each function forwards to one entry point of the C ABI (include/small_hip.h).
//
// Additions (no counterpart in the reference):
//   - every layer also exists with a leading `int batch` argument in namespace small::batched;
//     image n of a batched call equals the batch-1 call on image n
//   - Conv2D_Bias_Act / DepthwiseConv2D_Bias_Act: bias + convolution + activation in one pass
//     (the reference's Layer classes issue Bias, PartialConv2D and the activation separately)
//   - Accum and AveragePool2D for QUInt8Buffer (the reference leaves them unimplemented)
// Divergence: small::Dense computes y = W x (what every reference model means by a dense layer
// and spells as Conv2D on a 1x1 image); the reference's own small::Dense body is a per-channel
// scale with no callers and is available as small::DenseAsWritten.
#pragma once

#include <cstdlib>
#include <stdexcept>
#include <string>
#include <type_traits>

#include "../small_hip.h"
#include "Buffer.hpp"
#include "utils.hpp"

namespace small
{

enum ActivationType
{
    NONE = SMALL_HIP_ACT_NONE,
    RELU = SMALL_HIP_ACT_RELU,
    LEAKY = SMALL_HIP_ACT_LEAKY,
    SOFTMAX = 3   // Layer classes only: small::SoftMax applied after the layer (float)
};

namespace detail
{
template <class BufferT>
struct type_tag
{
    static const char *name() { return std::is_same<BufferT, FloatBuffer>::value ? "float" : "quint8"; }
};

// status -> the exception the reference throws from the same place
template <class BufferT>
inline void raise(int status, const char *op)
{
    if (status == SMALL_HIP_OK) return;
    const std::string head = std::string(op) + "<" + type_tag<BufferT>::name() + "> ERROR: ";
    switch (status)
    {
    case SMALL_HIP_ESTRIDE: throw std::invalid_argument(head + "stride unsupported.");
    case SMALL_HIP_ECHANNELS: throw std::invalid_argument(head + "in_channels unsupported.");
    case SMALL_HIP_ESCALE: throw std::invalid_argument(head + "scale factor unsupported (only 1 or 2).");
    case SMALL_HIP_ENOMEM: throw std::bad_alloc();
    case SMALL_HIP_EINVAL: throw std::invalid_argument(head + small_hip_last_error());
    default: throw std::runtime_error(head + small_hip_last_error());
    }
}

// "Conv2D<float> ERROR: ..." -> "Conv1D<float> ERROR: ..." for the 1-D functions built on the 2-D ones
inline std::string rename_op(std::string msg, std::string const &from, std::string const &to)
{
    if (msg.compare(0, from.size(), from) == 0) msg.replace(0, from.size(), to);
    return msg;
}

template <class BufferT>
using if_float = std::enable_if_t<std::is_same<FloatBuffer, BufferT>::value, bool>;
template <class BufferT>
using if_quint8 = std::enable_if_t<std::is_same<QUInt8Buffer, BufferT>::value, bool>;

inline small_hip_stream_t st() { return current_stream(); }

// SMALL_HIP_TUNE="fuse_pool=0" makes every convolution + pooling pair run as its two launches.  The one-launch form sums
// in another float32 order than the stand-alone convolution (another kernel), so a model class and the same layers
// called one by one agree within the float32 tolerance by default and bit for bit with this switch off (the
// reference's test_tinyyolov2.cpp asserts the latter of its two call paths).
inline bool pool_fusion_enabled()
{
    static const bool on = small_hip_tune_int("fuse_pool", 1) != 0;
    return on;
}

// Does Conv2D_*_DepthwiseConv2D_* run this pair as one launch?  The library answers (small_hip_conv2d_dwconv2d_one_launch_f32:
// first layers in front of a 3x3 stride-1 depthwise layer; pointwise convolutions of 16 to 64, 96 or 128 input channels in
// front of a 3x3 depthwise layer whose output fills the one-launch kernel's tiles), and says whether the one launch equals
// the two launches bit for bit.  By default only those pairs are fused: the reference's model tests compare a model class
// with its layer functions for equality.  SMALL_HIP_TUNE="fuse_conv_dw=0" switches the fusion off; =2 adds the pairs
// (96 / 128 input channels) that are faster as one launch but may differ from the two launches by float32 rounding.
template <class BufferT>
inline bool conv_dw_one_launch(int batch, int conv_kernel_height, int conv_kernel_width, int conv_stride, int conv_t_pad, int conv_b_pad,
                               int conv_l_pad, int conv_r_pad, int dw_kernel_height, int dw_kernel_width, int dw_stride,
                               int dw_t_pad, int dw_b_pad, int dw_l_pad, int dw_r_pad, int output_channels, int input_channels,
                               int input_height, int input_width)
{
    if (!std::is_same<typename BufferT::value_type, float>::value) return false;
    static const int fuse = small_hip_tune_int("fuse_conv_dw", 1);
    if (fuse <= 0) return false;
    const int form = small_hip_conv2d_dwconv2d_one_launch_f32(batch, conv_kernel_height, conv_kernel_width, conv_stride, conv_t_pad,
                                                              conv_b_pad, conv_l_pad, conv_r_pad, dw_kernel_height, dw_kernel_width,
                                                              dw_stride, dw_t_pad, dw_b_pad, dw_l_pad, dw_r_pad, output_channels,
                                                              input_channels, input_height, input_width);
    // six K-steps (96 channels) are bit-identical too but were measured with the 128-channel pairs: same switch
    const bool short_reduction = input_channels <= 64;
    return form == 1 ? (short_reduction || fuse >= 2) : form == 2 && fuse >= 2;
}
} // namespace detail

// =================================================================================================
namespace batched
{

// ---- Conv2D / PartialConv2D ------------------------------------------------------------------------
template <class BufferT, detail::if_float<BufferT> = true>
void Conv2D(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
            uint8_t l_pad, uint8_t r_pad, int output_channels, int input_channels, int input_height,
            int input_width, BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_conv2d_f32(batch, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad,
                                                r_pad, output_channels, input_channels, input_height,
                                                input_width, input_buf.device_in(), filter_buf.device_in(),
                                                output_buf.device_out(), detail::st()),
                           "Conv2D");
}

template <class BufferT, detail::if_quint8<BufferT> = true>
void Conv2D(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
            uint8_t l_pad, uint8_t r_pad, int output_channels, int input_channels, int input_height,
            int input_width, BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    const small_hip_quant iq = input_buf.quant(), fq = filter_buf.quant(), oq = output_buf.quant();
    detail::raise<BufferT>(small_hip_conv2d_u8(batch, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad,
                                               r_pad, output_channels, input_channels, input_height, input_width,
                                               input_buf.device_in(), &iq, filter_buf.device_in(), &fq,
                                               output_buf.device_out(), &oq, detail::st()),
                           "Conv2D");
}

template <class BufferT, detail::if_float<BufferT> = true>
void PartialConv2D(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
                   uint8_t l_pad, uint8_t r_pad, int output_channels, int input_channels, int input_height,
                   int input_width, BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_partial_conv2d_f32(batch, kernel_height, kernel_width, stride, t_pad, b_pad,
                                                        l_pad, r_pad, output_channels, input_channels,
                                                        input_height, input_width, input_buf.device_in(),
                                                        filter_buf.device_in(), output_buf.device_out(),
                                                        detail::st()),
                           "PartialConv2D");
}

// ---- GroupConv2D / PartialGroupConv2D (interface_abstract.hpp:1265-1533) ---------------------------------
// `output_groups` convolutions of input_channels -> input_channels, one per slab of input_channels channels
// of the packed tensors; filter_buf holds one packed Conv2D filter per group, group after group.
template <class BufferT, detail::if_float<BufferT> = true>
void GroupConv2D(int batch, int kernel_height, int kernel_width, int stride, int output_groups, uint8_t t_pad,
                 uint8_t b_pad, uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height,
                 int input_width, BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_group_conv2d_f32(batch, kernel_height, kernel_width, stride, output_groups,
                                                      t_pad, b_pad, l_pad, r_pad, input_channels, input_height,
                                                      input_width, input_buf.device_in(), filter_buf.device_in(),
                                                      0, output_buf.device_out(), detail::st()),
                           "GroupConv2D");
}

template <class BufferT, detail::if_quint8<BufferT> = true>
void GroupConv2D(int batch, int kernel_height, int kernel_width, int stride, int output_groups, uint8_t t_pad,
                 uint8_t b_pad, uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height,
                 int input_width, BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    const small_hip_quant iq = input_buf.quant(), fq = filter_buf.quant(), oq = output_buf.quant();
    detail::raise<BufferT>(small_hip_group_conv2d_u8(batch, kernel_height, kernel_width, stride, output_groups,
                                                     t_pad, b_pad, l_pad, r_pad, input_channels, input_height,
                                                     input_width, input_buf.device_in(), &iq,
                                                     filter_buf.device_in(), &fq, output_buf.device_out(), &oq,
                                                     detail::st()),
                           "GroupConv2D");
}

template <class BufferT, detail::if_float<BufferT> = true>
void PartialGroupConv2D(int batch, int kernel_height, int kernel_width, int stride, int output_groups,
                        uint8_t t_pad, uint8_t b_pad, uint8_t l_pad, uint8_t r_pad, int input_channels,
                        int input_height, int input_width, BufferT const &input_buf, BufferT const &filter_buf,
                        BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_group_conv2d_f32(batch, kernel_height, kernel_width, stride, output_groups,
                                                      t_pad, b_pad, l_pad, r_pad, input_channels, input_height,
                                                      input_width, input_buf.device_in(), filter_buf.device_in(),
                                                      1, output_buf.device_out(), detail::st()),
                           "PartialGroupConv2D");
}

// bias_buf may be empty (size 0): no bias
template <class BufferT, detail::if_float<BufferT> = true>
void Conv2D_Bias_Act(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
                     uint8_t l_pad, uint8_t r_pad, int output_channels, int input_channels, int input_height,
                     int input_width, BufferT const &input_buf, BufferT const &filter_buf,
                     BufferT const &bias_buf, ActivationType act, float negative_slope, BufferT &output_buf)
{
    detail::raise<BufferT>(
        small_hip_conv2d_bias_act_f32(batch, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad,
                                      output_channels, input_channels, input_height, input_width,
                                      input_buf.device_in(), filter_buf.device_in(),
                                      bias_buf.size() ? bias_buf.device_in() : nullptr, (int)act, negative_slope,
                                      output_buf.device_out(), detail::st()),
        "Conv2D_Bias_Act");
}

// out = act((out + conv(in, filter)) + bias): PartialConv2D + PartialBias + activation in one pass
template <class BufferT, detail::if_float<BufferT> = true>
void PartialConv2D_Bias_Act(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad,
                            uint8_t b_pad, uint8_t l_pad, uint8_t r_pad, int output_channels, int input_channels,
                            int input_height, int input_width, BufferT const &input_buf, BufferT const &filter_buf,
                            BufferT const &bias_buf, ActivationType act, float negative_slope, BufferT &output_buf)
{
    detail::raise<BufferT>(
        small_hip_partial_conv2d_bias_act_f32(batch, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad,
                                              r_pad, output_channels, input_channels, input_height, input_width,
                                              input_buf.device_in(), filter_buf.device_in(),
                                              bias_buf.size() ? bias_buf.device_in() : nullptr, (int)act,
                                              negative_slope, output_buf.device_out(), detail::st()),
        "PartialConv2D_Bias_Act");
}

// Conv2D [+ Accum(accum_buf, out)] [+ ReLU] on the quantised path in one launch, bit-identical to the
// separate calls; accum_buf may be null.  `prepared` (may be null) is the filter in the form
// small_hip_conv2d_u8_prepare_filter writes; with it the per-call filter pre-pass is skipped.
template <class BufferT, detail::if_quint8<BufferT> = true>
void Conv2D_Accum_ReLU(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
                       uint8_t l_pad, uint8_t r_pad, int output_channels, int input_channels, int input_height,
                       int input_width, BufferT const &input_buf, BufferT const &filter_buf, void const *prepared,
                       BufferT const *accum_buf, bool relu, BufferT &output_buf)
{
    const small_hip_quant iq = input_buf.quant(), fq = filter_buf.quant(), oq = output_buf.quant();
    small_hip_quant aq = oq;
    uint8_t const *acc = nullptr;
    if (accum_buf)
    {
        aq = accum_buf->quant();
        acc = accum_buf->device_in();
    }
    int rc;
    if (prepared)
        rc = small_hip_conv2d_accum_relu_u8_prepared(batch, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad,
                                                     r_pad, output_channels, input_channels, input_height,
                                                     input_width, input_buf.device_in(), &iq, prepared, &fq, acc,
                                                     &aq, relu ? 1 : 0, output_buf.device_out(), &oq, detail::st());
    else
        rc = small_hip_conv2d_accum_relu_u8(batch, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad,
                                            output_channels, input_channels, input_height, input_width,
                                            input_buf.device_in(), &iq, filter_buf.device_in(), &fq, acc, &aq,
                                            relu ? 1 : 0, output_buf.device_out(), &oq, detail::st());
    detail::raise<BufferT>(rc, "Conv2D");
}

// out = MaxPool2D(act(Conv2D(in, filter) + bias)) in one launch when the pooling window is 2x2 stride 2 without
// padding (the pooling runs on the accumulators; first layers only when the kernel's pixel tiles fill the map well); any
// other window runs the two layers through inter_output_buf.  bias_buf may be empty.
template <class BufferT, detail::if_float<BufferT> = true>
void Conv2D_Bias_Act_Maxpool2D(int batch, int conv_kernel_height, int conv_kernel_width, int conv_stride,
                               uint8_t conv_t_pad, uint8_t conv_b_pad, uint8_t conv_l_pad, uint8_t conv_r_pad,
                               int pool_kernel_height, int pool_kernel_width, int pool_stride, uint8_t pool_t_pad,
                               uint8_t pool_b_pad, uint8_t pool_l_pad, uint8_t pool_r_pad, int output_channels,
                               int input_channels, int input_height, int input_width, BufferT const &input_buf,
                               BufferT const &filter_buf, BufferT const &bias_buf, ActivationType act,
                               float negative_slope, BufferT &inter_output_buf, BufferT &output_buf)
{
    bool fusable = detail::pool_fusion_enabled() && pool_kernel_height == 2 && pool_kernel_width == 2 && pool_stride == 2 && !pool_t_pad &&
                   !pool_b_pad && !pool_l_pad && !pool_r_pad &&
                   (input_channels % (int)BufferT::C_ib == 0 || (conv_kernel_height == 3 && conv_kernel_width == 3)) &&
                   !(act == LEAKY && negative_slope < 0.f);
    if (fusable)
    {
        // first layers (1-3 input channels) are fused on 16 x 16 pixel tiles of one image: on small maps the ragged
        // tiles cost more than the saved pooling pass, so fuse from 90% fill; the main kernel counts pooling windows
        // straight through and loses nothing on any map
        const long Hc = (long)output_dim(input_height + conv_t_pad + conv_b_pad, conv_stride, conv_kernel_height);
        const long Wc = (long)output_dim(input_width + conv_l_pad + conv_r_pad, conv_stride, conv_kernel_width);
        const bool first = input_channels % (int)BufferT::C_ib != 0;
        const long slots = ((Hc + 15) / 16 * 16) * ((Wc + 15) / 16 * 16);
        fusable = Hc > 0 && Wc > 0 && (!first || 10 * Hc * Wc >= 9 * slots);
    }
    if (fusable)
    {
        detail::raise<BufferT>(
            small_hip_conv2d_bias_act_maxpool2d_f32(
                batch, conv_kernel_height, conv_kernel_width, conv_stride, conv_t_pad, conv_b_pad, conv_l_pad,
                conv_r_pad, 2, 2, 2, 0, 0, 0, 0, output_channels, input_channels, input_height, input_width,
                input_buf.device_in(), filter_buf.device_in(), bias_buf.size() ? bias_buf.device_in() : nullptr,
                (int)act, negative_slope, output_buf.device_out(), detail::st()),
            "Conv2D_Bias_ReLU_Maxpool2D");
        return;
    }
    Conv2D_Bias_Act(batch, conv_kernel_height, conv_kernel_width, conv_stride, conv_t_pad, conv_b_pad, conv_l_pad,
                    conv_r_pad, output_channels, input_channels, input_height, input_width, input_buf, filter_buf,
                    bias_buf, act, negative_slope, inter_output_buf);
    const int Ho = (int)output_dim(input_height + conv_t_pad + conv_b_pad, conv_stride, conv_kernel_height);
    const int Wo = (int)output_dim(input_width + conv_l_pad + conv_r_pad, conv_stride, conv_kernel_width);
    detail::raise<BufferT>(small_hip_maxpool2d_f32(batch, pool_kernel_height, pool_kernel_width, pool_stride,
                                                   pool_t_pad, pool_b_pad, pool_l_pad, pool_r_pad, output_channels,
                                                   Ho, Wo, inter_output_buf.device_in(), output_buf.device_out(),
                                                   detail::st()),
                           "MaxPool2D");
}

// ---- DepthwiseConv2D / PartialDepthwiseConv2D ------------------------------------------------------
template <class BufferT, detail::if_float<BufferT> = true>
void DepthwiseConv2D(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
                     uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height, int input_width,
                     BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_depthwise_conv2d_f32(batch, kernel_height, kernel_width, stride, t_pad, b_pad,
                                                          l_pad, r_pad, input_channels, input_height, input_width,
                                                          input_buf.device_in(), filter_buf.device_in(),
                                                          output_buf.device_out(), detail::st()),
                           "DepthwiseConv2D");
}

template <class BufferT, detail::if_quint8<BufferT> = true>
void DepthwiseConv2D(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
                     uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height, int input_width,
                     BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    const small_hip_quant iq = input_buf.quant(), fq = filter_buf.quant(), oq = output_buf.quant();
    detail::raise<BufferT>(small_hip_depthwise_conv2d_u8(batch, kernel_height, kernel_width, stride, t_pad, b_pad,
                                                         l_pad, r_pad, input_channels, input_height, input_width,
                                                         input_buf.device_in(), &iq, filter_buf.device_in(), &fq,
                                                         output_buf.device_out(), &oq, detail::st()),
                           "DepthwiseConv2D");
}

template <class BufferT, detail::if_float<BufferT> = true>
void PartialDepthwiseConv2D(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad,
                            uint8_t b_pad, uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height,
                            int input_width, BufferT const &input_buf, BufferT const &filter_buf,
                            BufferT &output_buf)
{
    detail::raise<BufferT>(
        small_hip_partial_depthwise_conv2d_f32(batch, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad,
                                               r_pad, input_channels, input_height, input_width,
                                               input_buf.device_in(), filter_buf.device_in(),
                                               output_buf.device_out(), detail::st()),
        "PartialDepthwiseConv2D");
}

template <class BufferT, detail::if_float<BufferT> = true>
void DepthwiseConv2D_Bias_Act(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad,
                              uint8_t b_pad, uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height,
                              int input_width, BufferT const &input_buf, BufferT const &filter_buf,
                              BufferT const &bias_buf, ActivationType act, float negative_slope,
                              BufferT &output_buf)
{
    detail::raise<BufferT>(
        small_hip_depthwise_conv2d_bias_act_f32(batch, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad,
                                                r_pad, input_channels, input_height, input_width,
                                                input_buf.device_in(), filter_buf.device_in(),
                                                bias_buf.size() ? bias_buf.device_in() : nullptr, (int)act,
                                                negative_slope, output_buf.device_out(), detail::st()),
        "DepthwiseConv2D_Bias_Act");
}

// Conv2D [+ bias] [+ act] followed by DepthwiseConv2D [+ bias] [+ act] (the reference's Conv2D_*_DepthwiseConv2D_*
// family, fused_interface_abstract.hpp:1513-2500).  ONE launch (small_hip_conv2d_bias_act_dwconv2d_bias_act_f32: the
// convolution's output never goes to memory, inter_output_buf is not touched) for the pairs detail::conv_dw_one_launch
// names.  Any other pair: two launches through inter_output_buf, which ends up holding the whole first layer's output.
// Bias buffers may be empty.
template <class BufferT, detail::if_float<BufferT> = true>
void Conv2D_Bias_Act_DepthwiseConv2D_Bias_Act(
    int batch, int conv_kernel_height, int conv_kernel_width, int conv_stride, uint8_t conv_t_pad, uint8_t conv_b_pad,
    uint8_t conv_l_pad, uint8_t conv_r_pad, int dw_kernel_height, int dw_kernel_width, int dw_stride,
    uint8_t dw_t_pad, uint8_t dw_b_pad, uint8_t dw_l_pad, uint8_t dw_r_pad, int output_channels, int input_channels,
    int input_height, int input_width, BufferT const &input_buf, BufferT const &filter_buf, BufferT const &bias_buf,
    BufferT &inter_output_buf, BufferT const &dwise_filter_buf, BufferT const &dwise_bias_buf, ActivationType act,
    float negative_slope, BufferT &output_buf)
{
    if (detail::conv_dw_one_launch<BufferT>(batch, conv_kernel_height, conv_kernel_width, conv_stride, conv_t_pad, conv_b_pad, conv_l_pad,
                                            conv_r_pad, dw_kernel_height, dw_kernel_width, dw_stride, dw_t_pad, dw_b_pad, dw_l_pad,
                                            dw_r_pad, output_channels, input_channels, input_height, input_width))
    {
        detail::raise<BufferT>(
            small_hip_conv2d_bias_act_dwconv2d_bias_act_f32(
                batch, conv_kernel_height, conv_kernel_width, conv_stride, conv_t_pad, conv_b_pad, conv_l_pad, conv_r_pad, 3, 3,
                dw_stride, dw_t_pad, dw_b_pad, dw_l_pad, dw_r_pad, output_channels,
                input_channels, input_height, input_width, input_buf.device_in(), filter_buf.device_in(),
                bias_buf.size() ? bias_buf.device_in() : nullptr, dwise_filter_buf.device_in(),
                dwise_bias_buf.size() ? dwise_bias_buf.device_in() : nullptr, (int)act, negative_slope,
                output_buf.device_out(), detail::st()),
            "Conv2D_ReLU_DepthwiseConv2D_ReLU");
        return;
    }
    Conv2D_Bias_Act(batch, conv_kernel_height, conv_kernel_width, conv_stride, conv_t_pad, conv_b_pad, conv_l_pad,
                    conv_r_pad, output_channels, input_channels, input_height, input_width, input_buf, filter_buf,
                    bias_buf, act, negative_slope, inter_output_buf);
    const int Ho = (int)output_dim(input_height + conv_t_pad + conv_b_pad, conv_stride, conv_kernel_height);
    const int Wo = (int)output_dim(input_width + conv_l_pad + conv_r_pad, conv_stride, conv_kernel_width);
    DepthwiseConv2D_Bias_Act(batch, dw_kernel_height, dw_kernel_width, dw_stride, dw_t_pad, dw_b_pad, dw_l_pad,
                             dw_r_pad, output_channels, Ho, Wo, inter_output_buf, dwise_filter_buf, dwise_bias_buf,
                             act, negative_slope, output_buf);
}

// ---- pooling -----------------------------------------------------------------------------------------
template <class BufferT, detail::if_float<BufferT> = true>
void MaxPool2D(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
               uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height, int input_width,
               BufferT const &input_buf, BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_maxpool2d_f32(batch, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad,
                                                   r_pad, input_channels, input_height, input_width,
                                                   input_buf.device_in(), output_buf.device_out(), detail::st()),
                           "MaxPool2D");
}

template <class BufferT, detail::if_quint8<BufferT> = true>
void MaxPool2D(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
               uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height, int input_width,
               BufferT const &input_buf, BufferT &output_buf)
{
    const small_hip_quant iq = input_buf.quant(), oq = output_buf.quant();
    detail::raise<BufferT>(small_hip_maxpool2d_u8(batch, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad,
                                                  r_pad, input_channels, input_height, input_width,
                                                  input_buf.device_in(), &iq, output_buf.device_out(), &oq,
                                                  detail::st()),
                           "MaxPool2D");
}

template <class BufferT, detail::if_float<BufferT> = true>
void AveragePool2D(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
                   uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height, int input_width,
                   BufferT const &input_buf, BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_avgpool2d_f32(batch, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad,
                                                   r_pad, input_channels, input_height, input_width,
                                                   input_buf.device_in(), output_buf.device_out(), detail::st()),
                           "AveragePool2D");
}

template <class BufferT, detail::if_quint8<BufferT> = true>
void AveragePool2D(int batch, int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
                   uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height, int input_width,
                   BufferT const &input_buf, BufferT &output_buf)
{
    const small_hip_quant iq = input_buf.quant(), oq = output_buf.quant();
    detail::raise<BufferT>(small_hip_avgpool2d_u8(batch, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad,
                                                  r_pad, input_channels, input_height, input_width,
                                                  input_buf.device_in(), &iq, output_buf.device_out(), &oq,
                                                  detail::st()),
                           "AveragePool2D");
}

// ---- activations, accumulation, bias ------------------------------------------------------------------
template <class BufferT, detail::if_float<BufferT> = true>
void ReLUActivation(int batch, int input_channels, int input_height, int input_width, BufferT const &input_buf,
                    BufferT &output_buf)
{
    float const *in = input_buf.device_in();
    detail::raise<BufferT>(small_hip_relu_f32(batch, input_channels, input_height, input_width, in,
                                              output_buf.device_out(), detail::st()),
                           "ReLUActivation");
}

template <class BufferT, detail::if_quint8<BufferT> = true>
void ReLUActivation(int batch, int input_channels, int input_height, int input_width, BufferT const &input_buf,
                    BufferT &output_buf)
{
    const small_hip_quant iq = input_buf.quant(), oq = output_buf.quant();
    uint8_t const *in = input_buf.device_in();
    detail::raise<BufferT>(small_hip_relu_u8(batch, input_channels, input_height, input_width, in, &iq,
                                             output_buf.device_out(), &oq, detail::st()),
                           "ReLUActivation");
}

// the slope arrives as a one-element buffer, as in the reference's definition
// (interface_abstract.hpp:1616-1621)
template <class BufferT, detail::if_float<BufferT> = true>
void LeakyReLUActivation(int batch, int input_channels, int input_height, int input_width,
                         BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    const float slope = filter_buf.data()[0];
    float const *in = input_buf.device_in();
    detail::raise<BufferT>(small_hip_leaky_relu_f32(batch, input_channels, input_height, input_width, in, slope,
                                                    output_buf.device_out(), detail::st()),
                           "LeakyReLUActivation");
}

// Dropout at inference: a multiplication by filter_buf[0] (interface_abstract.hpp:1697-1726); float only
template <class BufferT, detail::if_float<BufferT> = true>
void Dropout(int batch, int input_channels, int input_height, int input_width, BufferT const &input_buf,
             BufferT const &filter_buf, BufferT &output_buf)
{
    const float scale = filter_buf.data()[0];
    float const *in = input_buf.device_in();
    detail::raise<BufferT>(small_hip_dropout_f32(batch, input_channels, input_height, input_width, in, scale,
                                                 output_buf.device_out(), detail::st()),
                           "Dropout");
}

// SoftMax over the whole tensor of each image (interface_abstract.hpp:1778-1832); float only
template <class BufferT, detail::if_float<BufferT> = true>
void SoftMax(int batch, int input_channels, int input_height, int input_width, BufferT const &input_buf,
             BufferT &output_buf)
{
    float const *in = input_buf.device_in();
    detail::raise<BufferT>(small_hip_softmax_f32(batch, input_channels, input_height, input_width, in,
                                                 output_buf.device_out(), detail::st()),
                           "SoftMax");
}

template <class BufferT, detail::if_float<BufferT> = true>
void Accum(int batch, int input_channels, int input_height, int input_width, BufferT const &input_buf,
           BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_accum_f32(batch, input_channels, input_height, input_width,
                                               input_buf.device_in(), output_buf.device_out(), detail::st()),
                           "Accum");
}

template <class BufferT, detail::if_quint8<BufferT> = true>
void Accum(int batch, int input_channels, int input_height, int input_width, BufferT const &input_buf,
           BufferT &output_buf)
{
    const small_hip_quant iq = input_buf.quant(), oq = output_buf.quant();
    detail::raise<BufferT>(small_hip_accum_u8(batch, input_channels, input_height, input_width,
                                              input_buf.device_in(), &iq, output_buf.device_out(), &oq,
                                              detail::st()),
                           "Accum");
}

template <class BufferT, detail::if_float<BufferT> = true>
void Bias(int batch, int num_channels, int output_height, int output_width, BufferT const &input_buf,
          BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_bias_f32(batch, num_channels, output_height, output_width,
                                              input_buf.device_in(), output_buf.device_out(), detail::st()),
                           "Bias");
}

template <class BufferT, detail::if_float<BufferT> = true>
void PartialBias(int batch, int num_channels, int output_height, int output_width, BufferT const &input_buf,
                 BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_partial_bias_f32(batch, num_channels, output_height, output_width,
                                                      input_buf.device_in(), output_buf.device_out(),
                                                      detail::st()),
                           "PartialBias");
}

// ---- UpSample2D, Concat, Dense ----------------------------------------------------------------------------
template <class BufferT, detail::if_float<BufferT> = true>
void UpSample2D(int batch, int scale_factor, int input_channels, int input_height, int input_width,
                BufferT const &input_buf, BufferT &output_buf)
{
    if (scale_factor == 1)
    {
        output_buf = input_buf;   // the reference copy-assigns the buffer (interface_abstract.hpp:1858-1861)
        return;
    }
    const int status = small_hip_upsample2d_f32(batch, scale_factor, input_channels, input_height, input_width,
                                                input_buf.device_in(), output_buf.device_out(), detail::st());
    detail::raise<BufferT>(status, "Upsample");
}

template <class BufferT>
void Concat(int batch, uint32_t input0_channels, uint32_t input1_channels, uint32_t input_height,
            uint32_t input_width, BufferT const &input0_buf, BufferT const &input1_buf, BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_concat(batch, input0_channels, input1_channels, input_height, input_width,
                                            input0_buf.device_in(), input1_buf.device_in(),
                                            output_buf.device_out(), sizeof(typename BufferT::value_type),
                                            detail::st()),
                           "Concat");
}

template <class BufferT, detail::if_float<BufferT> = true>
void Dense(int batch, int output_elements, int input_elements, BufferT const &input_buf,
           BufferT const &filter_buf, BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_dense_f32(batch, output_elements, input_elements, input_buf.device_in(),
                                               filter_buf.device_in(), output_buf.device_out(), detail::st()),
                           "Dense");
}

template <class BufferT, detail::if_quint8<BufferT> = true>
void Dense(int batch, int output_elements, int input_elements, BufferT const &input_buf,
           BufferT const &filter_buf, BufferT &output_buf)
{
    const small_hip_quant iq = input_buf.quant(), fq = filter_buf.quant(), oq = output_buf.quant();
    detail::raise<BufferT>(small_hip_dense_u8(batch, output_elements, input_elements, input_buf.device_in(), &iq,
                                              filter_buf.device_in(), &fq, output_buf.device_out(), &oq,
                                              detail::st()),
                           "Dense");
}

} // namespace batched

// =================================================================================================
// The reference's batch-1 signatures (interface.hpp:49-497)
// =================================================================================================
template <class BufferT>
void Conv2D(int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad, uint8_t l_pad,
            uint8_t r_pad, int output_channels, int input_channels, int input_height, int input_width,
            BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    batched::Conv2D(1, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad, output_channels,
                    input_channels, input_height, input_width, input_buf, filter_buf, output_buf);
}

template <class BufferT>
void PartialConv2D(int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad, uint8_t l_pad,
                   uint8_t r_pad, int output_channels, int input_channels, int input_height, int input_width,
                   BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    batched::PartialConv2D(1, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad, output_channels,
                           input_channels, input_height, input_width, input_buf, filter_buf, output_buf);
}

template <class BufferT>
void GroupConv2D(int kernel_height, int kernel_width, int stride, int output_groups, uint8_t t_pad, uint8_t b_pad,
                 uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height, int input_width,
                 BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    batched::GroupConv2D(1, kernel_height, kernel_width, stride, output_groups, t_pad, b_pad, l_pad, r_pad,
                         input_channels, input_height, input_width, input_buf, filter_buf, output_buf);
}

template <class BufferT>
void PartialGroupConv2D(int kernel_height, int kernel_width, int stride, int output_groups, uint8_t t_pad,
                        uint8_t b_pad, uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height,
                        int input_width, BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    batched::PartialGroupConv2D(1, kernel_height, kernel_width, stride, output_groups, t_pad, b_pad, l_pad, r_pad,
                                input_channels, input_height, input_width, input_buf, filter_buf, output_buf);
}

template <class BufferT>
void DepthwiseConv2D(int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
                     uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height, int input_width,
                     BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    batched::DepthwiseConv2D(1, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad, input_channels,
                             input_height, input_width, input_buf, filter_buf, output_buf);
}

template <class BufferT>
void PartialDepthwiseConv2D(int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
                            uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height, int input_width,
                            BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    batched::PartialDepthwiseConv2D(1, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad,
                                    input_channels, input_height, input_width, input_buf, filter_buf,
                                    output_buf);
}

template <class BufferT>
void MaxPool2D(int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad, uint8_t l_pad,
               uint8_t r_pad, int input_channels, int input_height, int input_width, BufferT const &input_buf,
               BufferT &output_buf)
{
    batched::MaxPool2D(1, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad, input_channels,
                       input_height, input_width, input_buf, output_buf);
}

template <class BufferT>
void AveragePool2D(int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad, uint8_t l_pad,
                   uint8_t r_pad, int input_channels, int input_height, int input_width,
                   BufferT const &input_buf, BufferT &output_buf)
{
    batched::AveragePool2D(1, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad, input_channels,
                           input_height, input_width, input_buf, output_buf);
}

template <typename BufferT>
void UpSample2D(int scale_factor, int input_channels, int input_height, int input_width,
                BufferT const &input_buf, BufferT &output_buf)
{
    batched::UpSample2D(1, scale_factor, input_channels, input_height, input_width, input_buf, output_buf);
}

template <class BufferT>
void ReLUActivation(int input_channels, int input_height, int input_width, BufferT const &input_buf,
                    BufferT &output_buf)
{
    batched::ReLUActivation(1, input_channels, input_height, input_width, input_buf, output_buf);
}

template <class BufferT>
void LeakyReLUActivation(int input_channels, int input_height, int input_width, BufferT const &input_buf,
                         BufferT const &filter_buf, BufferT &output_buf)
{
    batched::LeakyReLUActivation(1, input_channels, input_height, input_width, input_buf, filter_buf, output_buf);
}

template <class BufferT>
void Dropout(int input_channels, int input_height, int input_width, BufferT const &input_buf,
             BufferT const &filter_buf, BufferT &output_buf)
{
    batched::Dropout(1, input_channels, input_height, input_width, input_buf, filter_buf, output_buf);
}

template <class BufferT>
void SoftMax(int input_channels, int input_height, int input_width, BufferT const &input_buf, BufferT &output_buf)
{
    batched::SoftMax(1, input_channels, input_height, input_width, input_buf, output_buf);
}

template <class BufferT>
void Accum(int input_channels, int input_height, int input_width, BufferT const &input_buf, BufferT &output_buf)
{
    batched::Accum(1, input_channels, input_height, input_width, input_buf, output_buf);
}

template <class BufferT>
void Bias(int num_channels, int output_height, int output_width, BufferT const &input_buf, BufferT &output_buf)
{
    batched::Bias(1, num_channels, output_height, output_width, input_buf, output_buf);
}

template <class BufferT>
void PartialBias(int num_channels, int output_height, int output_width, BufferT const &input_buf,
                 BufferT &output_buf)
{
    batched::PartialBias(1, num_channels, output_height, output_width, input_buf, output_buf);
}

template <class BufferT>
void Concat(uint32_t input0_channels, uint32_t input1_channels, uint32_t input_height, uint32_t input_width,
            BufferT const &input0_buf, BufferT const &input1_buf, BufferT &output_buf)
{
    batched::Concat(1, input0_channels, input1_channels, input_height, input_width, input0_buf, input1_buf,
                    output_buf);
}

template <class BufferT>
void Dense(int output_elements, int input_elements, BufferT const &input_buf, BufferT const &filter_buf,
           BufferT &output_buf)
{
    batched::Dense(1, output_elements, input_elements, input_buf, filter_buf, output_buf);
}

// The reference's fused convolution + pooling functions (fused_interface_abstract.hpp:354, 998, 683), same
// signatures; inter_output_buf is only written when the pooling window cannot be fused.
template <class BufferT>
void Conv2D_Bias_ReLU_Maxpool2D(int conv_kernel_height, int conv_kernel_width, int conv_stride, uint8_t conv_t_pad,
                                uint8_t conv_b_pad, uint8_t conv_l_pad, uint8_t conv_r_pad, int pool_kernel_height,
                                int pool_kernel_width, int pool_stride, uint8_t pool_t_pad, uint8_t pool_b_pad,
                                uint8_t pool_l_pad, uint8_t pool_r_pad, int output_channels, int input_channels,
                                int input_height, int input_width, BufferT const &input_buf,
                                BufferT const &filter_buf, BufferT const &bias_buf, BufferT &inter_output_buf,
                                BufferT &output_buf)
{
    batched::Conv2D_Bias_Act_Maxpool2D(1, conv_kernel_height, conv_kernel_width, conv_stride, conv_t_pad, conv_b_pad,
                                       conv_l_pad, conv_r_pad, pool_kernel_height, pool_kernel_width, pool_stride,
                                       pool_t_pad, pool_b_pad, pool_l_pad, pool_r_pad, output_channels,
                                       input_channels, input_height, input_width, input_buf, filter_buf, bias_buf,
                                       RELU, 0.f, inter_output_buf, output_buf);
}

template <class BufferT>
void Conv2D_ReLU_Maxpool2D(int conv_kernel_height, int conv_kernel_width, int conv_stride, uint8_t conv_t_pad,
                           uint8_t conv_b_pad, uint8_t conv_l_pad, uint8_t conv_r_pad, int pool_kernel_height,
                           int pool_kernel_width, int pool_stride, uint8_t pool_t_pad, uint8_t pool_b_pad,
                           uint8_t pool_l_pad, uint8_t pool_r_pad, int output_channels, int input_channels,
                           int input_height, int input_width, BufferT const &input_buf, BufferT const &filter_buf,
                           BufferT &inter_output_buf, BufferT &output_buf)
{
    batched::Conv2D_Bias_Act_Maxpool2D(1, conv_kernel_height, conv_kernel_width, conv_stride, conv_t_pad, conv_b_pad,
                                       conv_l_pad, conv_r_pad, pool_kernel_height, pool_kernel_width, pool_stride,
                                       pool_t_pad, pool_b_pad, pool_l_pad, pool_r_pad, output_channels,
                                       input_channels, input_height, input_width, input_buf, filter_buf, BufferT(),
                                       RELU, 0.f, inter_output_buf, output_buf);
}

template <class BufferT>
void Conv2D_Maxpool2D(int conv_kernel_height, int conv_kernel_width, int conv_stride, uint8_t conv_t_pad,
                      uint8_t conv_b_pad, uint8_t conv_l_pad, uint8_t conv_r_pad, int pool_kernel_height,
                      int pool_kernel_width, int pool_stride, uint8_t pool_t_pad, uint8_t pool_b_pad,
                      uint8_t pool_l_pad, uint8_t pool_r_pad, int output_channels, int input_channels,
                      int input_height, int input_width, BufferT const &input_buf, BufferT const &filter_buf,
                      BufferT &inter_output_buf, BufferT &output_buf)
{
    batched::Conv2D_Bias_Act_Maxpool2D(1, conv_kernel_height, conv_kernel_width, conv_stride, conv_t_pad, conv_b_pad,
                                       conv_l_pad, conv_r_pad, pool_kernel_height, pool_kernel_width, pool_stride,
                                       pool_t_pad, pool_b_pad, pool_l_pad, pool_r_pad, output_channels,
                                       input_channels, input_height, input_width, input_buf, filter_buf, BufferT(),
                                       NONE, 0.f, inter_output_buf, output_buf);
}

// The reference's single-layer "fused" functions (fused_interface_abstract.hpp:55, 217, 1332, 1419): one launch.
template <class BufferT>
void Conv2D_ReLU(int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad, uint8_t l_pad,
                 uint8_t r_pad, int output_channels, int input_channels, int input_height, int input_width,
                 BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    batched::Conv2D_Bias_Act(1, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad, output_channels,
                             input_channels, input_height, input_width, input_buf, filter_buf, BufferT(), RELU, 0.f,
                             output_buf);
}

template <class BufferT>
void Conv2D_Bias_ReLU(int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad, uint8_t l_pad,
                      uint8_t r_pad, int output_channels, int input_channels, int input_height, int input_width,
                      BufferT const &input_buf, BufferT const &filter_buf, BufferT const &bias_buf,
                      BufferT &output_buf)
{
    batched::Conv2D_Bias_Act(1, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad, output_channels,
                             input_channels, input_height, input_width, input_buf, filter_buf, bias_buf, RELU, 0.f,
                             output_buf);
}

template <class BufferT>
void DepthwiseConv2D_ReLU(int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
                          uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height, int input_width,
                          BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    batched::DepthwiseConv2D_Bias_Act(1, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad,
                                      input_channels, input_height, input_width, input_buf, filter_buf, BufferT(),
                                      RELU, 0.f, output_buf);
}

template <class BufferT>
void DepthwiseConv2D_Bias_ReLU(int kernel_height, int kernel_width, int stride, uint8_t t_pad, uint8_t b_pad,
                               uint8_t l_pad, uint8_t r_pad, int input_channels, int input_height, int input_width,
                               BufferT const &input_buf, BufferT const &filter_buf, BufferT const &bias_buf,
                               BufferT &output_buf)
{
    batched::DepthwiseConv2D_Bias_Act(1, kernel_height, kernel_width, stride, t_pad, b_pad, l_pad, r_pad,
                                      input_channels, input_height, input_width, input_buf, filter_buf, bias_buf,
                                      RELU, 0.f, output_buf);
}

// The reference's convolution + depthwise convolution functions (fused_interface_abstract.hpp:1513, 1840, 2170),
// same signatures (the reference names the depthwise window "pool_*").
template <class BufferT>
void Conv2D_DepthwiseConv2D(int conv_kernel_height, int conv_kernel_width, int conv_stride, uint8_t conv_t_pad,
                            uint8_t conv_b_pad, uint8_t conv_l_pad, uint8_t conv_r_pad, int pool_kernel_height,
                            int pool_kernel_width, int pool_stride, uint8_t pool_t_pad, uint8_t pool_b_pad,
                            uint8_t pool_l_pad, uint8_t pool_r_pad, int output_channels, int input_channels,
                            int input_height, int input_width, BufferT const &input_buf, BufferT const &filter_buf,
                            BufferT &inter_output_buf, BufferT const &dwise_filter_buf, BufferT &output_buf)
{
    batched::Conv2D_Bias_Act_DepthwiseConv2D_Bias_Act(
        1, conv_kernel_height, conv_kernel_width, conv_stride, conv_t_pad, conv_b_pad, conv_l_pad, conv_r_pad,
        pool_kernel_height, pool_kernel_width, pool_stride, pool_t_pad, pool_b_pad, pool_l_pad, pool_r_pad,
        output_channels, input_channels, input_height, input_width, input_buf, filter_buf, BufferT(),
        inter_output_buf, dwise_filter_buf, BufferT(), NONE, 0.f, output_buf);
}

template <class BufferT>
void Conv2D_ReLU_DepthwiseConv2D_ReLU(int conv_kernel_height, int conv_kernel_width, int conv_stride,
                                      uint8_t conv_t_pad, uint8_t conv_b_pad, uint8_t conv_l_pad, uint8_t conv_r_pad,
                                      int pool_kernel_height, int pool_kernel_width, int pool_stride,
                                      uint8_t pool_t_pad, uint8_t pool_b_pad, uint8_t pool_l_pad, uint8_t pool_r_pad,
                                      int output_channels, int input_channels, int input_height, int input_width,
                                      BufferT const &input_buf, BufferT const &filter_buf, BufferT &inter_output_buf,
                                      BufferT const &dwise_filter_buf, BufferT &output_buf)
{
    batched::Conv2D_Bias_Act_DepthwiseConv2D_Bias_Act(
        1, conv_kernel_height, conv_kernel_width, conv_stride, conv_t_pad, conv_b_pad, conv_l_pad, conv_r_pad,
        pool_kernel_height, pool_kernel_width, pool_stride, pool_t_pad, pool_b_pad, pool_l_pad, pool_r_pad,
        output_channels, input_channels, input_height, input_width, input_buf, filter_buf, BufferT(),
        inter_output_buf, dwise_filter_buf, BufferT(), RELU, 0.f, output_buf);
}

template <class BufferT>
void Conv2D_Bias_ReLU_DepthwiseConv2D_Bias_ReLU(
    int conv_kernel_height, int conv_kernel_width, int conv_stride, uint8_t conv_t_pad, uint8_t conv_b_pad,
    uint8_t conv_l_pad, uint8_t conv_r_pad, int pool_kernel_height, int pool_kernel_width, int pool_stride,
    uint8_t pool_t_pad, uint8_t pool_b_pad, uint8_t pool_l_pad, uint8_t pool_r_pad, int output_channels,
    int input_channels, int input_height, int input_width, BufferT const &input_buf, BufferT const &filter_buf,
    BufferT const &bias_buf, BufferT &inter_output_buf, BufferT const &dwise_filter_buf,
    BufferT const &dwise_bias_buf, BufferT &output_buf)
{
    batched::Conv2D_Bias_Act_DepthwiseConv2D_Bias_Act(
        1, conv_kernel_height, conv_kernel_width, conv_stride, conv_t_pad, conv_b_pad, conv_l_pad, conv_r_pad,
        pool_kernel_height, pool_kernel_width, pool_stride, pool_t_pad, pool_b_pad, pool_l_pad, pool_r_pad,
        output_channels, input_channels, input_height, input_width, input_buf, filter_buf, bias_buf,
        inter_output_buf, dwise_filter_buf, dwise_bias_buf, RELU, 0.f, output_buf);
}

// small::Dense exactly as the reference writes it (interface_abstract.hpp:2113-2132):
// output[o * Ni + i] = input[o * Ni + i] * filter[o]
template <class BufferT, detail::if_float<BufferT> = true>
void DenseAsWritten(int output_elements, int input_elements, BufferT const &input_buf,
                    BufferT const &filter_buf, BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_dense_literal_f32(output_elements, input_elements, input_buf.device_in(),
                                                       filter_buf.device_in(), output_buf.device_out(),
                                                       detail::st()),
                           "Dense");
}

} // namespace small
