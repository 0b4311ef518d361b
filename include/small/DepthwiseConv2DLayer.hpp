// DepthwiseConv2DLayer: depthwise convolution with constant weights, optional bias, folded batch
// normalisation and activation (same constructors, accessors, checks and messages as the
// reference's include/small/DepthwiseConv2DLayer.hpp:27-765).  compute_output() is one launch
// (bias + depthwise convolution + activation, small_hip_depthwise_conv2d_bias_act_f32) where the
// reference issues Bias, PartialDepthwiseConv2D and the activation (:681-730); the batch extent of
// the input shape is honoured.
#pragma once

#include "Conv2DLayer.hpp"   // detail::build_conv_weights

namespace small
{

template <typename BufferT>
class DepthwiseConv2DLayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    DepthwiseConv2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width,
                         uint32_t stride, PaddingEnum padding_type, BufferT const &filters,
                         bool buffers_are_packed = true, ActivationType activation_type = NONE,
                         float leaky_slope = 1.e-2)
        : DepthwiseConv2DLayer(input_shape, kernel_height, kernel_width, stride, padding_type, filters, BufferT(),
                               BufferT(), BufferT(), BufferT(), BufferT(), 0.f, buffers_are_packed, activation_type,
                               leaky_slope)
    {
    }

    DepthwiseConv2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width,
                         uint32_t stride, PaddingEnum padding_type, BufferT const &filters, BufferT const &bias,
                         bool buffers_are_packed = true, ActivationType activation_type = NONE,
                         float leaky_slope = 1.e-2)
        : DepthwiseConv2DLayer(input_shape, kernel_height, kernel_width, stride, padding_type, filters, bias,
                               BufferT(), BufferT(), BufferT(), BufferT(), 0.f, buffers_are_packed, activation_type,
                               leaky_slope)
    {
    }

    DepthwiseConv2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width,
                         uint32_t stride, PaddingEnum padding_type, BufferT const &filters,
                         BufferT const &bn_weight, BufferT const &bn_bias, BufferT const &bn_running_mean,
                         BufferT const &bn_running_variance, float const &bn_eps = 1.e-3,
                         bool buffers_are_packed = true, ActivationType activation_type = NONE,
                         float leaky_slope = 1.e-2)
        : DepthwiseConv2DLayer(input_shape, kernel_height, kernel_width, stride, padding_type, filters, BufferT(),
                               bn_weight, bn_bias, bn_running_mean, bn_running_variance, bn_eps, buffers_are_packed,
                               activation_type, leaky_slope)
    {
    }

    DepthwiseConv2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width,
                         uint32_t stride, PaddingEnum padding_type, BufferT const &filters, BufferT const &bias,
                         BufferT const &bn_weight, BufferT const &bn_bias, BufferT const &bn_running_mean,
                         BufferT const &bn_running_variance, float const &bn_eps = 1.e-3,
                         bool buffers_are_packed = true, ActivationType activation_type = NONE,
                         float leaky_slope = 1.e-2)
        : Layer<BufferT>(),
          m_input_shape(input_shape),
          m_window(input_shape, kernel_height, kernel_width, stride, padding_type),
          m_activation_type(activation_type),
          m_slope(leaky_slope)
    {
        if ((input_shape[CHANNEL] % BufferT::C_ib) != 0)
            throw std::invalid_argument("DepthwiseConv2DLayer::ctor ERROR: invalid number of input channels.");
        const uint32_t C = (uint32_t)input_shape[CHANNEL];
        this->set_output_shape({input_shape[BATCH], C, m_window.Ho, m_window.Wo});
        detail::build_conv_weights("DepthwiseConv2DLayer", true, C, C, 1U, kernel_height, kernel_width, filters,
                                   bias,
                                   detail::BatchNormRefs<BufferT>{bn_weight, bn_bias, bn_running_mean,
                                                                  bn_running_variance, bn_eps},
                                   buffers_are_packed, m_packed_filters, m_packed_bias);
        if constexpr (std::is_same<BufferT, QUInt8Buffer>::value)
        {
            if (m_packed_bias.size() > 0 || activation_type == LEAKY || activation_type == SOFTMAX)
                throw std::invalid_argument(
                    "DepthwiseConv2DLayer::ctor ERROR: bias / LeakyReLU / SoftMax have no quantised implementation.");
        }
    }

    virtual ~DepthwiseConv2DLayer() {}

    BufferT const &get_packed_filters() const { return m_packed_filters; }
    BufferT const &get_packed_bias() const { return m_packed_bias; }
    detail::Window const &window() const { return m_window; }
    ActivationType activation() const { return m_activation_type; }
    float slope() const { return m_slope; }


    virtual bool one_launch(small_hip_flayer &d) const
    {
        if constexpr (std::is_same<BufferT, FloatBuffer>::value)
        {
            if (m_activation_type == SOFTMAX) return false;
            d.kind = SMALL_HIP_FL_DWCONV;
            d.act = detail::fused_act(m_activation_type);
            d.slope = m_slope;
            d.kernel_height = (int)m_window.kh; d.kernel_width = (int)m_window.kw; d.stride = (int)m_window.stride;
            d.t_pad = m_window.t; d.b_pad = m_window.b; d.l_pad = m_window.l; d.r_pad = m_window.r;
            d.output_channels = (int)this->output_shape()[CHANNEL]; d.input_channels = (int)m_input_shape[CHANNEL];
            d.input_height = (int)m_input_shape[HEIGHT]; d.input_width = (int)m_input_shape[WIDTH];
            d.filter = m_packed_filters.device_in();
            d.bias = m_packed_bias.size() > 0 ? m_packed_bias.device_in() : nullptr;
            return true;
        }
        else
            return false;
    }

    virtual void compute_output(std::vector<Tensor<BufferT> const *> input, Tensor<BufferT> *output) const
    {
        this->check_single_input("DepthwiseConv2DLayer", input, m_input_shape, output);
        auto const &os = this->output_shape();
        const int batch = (int)m_input_shape[BATCH];
        const int C = (int)m_input_shape[CHANNEL], H = (int)m_input_shape[HEIGHT], W = (int)m_input_shape[WIDTH];
        if constexpr (std::is_same<BufferT, FloatBuffer>::value)
        {
            batched::DepthwiseConv2D_Bias_Act(batch, m_window.kh, m_window.kw, m_window.stride, m_window.t,
                                              m_window.b, m_window.l, m_window.r, C, H, W, input[0]->buffer(),
                                              m_packed_filters, m_packed_bias, detail::fused_act(m_activation_type), m_slope,
                                              output->buffer());
        }
        else
        {
            batched::DepthwiseConv2D(batch, m_window.kh, m_window.kw, m_window.stride, m_window.t, m_window.b,
                                     m_window.l, m_window.r, C, H, W, input[0]->buffer(), m_packed_filters,
                                     output->buffer());
            if (m_activation_type == RELU)
                batched::ReLUActivation(batch, C, (int)os[HEIGHT], (int)os[WIDTH], output->buffer(),
                                        output->buffer());
        }
        detail::softmax_in_place(m_activation_type, os, output->buffer());
        output->set_shape(os);
    }

private:
    shape_type const m_input_shape;
    detail::Window const m_window;
    ActivationType const m_activation_type;
    float const m_slope;
    BufferT m_packed_filters;
    BufferT m_packed_bias;
};

} // namespace small
