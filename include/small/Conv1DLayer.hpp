// Conv1DLayer: 1-D convolution over the rows of a [batch][C][rows][W] tensor with constant weights, optional
// bias, folded batch normalisation and activation (same constructors, checks and messages as the
// reference's include/small/Conv1DLayer.hpp:27-755; filters are [Co][Ci][kernel_width]).
//
// What differs underneath: compute_output() is one launch (bias + convolution + activation), where the
// reference issues Bias, PartialConv1D and the activation (Conv1DLayer.hpp:666-724); the batch extent of the
// shape is honoured; 1- and 2-channel inputs are accepted like 3.  The rows are the HEIGHT extent, as in
// the reference; more than one row needs stride 1 (small/interface_1D.hpp).
#pragma once

#include "Conv2DLayer.hpp"

namespace small
{

template <typename BufferT>
class Conv1DLayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    Conv1DLayer(shape_type const &input_shape, uint32_t kernel_width, uint32_t stride, PaddingEnum padding_type,
                uint32_t num_output_channels, BufferT const &filters, bool buffers_are_packed = true,
                ActivationType activation_type = NONE, float leaky_slope = 1.e-2)
        : Conv1DLayer(input_shape, kernel_width, stride, padding_type, num_output_channels, filters, BufferT(),
                      BufferT(), BufferT(), BufferT(), BufferT(), 0.f, buffers_are_packed, activation_type,
                      leaky_slope)
    {
    }

    Conv1DLayer(shape_type const &input_shape, uint32_t kernel_width, uint32_t stride, PaddingEnum padding_type,
                uint32_t num_output_channels, BufferT const &filters, BufferT const &bias,
                bool buffers_are_packed = true, ActivationType activation_type = NONE, float leaky_slope = 1.e-2)
        : Conv1DLayer(input_shape, kernel_width, stride, padding_type, num_output_channels, filters, bias, BufferT(),
                      BufferT(), BufferT(), BufferT(), 0.f, buffers_are_packed, activation_type, leaky_slope)
    {
    }

    Conv1DLayer(shape_type const &input_shape, uint32_t kernel_width, uint32_t stride, PaddingEnum padding_type,
                uint32_t num_output_channels, BufferT const &filters, BufferT const &bn_weight,
                BufferT const &bn_bias, BufferT const &bn_running_mean, BufferT const &bn_running_variance,
                float const &bn_eps = 1.e-5, bool buffers_are_packed = true, ActivationType activation_type = NONE,
                float leaky_slope = 1.e-2)
        : Conv1DLayer(input_shape, kernel_width, stride, padding_type, num_output_channels, filters, BufferT(),
                      bn_weight, bn_bias, bn_running_mean, bn_running_variance, bn_eps, buffers_are_packed,
                      activation_type, leaky_slope)
    {
    }

    Conv1DLayer(shape_type const &input_shape, uint32_t kernel_width, uint32_t stride, PaddingEnum padding_type,
                uint32_t num_output_channels, BufferT const &filters, BufferT const &bias, BufferT const &bn_weight,
                BufferT const &bn_bias, BufferT const &bn_running_mean, BufferT const &bn_running_variance,
                float const &bn_eps = 1.e-5, bool buffers_are_packed = true, ActivationType activation_type = NONE,
                float leaky_slope = 1.e-2)
        : Layer<BufferT>(),
          m_input_shape(input_shape),
          m_kernel_width(kernel_width),
          m_stride(stride),
          m_effective_output_channels(num_output_channels),
          m_activation_type(activation_type),
          m_slope(leaky_slope),
          m_l_pad(0),
          m_r_pad(0)
    {
        static_assert(std::is_same<BufferT, FloatBuffer>::value, "Conv1DLayer is a float32 layer");
        if ((input_shape[CHANNEL] % BufferT::C_ib) != 0 && (input_shape[CHANNEL] == 0 || input_shape[CHANNEL] > 3))
            throw std::invalid_argument("Conv1DLayer::ctor ERROR: invalid number of input channels.");
        uint32_t Co = num_output_channels;
        if (Co % BufferT::C_ob != 0)
        {
            if (buffers_are_packed)
                throw std::invalid_argument("Conv1DLayer::ctor ERROR: invalid number of output channels.");
            Co += BufferT::C_ob - Co % BufferT::C_ob;
        }
        size_t Wo = 0;
        compute_padding_output_dim(input_shape[WIDTH], kernel_width, stride, padding_type, m_l_pad, m_r_pad, Wo);
        this->set_output_shape({input_shape[BATCH], Co, input_shape[HEIGHT], Wo});
        detail::build_conv_weights("*Conv1DLayer", false, Co, m_effective_output_channels,
                                   (uint32_t)input_shape[CHANNEL], 1U, kernel_width, filters, bias,
                                   detail::BatchNormRefs<BufferT>{bn_weight, bn_bias, bn_running_mean,
                                                                  bn_running_variance, bn_eps},
                                   buffers_are_packed, m_packed_filters, m_packed_bias, /*conv1d_folding*/ true);
    }

    virtual ~Conv1DLayer() {}

    uint32_t get_effective_output_channels() const { return m_effective_output_channels; }

    virtual void compute_output(std::vector<Tensor<BufferT> const *> input, Tensor<BufferT> *output) const
    {
        this->check_single_input("Conv1DLayer", input, m_input_shape, output);
        auto const &os = this->output_shape();
        batched::Conv1D_Bias_Act((int)m_input_shape[BATCH], (int)m_kernel_width, (int)m_stride, m_l_pad, m_r_pad,
                                 (int)os[CHANNEL], (int)m_input_shape[CHANNEL], (int)m_input_shape[HEIGHT],
                                 (int)m_input_shape[WIDTH], input[0]->buffer(), m_packed_filters, m_packed_bias,
                                 detail::fused_act(m_activation_type), m_slope, output->buffer());
        detail::softmax_in_place(m_activation_type, os, output->buffer());
        output->set_shape(os);
    }

private:
    shape_type const m_input_shape;
    uint32_t const m_kernel_width;
    uint32_t const m_stride;
    uint32_t const m_effective_output_channels;
    ActivationType const m_activation_type;
    float const m_slope;
    uint8_t m_l_pad, m_r_pad;
    BufferT m_packed_filters;
    BufferT m_packed_bias;
};

} // namespace small
