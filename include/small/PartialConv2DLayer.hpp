// PartialConv2DLayer: output += convolution(input), then bias and activation (residual branches;
// same constructors, checks and messages as the reference's
// include/small/PartialConv2DLayer.hpp:27-572).
//
// float: one launch, out = act((out + conv(in)) + bias) (small_hip_partial_conv2d_bias_act_f32), where
// the reference issues PartialConv2D, PartialBias and the activation separately (:424-462).
// uint8: the reference's PartialConv2D<QUInt8Buffer> re-reads the output bytes as int32 partial sums
// (q_abstract_layer.hpp:302-305), which is not a residual add.  Here the layer is defined as
//     out = ReLU?( Accum( Conv2D(in), out ) ),   Accum(I, O) = requant_O((I + zI) + (O + zO))
// with the convolution written to a scratch tensor of the layer (quantisation fields of `out`):
// no counterpart in the reference.
#pragma once

#include "Conv2DLayer.hpp"   // detail::build_conv_weights

namespace small
{

template <typename BufferT>
class PartialConv2DLayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    PartialConv2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width,
                       uint32_t stride, PaddingEnum padding_type, uint32_t num_output_channels,
                       BufferT const &filters, bool buffers_are_packed = true,
                       ActivationType activation_type = NONE, float leaky_slope = 1.e-2)
        : PartialConv2DLayer(input_shape, kernel_height, kernel_width, stride, padding_type, num_output_channels,
                             filters, BufferT(), BufferT(), BufferT(), BufferT(), BufferT(), 0.f,
                             buffers_are_packed, activation_type, leaky_slope)
    {
    }

    PartialConv2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width,
                       uint32_t stride, PaddingEnum padding_type, uint32_t num_output_channels,
                       BufferT const &filters, BufferT const &bias, bool buffers_are_packed = true,
                       ActivationType activation_type = NONE, float leaky_slope = 1.e-2)
        : PartialConv2DLayer(input_shape, kernel_height, kernel_width, stride, padding_type, num_output_channels,
                             filters, bias, BufferT(), BufferT(), BufferT(), BufferT(), 0.f, buffers_are_packed,
                             activation_type, leaky_slope)
    {
    }

    PartialConv2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width,
                       uint32_t stride, PaddingEnum padding_type, uint32_t num_output_channels,
                       BufferT const &filters, BufferT const &bn_weight, BufferT const &bn_bias,
                       BufferT const &bn_running_mean, BufferT const &bn_running_variance,
                       float const &bn_eps = 1.e-5, bool buffers_are_packed = true,
                       ActivationType activation_type = NONE, float leaky_slope = 1.e-2)
        : PartialConv2DLayer(input_shape, kernel_height, kernel_width, stride, padding_type, num_output_channels,
                             filters, BufferT(), bn_weight, bn_bias, bn_running_mean, bn_running_variance, bn_eps,
                             buffers_are_packed, activation_type, leaky_slope)
    {
    }

    PartialConv2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width,
                       uint32_t stride, PaddingEnum padding_type, uint32_t num_output_channels,
                       BufferT const &filters, BufferT const &bias, BufferT const &bn_weight,
                       BufferT const &bn_bias, BufferT const &bn_running_mean, BufferT const &bn_running_variance,
                       float const &bn_eps = 1.e-5, bool buffers_are_packed = true,
                       ActivationType activation_type = NONE, float leaky_slope = 1.e-2)
        : Layer<BufferT>(),
          m_input_shape(input_shape),
          m_window(input_shape, kernel_height, kernel_width, stride, padding_type),
          m_activation_type(activation_type),
          m_slope(leaky_slope)
    {
        // 1 and 2 input channels are accepted like 3: small::Conv2D takes all three (the reference's layer
        // class only lets 3 through)
        if ((input_shape[CHANNEL] % BufferT::C_ib) != 0 && (input_shape[CHANNEL] == 0 || input_shape[CHANNEL] > 3))
            throw std::invalid_argument("PartialConv2DLayer::ctor ERROR: invalid number of input channels.");
        if ((num_output_channels % BufferT::C_ob) != 0)
            throw std::invalid_argument("PartialConv2DLayer::ctor ERROR: invalid number of output channels.");
        this->set_output_shape({input_shape[BATCH], num_output_channels, m_window.Ho, m_window.Wo});
        detail::build_conv_weights("*Conv2DLayer", false, num_output_channels, num_output_channels,
                                   (uint32_t)input_shape[CHANNEL], kernel_height, kernel_width, filters, bias,
                                   detail::BatchNormRefs<BufferT>{bn_weight, bn_bias, bn_running_mean,
                                                                  bn_running_variance, bn_eps},
                                   buffers_are_packed, m_packed_filters, m_packed_bias);
        if constexpr (std::is_same<BufferT, QUInt8Buffer>::value)
        {
            if (m_packed_bias.size() > 0 || activation_type == LEAKY || activation_type == SOFTMAX)
                throw std::invalid_argument(
                    "PartialConv2DLayer::ctor ERROR: bias / LeakyReLU / SoftMax have no quantised implementation.");
            m_scratch = BufferT(this->output_size());
        }
        m_prepared.build(kernel_height, kernel_width, num_output_channels, (uint32_t)input_shape[CHANNEL],
                         m_packed_filters);
    }

    virtual ~PartialConv2DLayer() {}

    BufferT const &get_packed_filters() const { return m_packed_filters; }
    BufferT const &get_packed_bias() const { return m_packed_bias; }

    virtual bool one_launch(small_hip_qlayer &d) const
    {
        if constexpr (std::is_same<BufferT, QUInt8Buffer>::value)
        {
            if (m_activation_type != NONE && m_activation_type != RELU) return false;
            auto const &os = this->output_shape();
            d.kind = SMALL_HIP_QL_CONV;
            d.accum_src = Layer<BufferT>::ONE_LAUNCH_ACCUM_ONTO_OUTPUT;
            d.relu = m_activation_type == RELU;
            d.kernel_height = (int)m_window.kh; d.kernel_width = (int)m_window.kw; d.stride = (int)m_window.stride;
            d.t_pad = m_window.t; d.b_pad = m_window.b; d.l_pad = m_window.l; d.r_pad = m_window.r;
            d.output_channels = (int)os[CHANNEL]; d.input_channels = (int)m_input_shape[CHANNEL];
            d.input_height = (int)m_input_shape[HEIGHT]; d.input_width = (int)m_input_shape[WIDTH];
            d.filter = m_packed_filters.device_in();
            d.filter_q = m_packed_filters.quant();
            return true;
        }
        else
            return false;
    }

    virtual void compute_output(std::vector<Tensor<BufferT> const *> input, Tensor<BufferT> *output) const
    {
        this->check_single_input("PartialConv2DLayer", input, m_input_shape, output);
        auto const &os = this->output_shape();
        const int batch = (int)m_input_shape[BATCH];
        const int Co = (int)os[CHANNEL], Ci = (int)m_input_shape[CHANNEL];
        const int H = (int)m_input_shape[HEIGHT], W = (int)m_input_shape[WIDTH];
        if constexpr (std::is_same<BufferT, FloatBuffer>::value)
        {
            batched::PartialConv2D_Bias_Act(batch, m_window.kh, m_window.kw, m_window.stride, m_window.t,
                                            m_window.b, m_window.l, m_window.r, Co, Ci, H, W, input[0]->buffer(),
                                            m_packed_filters, m_packed_bias, detail::fused_act(m_activation_type), m_slope,
                                            output->buffer());
        }
        else
        {
            // the scratch takes the output's quantisation, so that Conv2D requantises as a plain
            // Conv2DLayer writing `output` would
            detail::copy_quant(output->buffer(), m_scratch);
            batched::Conv2D_Accum_ReLU(batch, m_window.kh, m_window.kw, m_window.stride, m_window.t, m_window.b,
                                       m_window.l, m_window.r, Co, Ci, H, W, input[0]->buffer(), m_packed_filters,
                                       m_prepared.get(), (BufferT const *)nullptr, false, m_scratch);
            batched::Accum(batch, Co, (int)os[HEIGHT], (int)os[WIDTH], m_scratch, output->buffer());
            if (m_activation_type == RELU)
                batched::ReLUActivation(batch, Co, (int)os[HEIGHT], (int)os[WIDTH], output->buffer(),
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
    detail::PreparedFilter m_prepared;
    mutable BufferT m_scratch;    // quantised path only
};

} // namespace small
