// Conv2DLayer: convolution with constant weights, optional bias, folded batch normalisation and
// activation (same constructors, accessors, checks and messages as the reference's
// include/small/Conv2DLayer.hpp:27-916).
//
// What differs underneath:
//   - compute_output() is ONE launch: bias + convolution + activation fused
//     (small_hip_conv2d_bias_act_f32), where the reference issues Bias, PartialConv2D and the
//     activation as three passes over the output (Conv2DLayer.hpp:827-879);
//   - the batch extent of the input shape is honoured (N packed images per call);
//   - unpacked filters are packed on the device; on the quantised path the filter is also brought
//     into the kernel's operand order once, at construction.
#pragma once

#include <algorithm>
#include <cmath>

#include "Layer.hpp"

namespace small
{

namespace detail
{

// the quantisation fields travel with a QUInt8Buffer's data; a float buffer has none
inline void copy_quant(QUInt8Buffer const &from, QUInt8Buffer &to)
{
    to.scale = from.scale;
    to.offset = from.offset;
    to.multiplier = from.multiplier;
    to.lshift = from.lshift;
    to.rshift = from.rshift;
    to.m_zero = from.m_zero;
    to.min_val = from.min_val;
    to.max_val = from.max_val;
    to.b = from.b;
}
inline void copy_quant(FloatBuffer const &, FloatBuffer &) {}

// batch-normalisation statistics handed to a constructor; all four empty = none
template <class BufferT>
struct BatchNormRefs
{
    BufferT const &weight, &bias, &mean, &variance;
    float eps;
    bool any() const { return weight.size() || bias.size() || mean.size() || variance.size(); }
    bool all_sized(size_t n) const
    {
        return weight.size() == n && bias.size() == n && mean.size() == n && variance.size() == n;
    }
};

// Fills packed_filters ([Co/16][Ci/cib][kh][kw][cib][16], Co = num_output_channels, rows past
// num_effective_output_channels zero) and packed_bias (empty, or Co long) from the caller's buffers and
// folds the batch normalisation into both:
//     scale = gamma / sqrt(var + eps);  filter[co] *= scale;
//     bias[co] = beta - mean * scale               (no bias given)
//              = beta + scale * (bias[co] - mean)  (bias given)
// (conv1d_folding: scale = gamma / sqrt(var + eps), bias = scale * bias + beta - mean * scale, as Conv1DLayer.hpp does)
// the reference's initialize_conv2d_buffers (Conv2DLayer.hpp:135-341) with the same float expressions.
// `who` is the message prefix ("*Conv2DLayer" there).  Depthwise filters: num_input_channels = 1 and
// depthwise = true (tensor type FILTER_DW).
template <class BufferT>
void build_conv_weights(std::string const &who, bool depthwise, uint32_t num_output_channels,
                        uint32_t num_effective_output_channels, uint32_t num_input_channels, uint32_t kernel_height,
                        uint32_t kernel_width, BufferT const &filters, BufferT const &bias,
                        BatchNormRefs<BufferT> const &bn, bool buffers_are_packed, BufferT &packed_filters,
                        BufferT &packed_bias, bool conv1d_folding = false)
{
    typedef typename BufferT::value_type T;
    const size_t taps = (size_t)num_input_channels * kernel_height * kernel_width;
    if (filters.size() != num_effective_output_channels * taps)
        throw std::invalid_argument(who + "::ctor ERROR: filters buffer is incorrect size.");
    const size_t packed_size = (size_t)num_output_channels * taps;
    const BufferTypeEnum ftype = depthwise ? FILTER_DW : FILTER_CONV;
    const uint32_t cib = depthwise ? 1U : BufferT::C_ib;

    if (buffers_are_packed)
    {
        if (num_output_channels != num_effective_output_channels)
            throw std::invalid_argument("Conv2DLayer::ctor error: invalid number of output channels.");
        packed_filters = filters;
    }
    else
    {
        // zero rows up to the padded channel count, then one pack on the device
        BufferT flat(packed_size);
        T *f = flat.data();
        std::copy(filters.data(), filters.data() + filters.size(), f);
        std::fill(f + filters.size(), f + packed_size, T(0));
        BufferT packed(packed_size);
        pack_buffer(flat, ftype, num_output_channels, num_input_channels, kernel_height, kernel_width, BufferT::C_ib,
                    BufferT::C_ob, packed);
        packed_filters = std::move(packed);
        copy_quant(filters, packed_filters);   // the packed copy keeps the filter's zero point
    }

    if (bias.size() > 0)
    {
        if (bias.size() != num_effective_output_channels)
            throw std::invalid_argument(who + "::ctor ERROR: bias buffer incorrect size.");
        BufferT local(num_output_channels);
        std::fill(local.data(), local.data() + num_output_channels, T(0));
        std::copy(bias.data(), bias.data() + num_effective_output_channels, local.data());
        packed_bias = std::move(local);
    }

    if (!bn.any()) return;
    if (!bn.all_sized(num_effective_output_channels))
        throw std::invalid_argument(who + "::ctor ERROR: BN buffers incorrect size.");
    const bool no_bias = packed_bias.size() == 0;
    if (no_bias)
    {
        BufferT zeros(num_output_channels);
        std::fill(zeros.data(), zeros.data() + num_output_channels, T(0));
        packed_bias = std::move(zeros);
    }
    T *pf = packed_filters.data();
    T *pb = packed_bias.data();
    for (size_t co = 0; co < num_effective_output_channels; ++co)
    {
        float filter_scale;
        if (conv1d_folding)     // Conv1DLayer.hpp:262-277 divides and sums in another order
        {
            filter_scale = bn.weight[co] / std::sqrt(bn.variance[co] + bn.eps);
            if (no_bias) pb[co] = bn.bias[co] - bn.mean[co] * filter_scale;
            else pb[co] = filter_scale * pb[co] + bn.bias[co] - bn.mean[co] * filter_scale;
        }
        else
        {
            const float rsq = 1.0f / std::sqrt(bn.variance[co] + bn.eps);
            filter_scale = bn.weight[co] * rsq;
            if (no_bias) pb[co] = bn.bias[co] - bn.mean[co] * filter_scale;
            else pb[co] = bn.bias[co] + filter_scale * (pb[co] - bn.mean[co]);
        }
        for (size_t ci = 0; ci < num_input_channels; ++ci)
            for (size_t fh = 0; fh < kernel_height; ++fh)
                for (size_t fw = 0; fw < kernel_width; ++fw)
                    pf[packed_weight_index(num_output_channels, num_input_channels, kernel_height, kernel_width,
                                           BufferT::C_ob, cib, co, ci, fh, fw)] *= filter_scale;
    }
}

// quantised filters in the convolution kernel's operand order (device memory owned by the layer)
class PreparedFilter
{
public:
    PreparedFilter() = default;
    PreparedFilter(PreparedFilter const &) = delete;
    PreparedFilter &operator=(PreparedFilter const &) = delete;
    ~PreparedFilter() { if (m_dev) small_hip_free(m_dev); }

    // no-op unless the element type is uint8 and the kernel supports the shape (Ci % 16 == 0)
    template <class BufferT>
    void build(uint32_t kh, uint32_t kw, uint32_t Co, uint32_t Ci, BufferT const &packed_filters)
    {
        if constexpr (std::is_same<BufferT, QUInt8Buffer>::value)
        {
            if (Ci % QUInt8Buffer::C_ib != 0) return;
            const size_t bytes = small_hip_conv2d_u8_prepared_filter_bytes(kh, kw, Co, Ci);
            if (bytes == 0) return;
            hip_check(small_hip_malloc(&m_dev, bytes), "prepared filter allocation");
            hip_check(small_hip_conv2d_u8_prepare_filter(kh, kw, Co, Ci, packed_filters.device_in(), m_dev,
                                                         current_stream()),
                      "small_hip_conv2d_u8_prepare_filter");
        }
    }
    void const *get() const { return m_dev; }

private:
    void *m_dev = nullptr;
};

// the activation the fused convolution call applies itself; SOFTMAX runs as a second call on the output
inline ActivationType fused_act(ActivationType a) { return a == SOFTMAX ? NONE : a; }

template <class BufferT>
void softmax_in_place(ActivationType a, shape_type const &os, BufferT &buf)
{
    if constexpr (std::is_same<BufferT, FloatBuffer>::value)
    {
        if (a == SOFTMAX)
            batched::SoftMax((int)os[BATCH], (int)os[CHANNEL], (int)os[HEIGHT], (int)os[WIDTH], buf, buf);
    }
}

// padded output channel count, or the reference's error when packed buffers do not allow padding
template <class BufferT>
uint32_t padded_output_channels(uint32_t num_output_channels, bool buffers_are_packed)
{
    const uint32_t rem = num_output_channels % BufferT::C_ob;
    if (rem == 0) return num_output_channels;
    if (buffers_are_packed)
        throw std::invalid_argument("Conv2DLayer::ctor ERROR: invalid number of output channels.");
    return num_output_channels + (BufferT::C_ob - rem);
}

} // namespace detail

//****************************************************************************
template <typename BufferT>
class Conv2DLayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    Conv2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width, uint32_t stride,
                PaddingEnum padding_type, uint32_t num_output_channels, BufferT const &filters,
                bool buffers_are_packed = true, ActivationType activation_type = NONE, float leaky_slope = 1.e-2)
        : Conv2DLayer(input_shape, kernel_height, kernel_width, stride, padding_type, num_output_channels, filters,
                      BufferT(), BufferT(), BufferT(), BufferT(), BufferT(), 0.f, buffers_are_packed,
                      activation_type, leaky_slope)
    {
    }

    Conv2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width, uint32_t stride,
                PaddingEnum padding_type, uint32_t num_output_channels, BufferT const &filters, BufferT const &bias,
                bool buffers_are_packed = true, ActivationType activation_type = NONE, float leaky_slope = 1.e-2)
        : Conv2DLayer(input_shape, kernel_height, kernel_width, stride, padding_type, num_output_channels, filters,
                      bias, BufferT(), BufferT(), BufferT(), BufferT(), 0.f, buffers_are_packed, activation_type,
                      leaky_slope)
    {
    }

    Conv2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width, uint32_t stride,
                PaddingEnum padding_type, uint32_t num_output_channels, BufferT const &filters,
                BufferT const &bn_weight, BufferT const &bn_bias, BufferT const &bn_running_mean,
                BufferT const &bn_running_variance, float const &bn_eps = 1.e-3, bool buffers_are_packed = true,
                ActivationType activation_type = NONE, float leaky_slope = 1.e-2)
        : Conv2DLayer(input_shape, kernel_height, kernel_width, stride, padding_type, num_output_channels, filters,
                      BufferT(), bn_weight, bn_bias, bn_running_mean, bn_running_variance, bn_eps,
                      buffers_are_packed, activation_type, leaky_slope)
    {
    }

    Conv2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width, uint32_t stride,
                PaddingEnum padding_type, uint32_t num_output_channels, BufferT const &filters, BufferT const &bias,
                BufferT const &bn_weight, BufferT const &bn_bias, BufferT const &bn_running_mean,
                BufferT const &bn_running_variance, float const &bn_eps = 1.e-3, bool buffers_are_packed = true,
                ActivationType activation_type = NONE, float leaky_slope = 1.e-2)
        : Layer<BufferT>(),
          m_input_shape(input_shape),
          m_window(input_shape, kernel_height, kernel_width, stride, padding_type),
          m_effective_output_channels(num_output_channels),
          m_activation_type(activation_type),
          m_slope(leaky_slope)
    {
        // 1 and 2 input channels are accepted like 3: small::Conv2D takes all three (the reference's layer
        // class only lets 3 through)
        if ((input_shape[CHANNEL] % BufferT::C_ib) != 0 && (input_shape[CHANNEL] == 0 || input_shape[CHANNEL] > 3))
            throw std::invalid_argument("Conv2DLayer::ctor ERROR: invalid number of input channels.");
        const uint32_t Co = detail::padded_output_channels<BufferT>(num_output_channels, buffers_are_packed);
        this->set_output_shape({input_shape[BATCH], Co, m_window.Ho, m_window.Wo});
        detail::build_conv_weights("*Conv2DLayer", false, Co, m_effective_output_channels,
                                   (uint32_t)input_shape[CHANNEL], kernel_height, kernel_width, filters, bias,
                                   detail::BatchNormRefs<BufferT>{bn_weight, bn_bias, bn_running_mean,
                                                                  bn_running_variance, bn_eps},
                                   buffers_are_packed, m_packed_filters, m_packed_bias);
        if constexpr (std::is_same<BufferT, QUInt8Buffer>::value)
        {
            if (m_packed_bias.size() > 0 || activation_type == LEAKY || activation_type == SOFTMAX)
                throw std::invalid_argument(
                    "Conv2DLayer::ctor ERROR: bias / LeakyReLU / SoftMax have no quantised implementation.");
        }
        m_prepared.build(kernel_height, kernel_width, Co, (uint32_t)input_shape[CHANNEL], m_packed_filters);
    }

    virtual ~Conv2DLayer() {}

    uint32_t get_effective_output_channels() const { return m_effective_output_channels; }
    BufferT const &get_packed_filters() const { return m_packed_filters; }
    BufferT const &get_packed_bias() const { return m_packed_bias; }

    virtual bool one_launch(small_hip_qlayer &d) const
    {
        if constexpr (std::is_same<BufferT, QUInt8Buffer>::value)
        {
            if (m_activation_type != NONE && m_activation_type != RELU) return false;
            auto const &os = this->output_shape();
            d.kind = SMALL_HIP_QL_CONV;
            d.accum_src = SMALL_HIP_QM_NONE;
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


    virtual bool one_launch(small_hip_flayer &d) const
    {
        if constexpr (std::is_same<BufferT, FloatBuffer>::value)
        {
            if (m_activation_type == SOFTMAX) return false;
            d.kind = SMALL_HIP_FL_CONV;
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
        this->check_single_input("Conv2DLayer", input, m_input_shape, output);
        auto const &os = this->output_shape();
        const int batch = (int)m_input_shape[BATCH];
        if constexpr (std::is_same<BufferT, FloatBuffer>::value)
        {
            batched::Conv2D_Bias_Act(batch, m_window.kh, m_window.kw, m_window.stride, m_window.t, m_window.b,
                                     m_window.l, m_window.r, (int)os[CHANNEL], (int)m_input_shape[CHANNEL],
                                     (int)m_input_shape[HEIGHT], (int)m_input_shape[WIDTH], input[0]->buffer(),
                                     m_packed_filters, m_packed_bias, detail::fused_act(m_activation_type), m_slope, output->buffer());
        }
        else
        {
            batched::Conv2D_Accum_ReLU(batch, m_window.kh, m_window.kw, m_window.stride, m_window.t, m_window.b,
                                       m_window.l, m_window.r, (int)os[CHANNEL], (int)m_input_shape[CHANNEL],
                                       (int)m_input_shape[HEIGHT], (int)m_input_shape[WIDTH], input[0]->buffer(),
                                       m_packed_filters, m_prepared.get(), (BufferT const *)nullptr,
                                       m_activation_type == RELU, output->buffer());
        }
        detail::softmax_in_place(m_activation_type, os, output->buffer());
        output->set_shape(os);
    }

    // This layer followed by a MaxPool2DLayer with window `pool` in one call (small::batched::
    // Conv2D_Bias_Act_Maxpool2D: one launch for a 2x2 stride-2 un-padded pool on a map the kernel's tiles fill,
    // else the two launches through `inter`).  float32, ReLU / LeakyReLU / no activation; the caller checks
    // fusable_with_pool() first.  `pooled` receives the pooling layer's output shape.
    bool fusable_with_pool() const
    {
        return std::is_same<BufferT, FloatBuffer>::value && m_activation_type != SOFTMAX;
    }

    void compute_output_pooled(Tensor<BufferT> const *input, detail::Window const &pool, shape_type const &pooled_shape,
                               Tensor<BufferT> *inter, Tensor<BufferT> *pooled) const
    {
        if constexpr (std::is_same<BufferT, FloatBuffer>::value)
        {
            this->check_single_input("Conv2DLayer", {input}, m_input_shape, inter);
            if (pooled->capacity() < compute_size(pooled_shape))
                throw std::invalid_argument("Conv2DLayer::compute_output_pooled() ERROR: insufficient output buffer space.");
            auto const &os = this->output_shape();
            batched::Conv2D_Bias_Act_Maxpool2D(
                (int)m_input_shape[BATCH], m_window.kh, m_window.kw, m_window.stride, m_window.t, m_window.b, m_window.l,
                m_window.r, pool.kh, pool.kw, pool.stride, pool.t, pool.b, pool.l, pool.r, (int)os[CHANNEL],
                (int)m_input_shape[CHANNEL], (int)m_input_shape[HEIGHT], (int)m_input_shape[WIDTH], input->buffer(),
                m_packed_filters, m_packed_bias, m_activation_type, m_slope, inter->buffer(), pooled->buffer());
            pooled->set_shape(pooled_shape);
        }
        else
            throw std::invalid_argument("Conv2DLayer::compute_output_pooled() ERROR: float32 only.");
    }

    // This layer and the depthwise layer after it as one launch (the reference's Conv2D_ReLU_DepthwiseConv2D_ReLU pairing,
    // fused_interface_abstract.hpp:1840): true for the pairs small::detail::conv_dw_one_launch names, when both layers have
    // the same ReLU / LeakyReLU / no activation and this layer's channels are not padded.  DwLayerT: DepthwiseConv2DLayer.
    template <class DwLayerT>
    bool fusable_with_depthwise(DwLayerT const &dw) const
    {
        auto const &os = this->output_shape();
        auto const &w = dw.window();
        return std::is_same<BufferT, FloatBuffer>::value && m_activation_type != SOFTMAX && m_activation_type == dw.activation() &&
               (m_activation_type != LEAKY || m_slope == dw.slope()) && m_effective_output_channels == os[CHANNEL] &&
               detail::conv_dw_one_launch<BufferT>((int)m_input_shape[BATCH], (int)m_window.kh, (int)m_window.kw, (int)m_window.stride, m_window.t, m_window.b,
                                                   m_window.l, m_window.r, (int)w.kh, (int)w.kw, (int)w.stride, w.t, w.b, w.l, w.r,
                                                   (int)os[CHANNEL], (int)m_input_shape[CHANNEL], (int)m_input_shape[HEIGHT],
                                                   (int)m_input_shape[WIDTH]);
    }

    // `output` (not the input tensor) receives the depthwise layer's output; the caller checks fusable_with_depthwise() first
    template <class DwLayerT>
    void compute_output_depthwise(Tensor<BufferT> const *input, DwLayerT const &dw, Tensor<BufferT> *output) const
    {
        if constexpr (std::is_same<BufferT, FloatBuffer>::value)
        {
            this->check_single_input("Conv2DLayer", {input}, m_input_shape, output);
            if (output->capacity() < compute_size(dw.output_shape()))
                throw std::invalid_argument("Conv2DLayer::compute_output_depthwise() ERROR: insufficient output buffer space.");
            auto const &os = this->output_shape();
            auto const &w = dw.window();
            batched::Conv2D_Bias_Act_DepthwiseConv2D_Bias_Act(
                (int)m_input_shape[BATCH], m_window.kh, m_window.kw, m_window.stride, m_window.t, m_window.b, m_window.l,
                m_window.r, w.kh, w.kw, w.stride, w.t, w.b, w.l, w.r, (int)os[CHANNEL], (int)m_input_shape[CHANNEL],
                (int)m_input_shape[HEIGHT], (int)m_input_shape[WIDTH], input->buffer(), m_packed_filters, m_packed_bias,
                output->buffer() /* not touched: the pair runs as one launch */, dw.get_packed_filters(), dw.get_packed_bias(),
                m_activation_type, m_slope, output->buffer());
            output->set_shape(dw.output_shape());
        }
        else
            throw std::invalid_argument("Conv2DLayer::compute_output_depthwise() ERROR: float32 only.");
    }

private:
    shape_type const m_input_shape;
    detail::Window const m_window;
    uint32_t const m_effective_output_channels;
    ActivationType const m_activation_type;
    float const m_slope;
    BufferT m_packed_filters;
    BufferT m_packed_bias;
    detail::PreparedFilter m_prepared;
};

} // namespace small
