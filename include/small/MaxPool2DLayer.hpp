// MaxPool2DLayer: window maximum (padding counts as zero-valued pixels) over the window geometry of the padding type (same constructor, checks
// and messages as the reference's include/small/MaxPool2DLayer.hpp:24-116); the batch extent of the
// input shape is honoured.
#pragma once

#include <type_traits>

#include "Layer.hpp"

namespace small
{

template <typename BufferT>
class MaxPool2DLayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    MaxPool2DLayer(shape_type const &input_shape, uint32_t kernel_height, uint32_t kernel_width, uint32_t stride,
                  PaddingEnum padding_type)
        : Layer<BufferT>(),
          m_input_shape(input_shape),
          m_window(input_shape, kernel_height, kernel_width, stride, padding_type)
    {
        this->set_output_shape({input_shape[BATCH], input_shape[CHANNEL], m_window.Ho, m_window.Wo});
    }

    virtual ~MaxPool2DLayer() {}

    virtual void compute_output(std::vector<Tensor<BufferT> const *> input, Tensor<BufferT> *output) const
    {
        this->check_single_input("MaxPool2DLayer", input, m_input_shape, output);
        batched::MaxPool2D((int)m_input_shape[BATCH], m_window.kh, m_window.kw, m_window.stride, m_window.t, m_window.b,
                      m_window.l, m_window.r, (int)m_input_shape[CHANNEL], (int)m_input_shape[HEIGHT],
                      (int)m_input_shape[WIDTH], input[0]->buffer(), output->buffer());
        output->set_shape(this->output_shape());
    }

    // window geometry (kernel, stride, pads from the padding type)
    detail::Window const &window() const { return m_window; }

    virtual bool one_launch(small_hip_qlayer &d) const
    {
        if constexpr (std::is_same<BufferT, QUInt8Buffer>::value)
        {
            d.kind = SMALL_HIP_QL_GLOBAL_MAXPOOL;
            d.accum_src = SMALL_HIP_QM_NONE;
            d.relu = 0;
            d.kernel_height = (int)m_window.kh; d.kernel_width = (int)m_window.kw; d.stride = (int)m_window.stride;
            d.t_pad = m_window.t; d.b_pad = m_window.b; d.l_pad = m_window.l; d.r_pad = m_window.r;
            d.output_channels = d.input_channels = (int)m_input_shape[CHANNEL];
            d.input_height = (int)m_input_shape[HEIGHT]; d.input_width = (int)m_input_shape[WIDTH];
            d.filter = nullptr;
            return true;
        }
        else
            return false;
    }

    virtual bool one_launch(small_hip_flayer &d) const
    {
        if constexpr (std::is_same<BufferT, FloatBuffer>::value)
        {
            d.kind = SMALL_HIP_FL_GLOBAL_MAXPOOL;
            d.act = SMALL_HIP_ACT_NONE;
            d.slope = 0.f;
            d.kernel_height = (int)m_window.kh; d.kernel_width = (int)m_window.kw; d.stride = (int)m_window.stride;
            d.t_pad = m_window.t; d.b_pad = m_window.b; d.l_pad = m_window.l; d.r_pad = m_window.r;
            d.output_channels = d.input_channels = (int)m_input_shape[CHANNEL];
            d.input_height = (int)m_input_shape[HEIGHT]; d.input_width = (int)m_input_shape[WIDTH];
            d.filter = nullptr;
            d.bias = nullptr;
            return true;
        }
        else
            return false;
    }

private:
    shape_type const m_input_shape;
    detail::Window const m_window;
};

} // namespace small
