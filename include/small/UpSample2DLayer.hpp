// UpSample2DLayer: nearest-neighbour upsampling by 1 or 2 (reference
// include/small/UpSample2DLayer.hpp:24-97).
#pragma once

#include "Layer.hpp"

namespace small
{

template <typename BufferT>
class UpSample2DLayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    UpSample2DLayer(shape_type const &input_shape, uint32_t scale_factor)
        : Layer<BufferT>(), m_input_shape(input_shape), m_scale_factor(scale_factor)
    {
        if (scale_factor != 1 && scale_factor != 2)
            throw std::invalid_argument("UpSample2DLayer ERROR: unsupported scale factor.");
        this->set_output_shape({input_shape[BATCH], input_shape[CHANNEL], input_shape[HEIGHT] * scale_factor,
                                input_shape[WIDTH] * scale_factor});
    }
    virtual ~UpSample2DLayer() {}

    virtual void compute_output(std::vector<Tensor<BufferT> const *> input, Tensor<BufferT> *output) const
    {
        this->check_single_input("UpSample2DLayer", input, m_input_shape, output);
        batched::UpSample2D((int)m_input_shape[BATCH], (int)m_scale_factor, (int)m_input_shape[CHANNEL],
                            (int)m_input_shape[HEIGHT], (int)m_input_shape[WIDTH], input[0]->buffer(),
                            output->buffer());
        output->set_shape(this->output_shape());
    }

private:
    shape_type const m_input_shape;
    uint32_t const m_scale_factor;
};

} // namespace small
