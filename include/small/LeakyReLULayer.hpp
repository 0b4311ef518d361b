// LeakyReLULayer (reference include/small/LeakyReLULayer.hpp:24-82): x > 0 ? x : slope * x.
// float only, as in the reference; input and output may be the same tensor.
#pragma once

#include "Layer.hpp"

namespace small
{

template <typename BufferT>
class LeakyReLULayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    LeakyReLULayer(shape_type const &input_shape, float leaky_slope = 0.01f)
        : Layer<BufferT>(input_shape), m_leaky_slope(1)
    {
        m_leaky_slope[0] = leaky_slope;
    }
    virtual ~LeakyReLULayer() {}

    virtual void compute_output(std::vector<Tensor<BufferT> const *> input, Tensor<BufferT> *output) const
    {
        auto const &os = this->output_shape();
        this->check_single_input("LeakyReLULayer", input, os, output);
        batched::LeakyReLUActivation((int)os[BATCH], (int)os[CHANNEL], (int)os[HEIGHT], (int)os[WIDTH],
                                     input[0]->buffer(), m_leaky_slope, output->buffer());
        output->set_shape(os);
    }

private:
    BufferT m_leaky_slope;   // one element, the form small::LeakyReLUActivation takes
};

} // namespace small
