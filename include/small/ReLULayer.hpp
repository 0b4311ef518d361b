// ReLULayer (reference include/small/ReLULayer.hpp:24-73); input and output may be the same tensor.
#pragma once

#include "Layer.hpp"

namespace small
{

template <typename BufferT>
class ReLULayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    ReLULayer(shape_type const &input_shape) : Layer<BufferT>(input_shape) {}
    virtual ~ReLULayer() {}

    virtual void compute_output(std::vector<Tensor<BufferT> const *> input, Tensor<BufferT> *output) const
    {
        auto const &os = this->output_shape();
        this->check_single_input("ReLULayer", input, os, output);
        batched::ReLUActivation((int)os[BATCH], (int)os[CHANNEL], (int)os[HEIGHT], (int)os[WIDTH],
                                input[0]->buffer(), output->buffer());
        output->set_shape(os);
    }
};

} // namespace small
