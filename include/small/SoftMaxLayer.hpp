// SoftMaxLayer (reference include/small/SoftMaxLayer.hpp:24-73): small::SoftMax over the whole tensor
// of each image; float only, input and output may be the same tensor.
#pragma once

#include "Layer.hpp"

namespace small
{

template <typename BufferT>
class SoftMaxLayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    SoftMaxLayer(shape_type const &input_shape) : Layer<BufferT>(input_shape) {}
    virtual ~SoftMaxLayer() {}

    virtual void compute_output(std::vector<Tensor<BufferT> const *> input, Tensor<BufferT> *output) const
    {
        auto const &os = this->output_shape();
        this->check_single_input("SoftMaxLayer", input, os, output);
        batched::SoftMax((int)os[BATCH], (int)os[CHANNEL], (int)os[HEIGHT], (int)os[WIDTH], input[0]->buffer(),
                         output->buffer());
        output->set_shape(os);
    }
};

} // namespace small
