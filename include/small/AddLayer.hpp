// AddLayer: output += input (reference include/small/AddLayer.hpp:24-81; small::Accum).  For
// QUInt8Buffer the reference has no Accum; this build's definition is
// out = requant_out((in + in.zero) + (out + out.zero)).
#pragma once

#include "Layer.hpp"

namespace small
{

template <typename BufferT>
class AddLayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    AddLayer(shape_type const &input1_shape, shape_type const &input2_shape) : Layer<BufferT>(input1_shape)
    {
        if (input1_shape != input2_shape)
            throw std::invalid_argument("AddLayer ctor ERROR: predecessors do not have same output shape.");
    }
    virtual ~AddLayer() {}

    virtual void compute_output(std::vector<Tensor<BufferT> const *> input, Tensor<BufferT> *output) const
    {
        auto const &os = this->output_shape();
        if (input.size() != 1 || input[0]->shape() != os || output->shape() != os)
            throw std::invalid_argument("AddLayer::compute_output() ERROR: incorrect input buffer shape.");
        batched::Accum((int)os[BATCH], (int)os[CHANNEL], (int)os[HEIGHT], (int)os[WIDTH], input[0]->buffer(),
                       output->buffer());
    }
};

} // namespace small
