// DummyLayer: a placeholder that only carries a shape (a model's input node; reference
// include/small/DummyLayer.hpp:24-50).
#pragma once

#include "Layer.hpp"

namespace small
{

template <typename BufferT>
class DummyLayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    DummyLayer(shape_type const &shape) : Layer<BufferT>(shape) {}
    virtual ~DummyLayer() {}

    virtual void compute_output(std::vector<Tensor<BufferT> const *>, Tensor<BufferT> *) const {}
};

} // namespace small
