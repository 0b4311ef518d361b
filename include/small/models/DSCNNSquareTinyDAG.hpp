// DSCNNSquareTinyDAG: DSCNNSquareTiny run by the DAG executor (reference include/small/models/DSCNNSquareTinyDAG.hpp): the same layers,
// built by DSCNNSquareTiny's constructor and handed over, as vertices of a chain; tensors come from DAGModel's pool.
#pragma once

#include "../DAGModel.hpp"
#include "DSCNNSquareTiny.hpp"

namespace small
{

template <typename BufferT>
class DSCNNSquareTinyDAG : public DAGModel<BufferT>
{
public:
    DSCNNSquareTinyDAG() = delete;

    DSCNNSquareTinyDAG(shape_type const &input_shape, std::vector<BufferT *> const &filters,
                       bool filters_are_packed = false, uint32_t num_classes = 16)
        : DAGModel<BufferT>(input_shape)
    {
        DSCNNSquareTiny<BufferT> seq(input_shape, filters, filters_are_packed, num_classes);
        this->adopt_layers(seq.release_layers());
    }

    virtual ~DSCNNSquareTinyDAG() {}
};

} // namespace small
