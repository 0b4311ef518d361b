// DSCNNTinyDAG: DSCNNTiny run by the DAG executor (reference include/small/models/DSCNNTinyDAG.hpp): the same layers,
// built by DSCNNTiny's constructor and handed over, as vertices of a chain; tensors come from DAGModel's pool.
#pragma once

#include "../DAGModel.hpp"
#include "DSCNNTiny.hpp"

namespace small
{

template <typename BufferT>
class DSCNNTinyDAG : public DAGModel<BufferT>
{
public:
    DSCNNTinyDAG() = delete;

    DSCNNTinyDAG(shape_type const &input_shape, std::vector<BufferT *> const &filters, bool filters_are_packed = false,
                 uint32_t stem_kernel_height = 3, uint32_t stem_kernel_width = 1, uint32_t num_classes = 16,
                 bool average_pool = false)
        : DAGModel<BufferT>(input_shape)
    {
        DSCNNTiny<BufferT> seq(input_shape, filters, filters_are_packed, stem_kernel_height, stem_kernel_width, num_classes,
                               average_pool);
        this->adopt_layers(seq.release_layers());
    }

    virtual ~DSCNNTinyDAG() {}
};

} // namespace small
