// MobileNetTinyDAG: MobileNetTiny run by the DAG executor (reference include/small/models/MobileNetTinyDAG.hpp): the same layers,
// built by MobileNetTiny's constructor and handed over, as vertices of a chain; tensors come from DAGModel's pool.
#pragma once

#include "../DAGModel.hpp"
#include "MobileNetTiny.hpp"

namespace small
{

template <typename BufferT>
class MobileNetTinyDAG : public DAGModel<BufferT>
{
public:
    MobileNetTinyDAG() = delete;

    MobileNetTinyDAG(shape_type const &input_shape, std::vector<BufferT *> const &filters,
                     bool filters_are_packed = false, uint32_t first_channels = 32, uint32_t num_classes = 16,
                     bool average_pool = false)
        : DAGModel<BufferT>(input_shape)
    {
        MobileNetTiny<BufferT> seq(input_shape, filters, filters_are_packed, first_channels, num_classes, average_pool);
        this->adopt_layers(seq.release_layers());
    }

    virtual ~MobileNetTinyDAG() {}
};

} // namespace small
