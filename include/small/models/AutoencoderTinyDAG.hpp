// AutoencoderTinyDAG: AutoencoderTiny run by the DAG executor (reference include/small/models/AutoencoderTinyDAG.hpp): the same layers,
// built by AutoencoderTiny's constructor and handed over, as vertices of a chain; tensors come from DAGModel's pool.
#pragma once

#include "../DAGModel.hpp"
#include "AutoencoderTiny.hpp"

namespace small
{

template <typename BufferT>
class AutoencoderTinyDAG : public DAGModel<BufferT>
{
public:
    AutoencoderTinyDAG() = delete;

    AutoencoderTinyDAG(shape_type const &input_shape, size_t dimension_reduction,
                       std::vector<BufferT *> const &filters, bool filters_are_packed = false)
        : DAGModel<BufferT>(input_shape)
    {
        AutoencoderTiny<BufferT> seq(input_shape, dimension_reduction, filters, filters_are_packed);
        this->adopt_layers(seq.release_layers());
    }

    virtual ~AutoencoderTinyDAG() {}
};

} // namespace small
