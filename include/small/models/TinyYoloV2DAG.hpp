// TinyYoloV2DAG: TinyYoloV2 run by the DAG executor (reference include/small/models/TinyYoloV2DAG.hpp): the same layers,
// built by TinyYoloV2's constructor and handed over, as vertices of a chain; tensors come from DAGModel's pool.
#pragma once

#include "../DAGModel.hpp"
#include "TinyYoloV2.hpp"

namespace small
{

template <typename BufferT>
class TinyYoloV2DAG : public DAGModel<BufferT>
{
public:
    TinyYoloV2DAG() = delete;

    TinyYoloV2DAG(shape_type const &input_shape, std::vector<BufferT *> const &filters, bool filters_are_packed = false,
                  ActivationType activation = RELU, float leaky_slope = 0.1f, uint32_t num_outputs = 16,
                  bool activate_output = true)
        : DAGModel<BufferT>(input_shape)
    {
        TinyYoloV2<BufferT> seq(input_shape, filters, filters_are_packed, activation, leaky_slope, num_outputs,
                                activate_output);
        this->adopt_layers(seq.release_layers());
    }

    virtual ~TinyYoloV2DAG() {}
};

} // namespace small
