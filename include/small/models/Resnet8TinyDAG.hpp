// Resnet8TinyDAG: Resnet8Tiny run by the DAG executor (reference include/small/models/Resnet8TinyDAG.hpp:272-439): the
// same layers, built by Resnet8Tiny's constructor and handed over, as vertices of a graph with the three residual
// joins.  A PartialConv2DLayer's first parent is the shortcut tensor it accumulates onto, its second the convolution
// output it reads; tensors come from DAGModel's pool.
#pragma once

#include "../DAGModel.hpp"
#include "Resnet8Tiny.hpp"

namespace small
{

template <typename BufferT>
class Resnet8TinyDAG : public DAGModel<BufferT>
{
public:
    Resnet8TinyDAG() = delete;

    Resnet8TinyDAG(shape_type const &input_shape, std::vector<BufferT *> const &filters,
                   bool filters_are_packed = false, uint32_t num_classes = 16)
        : DAGModel<BufferT>(input_shape)
    {
        Resnet8Tiny<BufferT> seq(input_shape, filters, filters_are_packed, num_classes);
        // 0 stem, 1 conv, 2 partial (onto 0) | 3 conv a, 4 shortcut, 5 partial (onto 4) | 6, 7, 8 likewise | 9 pool, 10 fc
        this->adopt_layers(seq.release_layers(),
                           {{}, {0}, {0, 1}, {2}, {2}, {4, 3}, {5}, {5}, {7, 6}, {8}, {9}});
    }

    virtual ~Resnet8TinyDAG() {}
};

} // namespace small
