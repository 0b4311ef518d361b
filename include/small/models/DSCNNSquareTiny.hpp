// DSCNNSquareTiny: the keyword-spotting DS-CNN with a square 3x3 stride-2 stem, as the reference assembles it
// (include/small/models/DSCNNSquareTiny.hpp:108-190): Conv2D 3x3 s2 'f' + ReLU on the 3 x 49 x 10 input, then
// 4 x (DepthwiseConv2D 3x3 + ReLU, Conv2D 1x1 + ReLU) at 64 channels, MaxPool2D over the whole map and a 1x1
// convolution to 16 classes.  It is DSCNNTiny with another stem window.
#pragma once

#include "DSCNNTiny.hpp"

namespace small
{

template <typename BufferT>
class DSCNNSquareTiny : public DSCNNTiny<BufferT>
{
public:
    DSCNNSquareTiny() = delete;

    DSCNNSquareTiny(shape_type const &input_shape, std::vector<BufferT *> const &filters,
                    bool filters_are_packed = false, uint32_t num_classes = 16)
        : DSCNNTiny<BufferT>(input_shape, filters, filters_are_packed, 3, 3, num_classes, false)
    {
    }

    virtual ~DSCNNSquareTiny() {}
};

} // namespace small
