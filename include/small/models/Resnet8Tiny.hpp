// Resnet8Tiny: the MLPerf-Tiny ResNet-8 as the reference assembles it
// (include/small/models/Resnet8Tiny.hpp:232-420): Conv2D 3x3 + ReLU, one identity residual block,
// two down-sampling residual blocks (3x3 s2 + ReLU, 1x1 s2 shortcut, 3x3 accumulated onto the shortcut +
// ReLU), a pooling layer over the whole map and a 1x1 convolution as classifier.  Residual adds are
// PartialConv2DLayers that accumulate onto the tensor holding the shortcut.
//
// Filter order is the reference's, including the swapped 1x1 shortcut filters:
//   0 stem, 1-2 block 1, 3 conv a / 5 shortcut / 4 conv b of block 2, 6 / 8 / 7 of block 3, 9 classifier.
// Class count is a constructor argument (reference: 16); the batch extent of the input shape is honoured.
#pragma once

#include <algorithm>
#include <vector>

#include "../Conv2DLayer.hpp"
#include "../MaxPool2DLayer.hpp"
#include "../Model.hpp"
#include "../PartialConv2DLayer.hpp"

namespace small
{

template <typename BufferT>
class Resnet8Tiny : public Model<BufferT>
{
public:
    Resnet8Tiny() = delete;

    Resnet8Tiny(shape_type const &input_shape, std::vector<BufferT *> const &filters,
                bool filters_are_packed = false, uint32_t num_classes = 16)
        : Model<BufferT>(input_shape)
    {
        if (filters.size() != 10) throw std::invalid_argument("Resnet8Tiny ctor ERROR: 10 filter buffers expected.");
        uint32_t channels = 16;
        size_t cap = 0;
        auto grow = [&](Layer<BufferT> *l) { cap = std::max(cap, l->output_size()); return l; };
        Layer<BufferT> *prev = grow(this->add(new Conv2DLayer<BufferT>(input_shape, 3, 3, 1, PADDING_F, channels,
                                                                       *filters[0], filters_are_packed, RELU)));
        prev = grow(this->add(new Conv2DLayer<BufferT>(prev->output_shape(), 3, 3, 1, PADDING_F, channels,
                                                       *filters[1], filters_are_packed, RELU)));
        prev = grow(this->add(new PartialConv2DLayer<BufferT>(prev->output_shape(), 3, 3, 1, PADDING_F, channels,
                                                              *filters[2], filters_are_packed, RELU)));
        size_t f = 3;
        for (int blk = 0; blk < 2; ++blk)
        {
            Layer<BufferT> *block_in = prev;
            channels *= 2;
            Layer<BufferT> *a = grow(this->add(new Conv2DLayer<BufferT>(block_in->output_shape(), 3, 3, 2, PADDING_F,
                                                                        channels, *filters[f], filters_are_packed,
                                                                        RELU)));
            grow(this->add(new Conv2DLayer<BufferT>(block_in->output_shape(), 1, 1, 2, PADDING_V, channels,
                                                    *filters[f + 2], filters_are_packed)));
            prev = grow(this->add(new PartialConv2DLayer<BufferT>(a->output_shape(), 3, 3, 1, PADDING_F, channels,
                                                                  *filters[f + 1], filters_are_packed, RELU)));
            f += 3;
        }
        const uint32_t ph = (uint32_t)prev->output_shape()[HEIGHT], pw = (uint32_t)prev->output_shape()[WIDTH];
        prev = grow(this->add(new MaxPool2DLayer<BufferT>(prev->output_shape(), ph, pw, 1, PADDING_V)));
        grow(this->add(new Conv2DLayer<BufferT>(prev->output_shape(), 1, 1, 1, PADDING_V, num_classes, *filters[f],
                                                filters_are_packed)));
        for (auto &t : m_buffers) t.reset(new Tensor<BufferT>(cap));
    }

    virtual ~Resnet8Tiny() {}

    virtual std::vector<Tensor<BufferT> *> inference(Tensor<BufferT> const *input_tensor)
    {
        Tensor<BufferT> *b0 = m_buffers[0].get(), *b1 = m_buffers[1].get(), *b2 = m_buffers[2].get();
        std::vector<detail::LaunchStep<BufferT>> steps;
        size_t l = 0;
        auto step = [&](Tensor<BufferT> const *src, Tensor<BufferT> *dst) { steps.push_back({this->m_layers[l++], src, dst}); };
        step(input_tensor, b0);                                    // stem
        step(b0, b1);
        step(b1, b0);                                              // b0 += conv(b1), ReLU
        for (int blk = 0; blk < 2; ++blk)
        {
            step(b0, b1);                                          // 3x3 stride 2 + ReLU
            step(b0, b2);                                          // 1x1 stride 2 shortcut
            step(b1, b2);                                          // b2 += conv(b1), ReLU
            std::swap(b0, b2);
        }
        step(b0, b1);                                              // pooling
        step(b1, b0);                                              // classifier
        // quantised: the whole pass in one launch when it fits (only b0 is written then); else layer by layer
        if (!this->forward_one_launch(steps))
            for (auto const &s : steps) s.layer->compute_output({s.src}, s.dst);
        return {b0};
    }

private:
    std::unique_ptr<Tensor<BufferT>> m_buffers[3];
};

} // namespace small
