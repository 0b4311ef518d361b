// DSCNNTiny: the keyword-spotting DS-CNN as the reference assembles it
// (include/small/models/DSCNNTiny.hpp:170-262): a stem convolution + ReLU, 4 x (DepthwiseConv2D 3x3 + ReLU,
// Conv2D 1x1 + ReLU), a pooling layer over the whole map and a 1x1 convolution as classifier.
//
// The reference's stem is 3x1 stride 2 on a 3-channel 49x10 input (its padded-edge code cannot run the
// original 10x4 kernel); this build can, so the stem window and the pooling kind are constructor
// arguments, with the reference's values as defaults.
#pragma once

#include <algorithm>
#include <vector>

#include "../AveragePool2DLayer.hpp"
#include "../Conv2DLayer.hpp"
#include "../DepthwiseConv2DLayer.hpp"
#include "../MaxPool2DLayer.hpp"
#include "../Model.hpp"

namespace small
{

template <typename BufferT>
class DSCNNTiny : public Model<BufferT>
{
public:
    DSCNNTiny() = delete;

    // filters: stem, then (depthwise, pointwise) x 4, then the classifier: 10 buffers
    DSCNNTiny(shape_type const &input_shape, std::vector<BufferT *> const &filters, bool filters_are_packed = false,
              uint32_t stem_kernel_height = 3, uint32_t stem_kernel_width = 1, uint32_t num_classes = 16,
              bool average_pool = false)
        : Model<BufferT>(input_shape)
    {
        if (filters.size() != 10) throw std::invalid_argument("DSCNNTiny ctor ERROR: 10 filter buffers expected.");
        const uint32_t channels = 64;
        size_t f = 0, cap0 = 0, cap1 = 0;
        Layer<BufferT> *prev =
            this->add(new Conv2DLayer<BufferT>(input_shape, stem_kernel_height, stem_kernel_width, 2, PADDING_F,
                                               channels, *filters[f++], filters_are_packed, RELU));
        cap0 = std::max(cap0, prev->output_size());
        for (int blk = 0; blk < 4; ++blk)
        {
            prev = this->add(new DepthwiseConv2DLayer<BufferT>(prev->output_shape(), 3, 3, 1, PADDING_F,
                                                               *filters[f++], filters_are_packed, RELU));
            cap1 = std::max(cap1, prev->output_size());
            prev = this->add(new Conv2DLayer<BufferT>(prev->output_shape(), 1, 1, 1, PADDING_V, channels,
                                                      *filters[f++], filters_are_packed, RELU));
            cap0 = std::max(cap0, prev->output_size());
        }
        const uint32_t ph = (uint32_t)prev->output_shape()[HEIGHT], pw = (uint32_t)prev->output_shape()[WIDTH];
        if (average_pool)
            prev = this->add(new AveragePool2DLayer<BufferT>(prev->output_shape(), ph, pw, 1, PADDING_V));
        else
            prev = this->add(new MaxPool2DLayer<BufferT>(prev->output_shape(), ph, pw, 1, PADDING_V));
        cap1 = std::max(cap1, prev->output_size());
        prev = this->add(new Conv2DLayer<BufferT>(prev->output_shape(), 1, 1, 1, PADDING_V, num_classes,
                                                  *filters[f++], filters_are_packed));
        cap0 = std::max(cap0, prev->output_size());
        m_buffer_0.reset(new Tensor<BufferT>(cap0));
        m_buffer_1.reset(new Tensor<BufferT>(cap1));
    }

    virtual ~DSCNNTiny() {}

    virtual std::vector<Tensor<BufferT> *> inference(Tensor<BufferT> const *input_tensor)
    {
        Tensor<BufferT> *a = m_buffer_0.get(), *b = m_buffer_1.get();
        std::vector<detail::LaunchStep<BufferT>> steps;
        size_t l = 0;
        steps.push_back({this->m_layers[l++], input_tensor, a});
        while (l < this->m_layers.size())
        {
            steps.push_back({this->m_layers[l++], a, b});
            steps.push_back({this->m_layers[l++], b, a});
        }
        // the whole pass in one launch when the model fits one compute unit's LDS (only `a` is written then)
        if (!this->forward_one_launch(steps))
            for (auto const &s : steps) s.layer->compute_output({s.src}, s.dst);
        return {a};
    }

private:
    std::unique_ptr<Tensor<BufferT>> m_buffer_0, m_buffer_1;
};

} // namespace small
