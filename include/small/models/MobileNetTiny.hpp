// MobileNetTiny: MobileNetV1 as the reference assembles it (include/small/models/MobileNetTiny.hpp:421-540):
// Conv2D 3x3 s2 'f' + ReLU, 13 x (DepthwiseConv2D 3x3 + ReLU, Conv2D 1x1 + ReLU), a pooling layer over the
// remaining map and a 1x1 convolution as classifier, ping-ponging between two tensors.
//
// Generalised where the reference hard-codes the MLPerf-Tiny instance (32 first-layer channels, 16
// classes, MaxPool 3x3): width, class count and pooling kind are constructor arguments with the
// reference's values as defaults, the pooling window is the remaining feature map, and the batch
// extent of the input shape is honoured.
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
class MobileNetTiny : public Model<BufferT>
{
public:
    MobileNetTiny() = delete;

    // filters: stem, then (depthwise, pointwise) x 13, then the classifier: 28 buffers
    MobileNetTiny(shape_type const &input_shape, std::vector<BufferT *> const &filters,
                  bool filters_are_packed = false, uint32_t first_channels = 32, uint32_t num_classes = 16,
                  bool average_pool = false)
        : Model<BufferT>(input_shape)
    {
        if (filters.size() != 28) throw std::invalid_argument("MobileNetTiny ctor ERROR: 28 filter buffers expected.");
        size_t f = 0, cap0 = 0, cap1 = 0;
        Layer<BufferT> *prev = this->add(new Conv2DLayer<BufferT>(input_shape, 3, 3, 2, PADDING_F, first_channels,
                                                                  *filters[f++], filters_are_packed, RELU));
        cap0 = std::max(cap0, prev->output_size());
        static const uint32_t strides[13] = {1, 2, 1, 2, 1, 2, 1, 1, 1, 1, 1, 2, 1};
        static const uint32_t widen[13] = {2, 2, 1, 2, 1, 2, 1, 1, 1, 1, 1, 2, 1};
        for (int blk = 0; blk < 13; ++blk)
        {
            prev = this->add(new DepthwiseConv2DLayer<BufferT>(prev->output_shape(), 3, 3, strides[blk], PADDING_F,
                                                               *filters[f++], filters_are_packed, RELU));
            cap1 = std::max(cap1, prev->output_size());
            const uint32_t co = (uint32_t)prev->output_shape()[CHANNEL] * widen[blk];
            prev = this->add(new Conv2DLayer<BufferT>(prev->output_shape(), 1, 1, 1, PADDING_V, co, *filters[f++],
                                                      filters_are_packed, RELU));
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
        // a fused convolution + depthwise step shifts which of the two tensors a layer writes: one size for both
        cap0 = std::max(cap0, cap1);
        m_buffer_0.reset(new Tensor<BufferT>(cap0));
        m_buffer_1.reset(new Tensor<BufferT>(cap0));
    }

    virtual ~MobileNetTiny() {}

    virtual std::vector<Tensor<BufferT> *> inference(Tensor<BufferT> const *input_tensor)
    {
        // every step reads the tensor the previous step wrote and writes the other one; a convolution and the depthwise
        // layer after it are one step (one launch) where that is faster than two (Conv2DLayer::fusable_with_depthwise)
        Tensor<BufferT> *bufs[2] = {m_buffer_0.get(), m_buffer_1.get()};
        Tensor<BufferT> const *cur = input_tensor;
        int w = 0;
        const size_t n = this->m_layers.size();
        for (size_t l = 0; l < n; w ^= 1)
        {
            Tensor<BufferT> *out = bufs[w];
            auto *conv = dynamic_cast<Conv2DLayer<BufferT> *>(this->m_layers[l]);
            auto *dw = l + 1 < n ? dynamic_cast<DepthwiseConv2DLayer<BufferT> *>(this->m_layers[l + 1]) : nullptr;
            if (conv && dw && conv->fusable_with_depthwise(*dw))
            {
                conv->compute_output_depthwise(cur, *dw, out);
                l += 2;
            }
            else
                this->m_layers[l++]->compute_output({cur}, out);
            cur = out;
        }
        return {bufs[w ^ 1]};
    }

private:
    std::unique_ptr<Tensor<BufferT>> m_buffer_0, m_buffer_1;
};

} // namespace small
