// AutoencoderTiny: the anomaly-detection autoencoder as the reference assembles it
// (include/small/models/AutoencoderTiny.hpp:103-211): dense layers spelled as 1x1 convolutions + ReLU on a
// 1x1 image; every layer has 128 outputs but the fifth (index 4), the bottleneck, which has
// `dimension_reduction`.  One filter buffer per layer; the layer count is the filter count.
#pragma once

#include <algorithm>
#include <vector>

#include "../Conv2DLayer.hpp"
#include "../Model.hpp"

namespace small
{

template <typename BufferT>
class AutoencoderTiny : public Model<BufferT>
{
public:
    AutoencoderTiny() = delete;

    AutoencoderTiny(shape_type const &input_shape, size_t dimension_reduction, std::vector<BufferT *> const &filters,
                    bool filters_are_packed = false)
        : Model<BufferT>(input_shape)
    {
        size_t cap0 = 0, cap1 = 0;
        shape_type prev_shape(input_shape);
        for (size_t ix = 0; ix < filters.size(); ++ix)
        {
            const uint32_t channels = ix == 4 ? (uint32_t)dimension_reduction : 128U;
            Layer<BufferT> *l = this->add(new Conv2DLayer<BufferT>(prev_shape, 1, 1, 1, PADDING_V, channels,
                                                                   *filters[ix], filters_are_packed, RELU));
            prev_shape = l->output_shape();
            if (ix == 0) cap0 = std::max(cap0, l->output_size());
            else cap1 = std::max(cap1, l->output_size());
        }
        cap0 = std::max(cap0, cap1);      // the two tensors trade places after every layer
        m_buffer_0.reset(new Tensor<BufferT>(cap0));
        m_buffer_1.reset(new Tensor<BufferT>(std::max<size_t>(cap1, 1)));
    }

    virtual ~AutoencoderTiny() {}

    virtual std::vector<Tensor<BufferT> *> inference(Tensor<BufferT> const *input_tensor)
    {
        Tensor<BufferT> *a = m_buffer_0.get(), *b = m_buffer_1.get();
        size_t l = 0;
        if (this->m_layers.empty()) return {a};
        this->m_layers[l++]->compute_output({input_tensor}, a);
        while (l < this->m_layers.size())
        {
            this->m_layers[l++]->compute_output({a}, b);
            std::swap(a, b);
        }
        return {a};
    }

private:
    std::unique_ptr<Tensor<BufferT>> m_buffer_0, m_buffer_1;
};

} // namespace small
