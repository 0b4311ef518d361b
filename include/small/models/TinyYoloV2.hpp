// TinyYoloV2: the convolutional trunk as the reference assembles it
// (include/small/models/TinyYoloV2.hpp:133-265): 6 x (Conv2D 3x3 'f' + activation, MaxPool2D 2x2 'f' with
// strides 2,2,2,2,2,1), two more 3x3 convolutions and a 1x1 output convolution, channels 16 doubling
// per block.  The reference hard-codes ReLU everywhere and 16 output channels; activation kind, slope,
// output channel count and whether the output layer is activated are constructor arguments here
// (defaults = the reference), so the original network (LeakyReLU 0.1, 125 linear outputs) can be built.
#pragma once

#include <algorithm>
#include <vector>

#include "../Conv2DLayer.hpp"
#include "../MaxPool2DLayer.hpp"
#include "../Model.hpp"

namespace small
{

template <typename BufferT>
class TinyYoloV2 : public Model<BufferT>
{
public:
    TinyYoloV2() = delete;

    // filters: 9 buffers in layer order
    TinyYoloV2(shape_type const &input_shape, std::vector<BufferT *> const &filters, bool filters_are_packed = false,
               ActivationType activation = RELU, float leaky_slope = 0.1f, uint32_t num_outputs = 16,
               bool activate_output = true)
        : Model<BufferT>(input_shape)
    {
        if (filters.size() != 9) throw std::invalid_argument("TinyYoloV2 ctor ERROR: 9 filter buffers expected.");
        static const uint32_t pool_strides[6] = {2, 2, 2, 2, 2, 1};
        size_t f = 0, cap0 = 0, cap1 = 0;
        uint32_t channels = 16;
        shape_type shape = input_shape;
        for (int blk = 0; blk < 6; ++blk)
        {
            Layer<BufferT> *conv = this->add(new Conv2DLayer<BufferT>(shape, 3, 3, 1, PADDING_F, channels,
                                                                      *filters[f++], filters_are_packed, activation,
                                                                      leaky_slope));
            cap1 = std::max(cap1, conv->output_size());
            Layer<BufferT> *pool = this->add(
                new MaxPool2DLayer<BufferT>(conv->output_shape(), 2, 2, pool_strides[blk], PADDING_F));
            cap0 = std::max(cap0, pool->output_size());
            shape = pool->output_shape();
            channels *= 2;
        }
        for (int tail = 0; tail < 3; ++tail)
        {
            const bool last = tail == 2;
            Layer<BufferT> *conv = this->add(new Conv2DLayer<BufferT>(
                shape, last ? 1 : 3, last ? 1 : 3, 1, PADDING_F, last ? num_outputs : channels, *filters[f++],
                filters_are_packed, (last && !activate_output) ? NONE : activation, leaky_slope));
            cap1 = std::max(cap1, conv->output_size());
            shape = conv->output_shape();
        }
        cap0 = std::max(cap0, cap1);   // the tail swaps the two tensors
        m_buffer_0.reset(new Tensor<BufferT>(cap0));
        m_buffer_1.reset(new Tensor<BufferT>(cap0));
        m_buffer_2.reset(new Tensor<BufferT>(cap0));
    }

    virtual ~TinyYoloV2() {}

    virtual std::vector<Tensor<BufferT> *> inference(Tensor<BufferT> const *input_tensor)
    {
        // b takes convolution outputs; the pooled maps alternate between a and c, so that the one-launch
        // convolution + pooling never writes over its own input
        Tensor<BufferT> *a = m_buffer_0.get(), *b = m_buffer_1.get(), *c = m_buffer_2.get();
        size_t l = 0;
        Tensor<BufferT> const *src = input_tensor;
        for (int blk = 0; blk < 6; ++blk)
        {
            // convolution + activation + pooling: one call (one launch where the pool is 2x2 stride 2 on a map the
            // kernel's tiles fill; the wrapper falls back to the two launches through b otherwise)
            auto *conv = static_cast<Conv2DLayer<BufferT> *>(this->m_layers[l]);
            auto *pool = static_cast<MaxPool2DLayer<BufferT> *>(this->m_layers[l + 1]);
            if (conv->fusable_with_pool())
                conv->compute_output_pooled(src, pool->window(), pool->output_shape(), b, a);
            else
            {
                conv->compute_output({src}, b);
                pool->compute_output({b}, a);
            }
            l += 2;
            src = a;
            std::swap(a, c);          // the next block reads what was just written (now c) and writes the other one
        }
        std::swap(a, c);              // a = the last pooled map
        for (int tail = 0; tail < 3; ++tail)
        {
            this->m_layers[l++]->compute_output({a}, b);
            std::swap(a, b);
        }
        return {a};
    }

private:
    std::unique_ptr<Tensor<BufferT>> m_buffer_0, m_buffer_1, m_buffer_2;
};

} // namespace small
