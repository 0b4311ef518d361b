// RouteLayer: passes one tensor through, or concatenates two along the channel axis (Darknet's
// "route"; reference include/small/RouteLayer.hpp:24-163).  With packed tensors the concatenation
// is two contiguous copies per image (small::Concat).
#pragma once

#include "Layer.hpp"

namespace small
{

template <typename BufferT>
class RouteLayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    RouteLayer(shape_type const &input0_shape)
        : Layer<BufferT>(input0_shape), m_num_inputs(1U), m_input0_shape(input0_shape), m_input1_shape({0, 0, 0, 0})
    {
    }

    RouteLayer(shape_type const &input0_shape, shape_type const &input1_shape)
        : Layer<BufferT>(), m_num_inputs(2U), m_input0_shape(input0_shape), m_input1_shape(input1_shape)
    {
        if (input1_shape[BATCH] != input0_shape[BATCH] || input1_shape[HEIGHT] != input0_shape[HEIGHT] ||
            input1_shape[WIDTH] != input0_shape[WIDTH])
            throw std::invalid_argument("RouteLayer ctor ERROR: predecessors do not have same output shape.");
        shape_type out = input0_shape;
        out[CHANNEL] = input0_shape[CHANNEL] + input1_shape[CHANNEL];
        this->set_output_shape(out);
    }

    virtual ~RouteLayer() {}

    virtual void compute_output(std::vector<Tensor<BufferT> const *> input, Tensor<BufferT> *output) const
    {
        if (input.size() != m_num_inputs)
            throw std::invalid_argument("RouteLayer::compute_output() ERROR: incorrect number of input buffers.");
        if (input[0]->shape() != m_input0_shape)
            throw std::invalid_argument("RouteLayer::compute_output() ERROR: incorrect input[0] buffer shape.");
        if (m_num_inputs == 2 && input[1]->shape() != m_input1_shape)
            throw std::invalid_argument("RouteLayer::compute_output() ERROR: incorrect input[1] buffer shape.");
        if (output->capacity() < this->output_size())
            throw std::invalid_argument("RouteLayer::compute_output() ERROR: insufficient output buffer space.");
        auto const &os = this->output_shape();
        if (m_num_inputs == 1)
        {
            if (input[0] == output) return;
            detail::hip_check(small_hip_memcpy_d2d(output->buffer().device_out(), input[0]->buffer().device_in(),
                                                   this->output_size() * sizeof(value_type),
                                                   detail::current_stream()),
                              "RouteLayer copy");
        }
        else
        {
            batched::Concat((int)os[BATCH], (uint32_t)m_input0_shape[CHANNEL], (uint32_t)m_input1_shape[CHANNEL],
                            (uint32_t)m_input0_shape[HEIGHT], (uint32_t)m_input0_shape[WIDTH], input[0]->buffer(),
                            input[1]->buffer(), output->buffer());
        }
        output->set_shape(os);
    }

private:
    uint32_t const m_num_inputs;
    shape_type const m_input0_shape;
    shape_type const m_input1_shape;
};

} // namespace small
