// Layer: base class of the layer objects (reference include/small/Layer.hpp:22-76) plus the
// argument checks every compute_output() of this build shares.
//
// The reference carries shape[BATCH] through its Layer classes but computes one image; here
// the batch extent is passed on to the batched entry points, so a layer built for
// {N, C, H, W} processes N consecutive packed images per call.
#pragma once

#include <string>
#include <vector>

#include "Tensor.hpp"
#include "interface.hpp"   // ActivationType {NONE, RELU, LEAKY, SOFTMAX}
#include "utils.hpp"

namespace small
{

template <typename BufferT>
class Layer
{
public:
    Layer() : m_output_shape({0, 0, 0, 0}), m_output_size(0) {}
    Layer(shape_type const &output_shape) { set_output_shape(output_shape); }
    virtual ~Layer() {}

    size_t output_size() const { return m_output_size; }
    shape_type const &output_shape() const { return m_output_shape; }

    // inputs by value so that callers can write compute_output({&in}, &out)
    virtual void compute_output(std::vector<Tensor<BufferT> const *> input, Tensor<BufferT> *output) const = 0;

    // This layer as one record of a whole-model launch (small_hip_qmodel_create): kind, window, channels, filter and
    // its quantisation, ReLU flag; accum_src = ONE_LAUNCH_ACCUM_ONTO_OUTPUT when the layer accumulates onto its output
    // tensor.  The model fills in tensor ids and the tensors' quantisation.  false: the layer has no such form.
    static constexpr int ONE_LAUNCH_ACCUM_ONTO_OUTPUT = -100;
    virtual bool one_launch(small_hip_qlayer &) const { return false; }
    // the float32 form (small_hip_fmodel_create): kind, window, channels, filter, bias and activation
    virtual bool one_launch(small_hip_flayer &) const { return false; }

protected:
    void set_output_shape(shape_type const &output_shape)
    {
        m_output_shape = output_shape;
        m_output_size = compute_size(output_shape);
    }

    // "<who>::compute_output() ERROR: incorrect input buffer shape." / "... insufficient output buffer space."
    void check_single_input(char const *who, std::vector<Tensor<BufferT> const *> const &input,
                            shape_type const &expected, Tensor<BufferT> const *output) const
    {
        if (input.size() != 1 || input[0]->shape() != expected)
            throw std::invalid_argument(std::string(who) + "::compute_output() ERROR: incorrect input buffer shape.");
        if (output->capacity() < m_output_size)
            throw std::invalid_argument(std::string(who) +
                                        "::compute_output() ERROR: insufficient output buffer space.");
    }

    shape_type m_output_shape;
    size_t m_output_size;
};

namespace detail
{
// window geometry shared by the convolution and pooling layers: pads from the padding type,
// output extent from utils.hpp
struct Window
{
    uint32_t kh, kw, stride;
    uint8_t t, b, l, r;
    size_t Ho, Wo;

    Window(shape_type const &in, uint32_t kernel_height, uint32_t kernel_width, uint32_t stride_, PaddingEnum padding)
        : kh(kernel_height), kw(kernel_width), stride(stride_), t(0), b(0), l(0), r(0), Ho(0), Wo(0)
    {
        compute_padding_output_dim(in[HEIGHT], kh, stride, padding, t, b, Ho);
        compute_padding_output_dim(in[WIDTH], kw, stride, padding, l, r, Wo);
    }
};
} // namespace detail

} // namespace small
