// YOLOLayer: decodes one detection head into box records (same constructor, output shape and arithmetic as the
// reference's include/small/YOLOLayer.hpp:43-239): input [batch][padded channels][H][W] with channel
// a*(5+classes)+f = field f of masked anchor a, output [batch][1][anchors*H*W][5+classes] =
// {centre x, centre y, width, height, objectness, class scores} in input-image pixels.
//
// What differs underneath: the reference unpacks the tensor and decodes on the host; here one kernel reads
// the packed tensor and writes the records (small_hip_yolo_decode_f32), and the batch extent is honoured.
#pragma once

#include <utility>
#include <vector>

#include "Layer.hpp"

namespace small
{

template <typename BufferT>
class YOLOLayer : public Layer<BufferT>
{
public:
    typedef typename BufferT::value_type value_type;

    YOLOLayer(shape_type const &input_shape, std::vector<std::pair<uint32_t, uint32_t>> masked_anchors,
              size_t num_classes, size_t input_img_size)
        : Layer<BufferT>(),
          m_input_shape(input_shape),
          m_anchors(masked_anchors),
          m_num_classes(num_classes),
          m_num_outputs(num_classes + 5),
          m_num_pred(masked_anchors.size() * input_shape[HEIGHT] * input_shape[WIDTH]),
          m_image_size(input_img_size)
    {
        static_assert(std::is_same<BufferT, FloatBuffer>::value, "YOLOLayer is a float32 layer");
        if (m_anchors.empty() || m_anchors.size() > 8)
            throw std::invalid_argument("YOLOLayer::ctor ERROR: 1 to 8 anchors per head are supported.");
        if (m_anchors.size() * m_num_outputs > input_shape[CHANNEL])
            throw std::invalid_argument("YOLOLayer::ctor ERROR: too few input channels for the anchors.");
        for (auto const &a : m_anchors)
        {
            m_anchors_flat.push_back(a.first);
            m_anchors_flat.push_back(a.second);
        }
        this->set_output_shape({input_shape[BATCH], 1U, m_num_pred, m_num_outputs});
    }

    virtual ~YOLOLayer() {}

    size_t get_num_pred() const { return m_num_pred; }
    size_t get_num_outputs() const { return m_num_outputs; }

    virtual void compute_output(std::vector<Tensor<BufferT> const *> input, Tensor<BufferT> *output) const
    {
        this->check_single_input("YOLOLayer", input, m_input_shape, output);
        detail::raise<BufferT>(
            small_hip_yolo_decode_f32((int)m_input_shape[BATCH], (int)m_input_shape[CHANNEL], (int)m_input_shape[HEIGHT],
                                      (int)m_input_shape[WIDTH], (int)m_anchors.size(), m_anchors_flat.data(),
                                      (int)m_num_classes, (int)m_image_size, input[0]->buffer().device_in(),
                                      output->buffer().device_out(), detail::st()),
            "YOLOLayer");
        output->set_shape(this->output_shape());
    }

private:
    shape_type const m_input_shape;
    std::vector<std::pair<uint32_t, uint32_t>> const m_anchors;
    std::vector<uint32_t> m_anchors_flat;
    size_t const m_num_classes;
    size_t const m_num_outputs;
    size_t const m_num_pred;
    size_t const m_image_size;
};

} // namespace small
