// Darknet: builds a DAGModel from a Darknet .cfg file and its .weights file (same constructor, accessors,
// supported blocks, defaults and weight order as the reference's include/small/models/Darknet.hpp:40-1046):
//   [net] / [network]            height, width, channels  -> input shape {batch, C, H, W}
//   [convolutional] / [conv]     batch_normalize, filters, size, stride, pad (1 -> 'f' padding, 0 -> 'v'),
//                                activation (leaky with slope 0.1 | relu | linear)
//   [maxpool] / [max]            size, stride ('f' padding always)
//   [shortcut]                   from (relative)          -> AddLayer onto the previous layer's output
//   [route]                      layers (1 or 2, relative when negative)
//   [upsample]                   stride
//   [yolo]                       mask, anchors, classes   -> YOLOLayer on the masked anchors
// Any other block is reported on stderr and makes the constructor throw once the file has been read.
// Weights file: 20 header bytes (3 x uint32 version, uint64 images seen), then float32 values in layer order; a
// convolution with batch normalisation stores beta, gamma, running mean, running variance (eps 1e-5), then
// the filters [Co][Ci][k][k]; without it the bias, then the filters.
//
// What differs: the file is read block by block into key/value lists before any layer is built (no seeking), a
// weights file that ends early is an error instead of a read past the buffer, and an optional batch extent
// makes every layer run `batch` images per call.
#pragma once

#include <cstdint>
#include <fstream>
#include <iostream>
#include <string>
#include <utility>
#include <vector>

#include "../Conv2DLayer.hpp"
#include "../DAGModel.hpp"
#include "../MaxPool2DLayer.hpp"
#include "../RouteLayer.hpp"
#include "../UpSample2DLayer.hpp"
#include "../YOLOLayer.hpp"
#include "../non_max_suppression.hpp"

namespace small
{

template <typename BufferT>
class Darknet : public DAGModel<BufferT>
{
public:
    Darknet() = delete;

    Darknet(std::string cfg_pathname, std::string weights_pathname, bool save_outputs = false, uint32_t batch = 1)
        : DAGModel<BufferT>({0, 0, 0, 0}, save_outputs), m_num_classes(0)
    {
        const size_t max_buffer_size = parse_cfg_and_weights(cfg_pathname, weights_pathname, batch);
        this->initializeDAG(max_buffer_size);
    }

    virtual ~Darknet() {}

    size_t get_num_classes() const { return m_num_classes; }

    // Detections of every head above the confidence threshold (objectness AND class score; one detection per
    // such class), then per-class non-maximum suppression.  outputs: one [1, 1, predictions, 5 + classes]
    // tensor per YOLO layer, as inference() returns them (image 0 of a batch).
    std::vector<Detection> process_outputs(std::vector<Tensor<BufferT> *> const &outputs, float confidence_threshold,
                                           float iou_threshold)
    {
        std::vector<Detection> predictions;
        for (auto *t : outputs)
        {
            if (t->shape()[3] != 5 + m_num_classes)
                throw std::invalid_argument("Darknet::process_outputs ERROR: unexpected record length.");
            BufferT const &buf = t->buffer();
            const size_t rec = t->shape()[3];
            for (size_t p = 0; p < t->shape()[2]; ++p)
            {
                const size_t at = p * rec;
                if (!(buf[at + 4] > confidence_threshold)) continue;
                for (size_t c = 0; c < m_num_classes; ++c)
                    if (buf[at + 5 + c] > confidence_threshold)
                        predictions.push_back(Detection{{buf[at + 0], buf[at + 1], buf[at + 2], buf[at + 3]},
                                                        buf[at + 4], buf[at + 5 + c], c});
            }
        }
        return basic_nms(predictions, iou_threshold);
    }

private:
    typedef std::vector<std::pair<std::string, std::string>> Fields;
    struct Block
    {
        std::string name;
        size_t line;
        Fields fields;
    };

    size_t m_num_classes;

    static std::vector<Block> read_blocks(std::string const &cfg_path)
    {
        std::ifstream cfg(cfg_path);
        if (!cfg)
            throw std::invalid_argument("Darknet::parse_cfg_and_weights ERROR: Could not open cfg file: " + cfg_path);
        std::vector<Block> blocks;
        std::string line;
        size_t line_num = 0;
        while (std::getline(cfg, line))
        {
            ++line_num;
            std::string s;
            for (char ch : line)
                if (ch != ' ' && ch != '\r' && ch != '\t') s.push_back(ch);
            if (s.empty() || s[0] == '#') continue;
            if (s[0] == '[') { blocks.push_back(Block{s, line_num, {}}); continue; }
            if (blocks.empty()) continue;                 // text before the first block
            const size_t eq = s.find('=');
            blocks.back().fields.emplace_back(s.substr(0, eq), eq == std::string::npos ? std::string() : s.substr(eq + 1));
        }
        return blocks;
    }

    static std::vector<int> int_list(std::string const &s)
    {
        std::vector<int> v;
        size_t last = 0, next;
        while ((next = s.find(',', last)) != std::string::npos)
        {
            v.push_back(std::stoi(s.substr(last, next - last)));
            last = next + 1;
        }
        v.push_back(std::stoi(s.substr(last)));
        return v;
    }

    static ActivationType activation_of(std::string const &v)
    {
        if (v == "leaky") return LEAKY;
        if (v == "relu") return RELU;
        if (v != "linear") std::cerr << "WARNING: Activation type " << v << " not supported. Using NONE\n";
        return NONE;
    }

    // the next n floats of the weights file as a buffer
    struct Weights
    {
        std::vector<float> data;
        size_t at = 0;
        BufferT take(size_t n)
        {
            if (at + n > data.size())
                throw std::invalid_argument("Darknet::parse_cfg_and_weights ERROR: the weights file ends early.");
            BufferT b(n);
            std::copy(data.begin() + at, data.begin() + at + n, b.data());
            at += n;
            return b;
        }
    };

    static Weights read_weights(std::string const &path)
    {
        std::ifstream f(path, std::ios::binary | std::ios::ate);
        if (!f)
            throw std::invalid_argument("Darknet::parse_cfg_and_weights ERROR: Could not open weights file: " + path);
        const std::streamoff bytes = f.tellg();
        Weights w;
        if (bytes > 20)
        {
            w.data.resize((size_t)(bytes - 20) / sizeof(float));
            f.seekg(20);                                   // 3 x uint32 version + uint64 images seen
            f.read(reinterpret_cast<char *>(w.data.data()), (std::streamsize)(w.data.size() * sizeof(float)));
        }
        return w;
    }

    Layer<BufferT> *make_conv(Block const &b, shape_type const &in, Weights &w)
    {
        bool bn = false;
        size_t filters = 0, size = 0, stride = 0;
        PaddingEnum pad = PADDING_F;
        ActivationType act = NONE;
        for (auto const &kv : b.fields)
        {
            if (kv.first == "batch_normalize") bn = kv.second == "1";
            else if (kv.first == "filters") filters = std::stoul(kv.second);
            else if (kv.first == "size") size = std::stoul(kv.second);
            else if (kv.first == "stride") stride = std::stoul(kv.second);
            else if (kv.first == "pad") pad = kv.second == "0" ? PADDING_V : PADDING_F;
            else if (kv.first == "activation") act = activation_of(kv.second);
        }
        const size_t nfilt = filters * size * size * in[CHANNEL];
        if (bn)
        {
            BufferT beta = w.take(filters), gamma = w.take(filters), mean = w.take(filters), var = w.take(filters);
            BufferT filt = w.take(nfilt);
            return new Conv2DLayer<BufferT>(in, size, size, stride, pad, filters, filt, gamma, beta, mean, var, 1.e-5,
                                            false, act, 0.1);
        }
        BufferT bias = w.take(filters);
        BufferT filt = w.take(nfilt);
        return new Conv2DLayer<BufferT>(in, size, size, stride, pad, filters, filt, bias, false, act, 0.1);
    }

    Layer<BufferT> *make_yolo(Block const &b, shape_type const &in)
    {
        std::vector<int> mask, flat;
        size_t classes = 0;
        for (auto const &kv : b.fields)
        {
            if (kv.first == "mask") mask = int_list(kv.second);
            else if (kv.first == "anchors") flat = int_list(kv.second);
            else if (kv.first == "classes")
            {
                classes = std::stoul(kv.second);
                if (m_num_classes == 0) m_num_classes = classes;
                else if (classes != m_num_classes)
                    throw std::invalid_argument("Darknet::parse_yolo ERROR: inconsistent number of classes.");
            }
        }
        if (mask.empty() || flat.size() < 2)
            throw std::invalid_argument("Darknet::parse_yolo ERROR: missing anchors or mask fields.");
        std::vector<std::pair<uint32_t, uint32_t>> anchors;
        for (int m : mask)
        {
            if (m < 0 || 2 * (size_t)m + 1 >= flat.size())
                throw std::invalid_argument("Darknet::parse_yolo ERROR: mask index out of range.");
            anchors.emplace_back((uint32_t)flat[2 * m], (uint32_t)flat[2 * m + 1]);
        }
        return new YOLOLayer<BufferT>(in, anchors, classes, this->m_input_shape[HEIGHT]);
    }

    size_t parent_index(int rel_or_abs, Block const &b) const
    {
        const long n = (long)this->m_layers.size();
        const long idx = rel_or_abs < 0 ? n + rel_or_abs : rel_or_abs;
        if (idx < 0 || idx >= n)
            throw std::invalid_argument("Darknet ERROR: " + b.name + " on line " + std::to_string(b.line) +
                                        " refers to a layer that does not exist.");
        return (size_t)idx;
    }

    size_t parse_cfg_and_weights(std::string const &cfg_path, std::string const &weights_path, uint32_t batch)
    {
        const std::vector<Block> blocks = read_blocks(cfg_path);
        Weights weights = read_weights(weights_path);
        size_t max_buffer_size = 0;
        bool error = false;
        shape_type prev_shape = {0, 0, 0, 0};

        for (Block const &b : blocks)
        {
            if (b.name == "[network]" || b.name == "[net]")
            {
                shape_type s = {batch, 0, 0, 0};
                for (auto const &kv : b.fields)
                {
                    if (kv.first == "height") s[HEIGHT] = std::stoul(kv.second);
                    else if (kv.first == "width") s[WIDTH] = std::stoul(kv.second);
                    else if (kv.first == "channels") s[CHANNEL] = std::stoul(kv.second);
                }
                if (s[0] == 0 || s[1] == 0 || s[2] == 0 || s[3] == 0)
                    throw std::invalid_argument("Darknet::parse_network ERROR: a zero input dimension.");
                this->m_input_shape = prev_shape = s;
                max_buffer_size = std::max(max_buffer_size, compute_size(s));
                continue;
            }
            const size_t idx = this->m_layers.size();
            std::vector<size_t> parents;
            if (idx > 0) parents.push_back(idx - 1);
            Layer<BufferT> *layer = nullptr;
            if (b.name == "[convolutional]" || b.name == "[conv]") layer = make_conv(b, prev_shape, weights);
            else if (b.name == "[maxpool]" || b.name == "[max]")
            {
                size_t size = 0, stride = 0;
                for (auto const &kv : b.fields)
                {
                    if (kv.first == "size") size = std::stoul(kv.second);
                    else if (kv.first == "stride") stride = std::stoul(kv.second);
                }
                layer = new MaxPool2DLayer<BufferT>(prev_shape, size, size, stride, PADDING_F);
            }
            else if (b.name == "[shortcut]")
            {
                int from = 0;
                for (auto const &kv : b.fields)
                {
                    if (kv.first == "from") from = std::stoi(kv.second);
                    else if (kv.first == "activation" && activation_of(kv.second) != NONE)
                        std::cerr << "WARNING: Activation type " << kv.second << " not supported for shortcut layer\n";
                }
                if (from >= 0 || idx == 0)
                    throw std::invalid_argument("Darknet ERROR: [shortcut] needs a negative 'from' and a previous layer.");
                const size_t other = parent_index(from, b);
                layer = new AddLayer<BufferT>(prev_shape, this->m_layers[other]->output_shape());
                parents = {idx - 1, other};
            }
            else if (b.name == "[route]")
            {
                std::vector<int> ids;
                for (auto const &kv : b.fields)
                    if (kv.first == "layers") ids = int_list(kv.second);
                parents.clear();
                for (int id : ids) parents.push_back(parent_index(id, b));
                if (parents.size() == 1) layer = new RouteLayer<BufferT>(this->m_layers[parents[0]]->output_shape());
                else if (parents.size() == 2)
                    layer = new RouteLayer<BufferT>(this->m_layers[parents[0]]->output_shape(),
                                                    this->m_layers[parents[1]]->output_shape());
                else throw std::invalid_argument("ERROR: route layer must have only 1 or 2 layers");
            }
            else if (b.name == "[upsample]")
            {
                uint32_t stride = 0;
                for (auto const &kv : b.fields)
                    if (kv.first == "stride") stride = (uint32_t)std::stoul(kv.second);
                layer = new UpSample2DLayer<BufferT>(prev_shape, stride);
            }
            else if (b.name == "[yolo]") layer = make_yolo(b, prev_shape);
            else
            {
                error = true;
                std::cerr << "[ERROR]: Unsupported block (" << b.name << ") on line " << b.line << "\n";
                continue;
            }
            this->m_graph.add_vertex(idx);
            for (size_t p : parents) this->m_graph.add_edge(p, idx);
            this->add(layer);
            prev_shape = layer->output_shape();
            max_buffer_size = std::max(max_buffer_size, compute_size(prev_shape));
        }
        if (error) throw std::invalid_argument("Failure to build model. Check errors and try again.");
        if (this->m_layers.empty() || this->m_input_shape[CHANNEL] == 0)
            throw std::invalid_argument("Darknet ERROR: the cfg file defines no network.");
        return max_buffer_size;
    }
};

} // namespace small
