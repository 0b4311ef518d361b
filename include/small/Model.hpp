// Model: owns a list of layers and runs them on an input tensor (reference
// include/small/Model.hpp:22-94).  Output tensors stay owned by the model.
#pragma once

#include <memory>
#include <vector>

#include "Layer.hpp"

namespace small
{

template <typename BufferT>
class Model
{
public:
    Model() = delete;
    Model(shape_type const &input_shape) : m_input_shape(input_shape) {}
    Model(Model const &) = delete;
    Model &operator=(Model const &) = delete;

    virtual ~Model()
    {
        for (auto *layer : m_layers) delete layer;
    }

    shape_type const &get_input_shape() const { return m_input_shape; }

    virtual std::vector<Tensor<BufferT> *> inference(Tensor<BufferT> const *input) = 0;

    size_t get_num_layers() const { return m_layers.size(); }
    Layer<BufferT> *get_layer(size_t idx)
    {
        if (idx >= m_layers.size()) throw std::invalid_argument("ERROR: invalid layer index.");
        return m_layers[idx];
    }

    // hands the layers (and their ownership) to the caller and leaves the model empty; used to re-host a
    // model's layer list in another executor (DAGModel::adopt_layers)
    std::vector<Layer<BufferT> *> release_layers()
    {
        std::vector<Layer<BufferT> *> out;
        out.swap(m_layers);
        return out;
    }

protected:
    // takes ownership; returns the layer for chaining on its output_shape()
    Layer<BufferT> *add(Layer<BufferT> *layer)
    {
        m_layers.push_back(layer);
        return layer;
    }

    shape_type m_input_shape;
    std::vector<Layer<BufferT> *> m_layers;
};

} // namespace small
