// DAGModel: a model whose layers form a directed acyclic graph (one source; routes and shortcuts have several
// parents).  Same interface and buffer discipline as the reference's include/small/DAGModel.hpp:33-319: layers
// run in topological order, each output lives in a pooled tensor until its last consumer has run, and a layer
// that accumulates (AddLayer, PartialConv2DLayer) writes into the tensor of its FIRST parent, which must have
// no other consumer.  With save_outputs every layer's output stays readable until the next inference().
// A float32 convolution whose only consumer is a max-pooling layer runs together with it, and so does one whose only
// consumer is a depthwise layer that it can take into its launch (neither with save_outputs).
#pragma once

#include <deque>
#include <typeinfo>
#include <vector>

#include "AddLayer.hpp"
#include "Conv2DLayer.hpp"
#include "DepthwiseConv2DLayer.hpp"
#include "MaxPool2DLayer.hpp"
#include "Model.hpp"
#include "PartialConv2DLayer.hpp"
#include "utils/BufferPool.hpp"
#include "utils/Graph.hpp"

namespace small
{

template <typename BufferT>
class DAGModel : public Model<BufferT>
{
public:
    DAGModel() = delete;
    DAGModel(shape_type const &input_shape, bool save_outputs = false)
        : Model<BufferT>(input_shape), m_save_outputs(save_outputs)
    {
    }

    virtual ~DAGModel()
    {
        for (auto *t : m_cached) delete t;
    }

    virtual std::vector<Tensor<BufferT> *> inference(Tensor<BufferT> const *input)
    {
        if (input->shape() != this->m_input_shape)
            throw std::runtime_error("Input shape does not match model input shape");
        // tensors kept from the previous pass (saved outputs) go back to the pool
        for (size_t i = 0; i < m_cached.size(); ++i) release(i);

        for (size_t step = 0; step < m_order.size(); ++step)
        {
            const size_t cur = m_order[step];
            std::vector<Tensor<BufferT> const *> ins;
            Tensor<BufferT> *out = nullptr;
            auto const &parents = m_graph.in_neighbors(cur);
            if (step == 0)
            {
                ins.push_back(input);
                out = m_pool.pop_buffer();
            }
            else if (accumulates(cur))
            {
                if (parents.size() != 2 || m_count[parents[0]] != 1 || m_cached[parents[0]] == nullptr)
                    throw std::runtime_error("DAGModel ERROR: an accumulating layer needs two parents, the first "
                                             "with no other consumer.");
                out = m_cached[parents[0]];
                m_cached[parents[0]] = nullptr;
                m_count[parents[0]] = 0;
                ins.push_back(m_cached[parents[1]]);
            }
            else
            {
                for (size_t p : parents) ins.push_back(m_cached[p]);
                out = m_pool.pop_buffer();
            }
            if (!m_save_outputs && m_pool_after[cur] != NO_POOL && step + 1 < m_order.size() &&
                m_order[step + 1] == m_pool_after[cur])
            {
                // convolution whose only consumer is a max-pooling layer: both in one call (one launch for a 2x2
                // stride-2 pool); the convolution's own output is never cached
                const size_t pl = m_pool_after[cur];
                auto *conv = static_cast<Conv2DLayer<BufferT> *>(this->m_layers[cur]);
                auto *pool = static_cast<MaxPool2DLayer<BufferT> *>(this->m_layers[pl]);
                Tensor<BufferT> *inter = m_pool.pop_buffer();
                try
                {
                    conv->compute_output_pooled(ins[0], pool->window(), pool->output_shape(), inter, out);
                }
                catch (...)
                {
                    m_pool.push_buffer(inter);
                    m_pool.push_buffer(out);
                    throw;
                }
                m_pool.push_buffer(inter);
                if (step != 0)
                    for (size_t k = 0; k < parents.size(); ++k)
                        if (m_count[parents[k]] > 0 && --m_count[parents[k]] == 0) release(parents[k]);
                m_count[pl] = m_graph.out_neighbors(pl).size();
                m_cached[pl] = out;
                ++step;                  // the pooling layer has run
                continue;
            }
            if (!m_save_outputs && m_dw_after[cur] != NO_POOL && step + 1 < m_order.size() && m_order[step + 1] == m_dw_after[cur])
            {
                // convolution whose only consumer is a depthwise layer it can run in its own launch: one call, the
                // convolution's output is never written or cached
                const size_t dl = m_dw_after[cur];
                auto *conv = static_cast<Conv2DLayer<BufferT> *>(this->m_layers[cur]);
                auto *dw = static_cast<DepthwiseConv2DLayer<BufferT> *>(this->m_layers[dl]);
                try
                {
                    conv->compute_output_depthwise(ins[0], *dw, out);
                }
                catch (...)
                {
                    m_pool.push_buffer(out);
                    throw;
                }
                if (step != 0)
                    for (size_t k = 0; k < parents.size(); ++k)
                        if (m_count[parents[k]] > 0 && --m_count[parents[k]] == 0) release(parents[k]);
                m_count[dl] = m_graph.out_neighbors(dl).size();
                m_cached[dl] = out;
                ++step;                  // the depthwise layer has run
                continue;
            }
            try
            {
                this->m_layers[cur]->compute_output(ins, out);
            }
            catch (...)
            {
                m_pool.push_buffer(out);     // nothing refers to it yet: back to the pool, then let the caller see the error
                throw;
            }
            // a parent's tensor returns to the pool after its last consumer; the stream orders the reuse
            if (step != 0)
                for (size_t k = accumulates(cur) ? 1 : 0; k < parents.size(); ++k)
                    if (m_count[parents[k]] > 0 && --m_count[parents[k]] == 0 && !m_save_outputs) release(parents[k]);
            m_count[cur] = m_graph.out_neighbors(cur).size();
            m_cached[cur] = out;
        }

        // the tensors handed out stay the model's: they are recycled by the next inference() call
        std::vector<Tensor<BufferT> *> outs;
        for (size_t o : m_outputs) outs.push_back(m_cached[o]);
        return outs;
    }

    std::vector<size_t> const &get_parent_ids(size_t layer_num) const
    {
        if (layer_num >= m_graph.get_num_nodes())
            throw std::invalid_argument("Darknet::get_parent_ids ERROR: invalid layer_num.");
        return m_graph.in_neighbors(layer_num);
    }

    std::vector<Tensor<BufferT> *> get_layer_outputs() const
    {
        if (!m_save_outputs) throw std::invalid_argument("Saving layer outputs is disabled.");
        return m_cached;
    }

protected:
    // call once the layers and the graph are complete; every pooled tensor holds max_buffer_size elements
    void initializeDAG(size_t max_buffer_size)
    {
        m_outputs = m_graph.sinks();
        m_order = m_graph.topological_sort();
        auto const sources = m_graph.sources();
        if (sources.size() != 1 || m_order.empty() || m_order[0] != sources[0] ||
            m_graph.get_num_nodes() != this->m_layers.size())
            throw std::invalid_argument("ERROR: darknet graph input node error.");
        const size_t num_bufs = 2 + (m_graph.max_width(sources[0]) - 1) + (m_outputs.size() - 1);
        m_pool = BufferPool<BufferT>(max_buffer_size, num_bufs);
        m_count.assign(this->m_layers.size(), 0);
        m_cached.assign(this->m_layers.size(), nullptr);
        // convolution -> max-pool pairs that can run as one call: the pool is the convolution's only consumer
        // and the convolution the pool's only input
        m_pool_after.assign(this->m_layers.size(), NO_POOL);
        for (size_t i = 0; i < this->m_layers.size(); ++i)
        {
            auto *conv = dynamic_cast<Conv2DLayer<BufferT> *>(this->m_layers[i]);
            auto const &outs = m_graph.out_neighbors(i);
            if (!conv || !conv->fusable_with_pool() || outs.size() != 1) continue;
            if (dynamic_cast<MaxPool2DLayer<BufferT> *>(this->m_layers[outs[0]]) && m_graph.in_neighbors(outs[0]).size() == 1)
                m_pool_after[i] = outs[0];
        }
        // convolution -> depthwise pairs that run as one launch (Conv2DLayer::fusable_with_depthwise), same conditions
        m_dw_after.assign(this->m_layers.size(), NO_POOL);
        for (size_t i = 0; i < this->m_layers.size(); ++i)
        {
            auto *conv = dynamic_cast<Conv2DLayer<BufferT> *>(this->m_layers[i]);
            auto const &outs = m_graph.out_neighbors(i);
            if (!conv || outs.size() != 1 || m_graph.in_neighbors(outs[0]).size() != 1) continue;
            auto *dw = dynamic_cast<DepthwiseConv2DLayer<BufferT> *>(this->m_layers[outs[0]]);
            if (dw && conv->fusable_with_depthwise(*dw)) m_dw_after[i] = outs[0];
        }
    }

    // Takes over a finished layer list as the graph's vertices 0..n-1 and initialises the DAG.  parents[i] lists
    // the layers feeding layer i, in input order (for an accumulating layer: the tensor it adds onto first);
    // an empty list means the previous layer, so an empty `parents` describes a plain chain.
    void adopt_layers(std::vector<Layer<BufferT> *> layers, std::vector<std::vector<size_t>> const &parents = {})
    {
        size_t max_size = compute_size(this->m_input_shape);
        for (size_t i = 0; i < layers.size(); ++i)
        {
            this->add(layers[i]);
            max_size = std::max(max_size, layers[i]->output_size());
            m_graph.add_vertex(i);
            if (i < parents.size() && !parents[i].empty())
                for (size_t p : parents[i]) m_graph.add_edge(p, i);
            else if (i > 0)
                m_graph.add_edge(i - 1, i);
        }
        initializeDAG(max_size);
    }

    Graph m_graph;

private:
    bool accumulates(size_t idx) const
    {
        std::type_info const &t = typeid(*this->m_layers[idx]);
        return t == typeid(AddLayer<BufferT>) || t == typeid(PartialConv2DLayer<BufferT>);
    }

    void release(size_t idx)
    {
        if (m_cached[idx] != nullptr) m_pool.push_buffer(m_cached[idx]);
        m_cached[idx] = nullptr;
        m_count[idx] = 0;
    }

    static constexpr size_t NO_POOL = (size_t)-1;

    bool m_save_outputs;
    std::vector<size_t> m_pool_after;          // per layer: the max-pooling layer fused behind it, or NO_POOL
    std::vector<size_t> m_dw_after;            // per layer: the depthwise layer that runs in its launch, or NO_POOL
    std::deque<size_t> m_order;
    BufferPool<BufferT> m_pool;
    std::vector<size_t> m_count;
    std::vector<Tensor<BufferT> *> m_cached;
    std::vector<Graph::VertexID> m_outputs;
};

} // namespace small
