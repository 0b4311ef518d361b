// Model: owns a list of layers and runs them on an input tensor (reference
// include/small/Model.hpp:22-94).  Output tensors stay owned by the model.
#pragma once

#include <cstdlib>
#include <memory>
#include <string>
#include <type_traits>
#include <vector>

#include "Layer.hpp"

namespace small
{

namespace detail
{
// one compute_output() call of a model's forward pass: layer, the tensor it reads, the tensor it writes (an
// accumulating layer adds onto the tensor it writes)
template <typename BufferT>
struct LaunchStep
{
    Layer<BufferT> const *layer;
    Tensor<BufferT> const *src;
    Tensor<BufferT> *dst;
};
} // namespace detail

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
        if (m_qmodel) (void)small_hip_qmodel_destroy(m_qmodel);
        if (m_fmodel) (void)small_hip_fmodel_destroy(m_fmodel);
    }

    // Small models whose tensors (and, quantised, filters) fit one compute unit's LDS run their whole forward pass as ONE
    // launch: small_hip_qmodel_forward for QUInt8Buffer, bit-identical to the layer-by-layer calls and used by default;
    // small_hip_fmodel_forward for FloatBuffer, within the float32 tolerance of them (another summation order) and
    // therefore only on request.  Only the returned tensor is written.
    // true / false: use / never use that form (environment: SMALL_HIP_TUNE=one_launch=1 / 0).
    void set_one_launch(bool on) { m_one_launch = on; }
    // true once inference() has planned (and used) the one-launch form
    bool one_launch_planned() const { return m_qmodel != nullptr || m_fmodel != nullptr; }
    // why the whole-model launch was not planned (the library's message: which limit the model exceeds); empty if it was,
    // or was never asked for.  Only "not built for this model" falls back to the layer calls; a bad argument throws.
    std::string const &one_launch_refusal() const { return m_refusal; }

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

    // Runs `steps` (the forward pass as the sequence of compute_output() calls, first step reading the model input,
    // last step writing the result) as one launch.  The launch is planned on first use and again whenever the
    // quantisation fields of a tensor change (they travel with the buffers, so they are only known at call time).
    // false: this model has no such form (a layer kind, padding or size the launch does not cover; float32) and
    // nothing was computed: the caller issues the layers one by one.
    bool forward_one_launch(std::vector<detail::LaunchStep<BufferT>> const &steps)
    {
        if constexpr (std::is_same<BufferT, QUInt8Buffer>::value)
        {
            if (!m_one_launch || steps.empty()) return false;
            if (steps.front().src->shape() != m_input_shape)
                throw std::invalid_argument("Model::inference() ERROR: incorrect input buffer shape.");
            // tensor ids in order of first use; the model input and the last destination have their own names
            std::vector<Tensor<BufferT> const *> ids;
            auto id_of = [&](Tensor<BufferT> const *t) {
                for (size_t i = 0; i < ids.size(); ++i)
                    if (ids[i] == t) return (int)i;
                ids.push_back(t);
                return (int)ids.size() - 1;
            };
            std::vector<small_hip_qlayer> recs(steps.size());
            std::vector<int32_t> sig;
            for (size_t i = 0; i < steps.size(); ++i)
            {
                small_hip_qlayer &d = recs[i];
                if (!steps[i].layer->one_launch(d)) return false;
                d.src = i == 0 ? SMALL_HIP_QM_INPUT : id_of(steps[i].src);
                const int dst = id_of(steps[i].dst);
                d.dst = i + 1 == steps.size() ? SMALL_HIP_QM_OUTPUT : dst;
                d.input_q = steps[i].src->buffer().quant();
                d.output_q = steps[i].dst->buffer().quant();
                d.accum_q = d.output_q;
                if (d.accum_src == Layer<BufferT>::ONE_LAUNCH_ACCUM_ONTO_OUTPUT) d.accum_src = dst;
                for (small_hip_quant const &q : {d.input_q, d.output_q})
                    sig.insert(sig.end(), {q.zero, q.multiplier, (int32_t)q.lshift, (int32_t)q.rshift});
            }
            if (!m_qmodel || sig != m_qsig)
            {
                if (m_qmodel) (void)small_hip_qmodel_destroy(m_qmodel);
                m_qmodel = nullptr;
                m_qsig = sig;
                if (m_qrefused == sig) return false;
                const int rc = small_hip_qmodel_create((int)recs.size(), recs.data(), &m_qmodel, detail::current_stream());
                if (rc == SMALL_HIP_EUNSUPPORTED)
                {
                    m_qrefused = sig;         // does not fit one launch: not an error, and not worth asking again
                    m_refusal = small_hip_last_error();
                    return false;
                }
                detail::hip_check(rc, "small_hip_qmodel_create");     // anything else is a genuine error: raised
            }
            Tensor<BufferT> *out = steps.back().dst;
            if (out->capacity() < steps.back().layer->output_size())
                throw std::invalid_argument("Model::forward_one_launch() ERROR: insufficient output buffer space.");
            detail::hip_check(small_hip_qmodel_forward(m_qmodel, (int)m_input_shape[BATCH], steps.front().src->buffer().device_in(),
                                                       out->buffer().device_out(), detail::current_stream()),
                              "small_hip_qmodel_forward");
            out->set_shape(steps.back().layer->output_shape());
            return true;
        }
        else
        {
            if (!m_one_launch || steps.empty() || m_frefused) return false;
            if (steps.front().src->shape() != m_input_shape)
                throw std::invalid_argument("Model::inference() ERROR: incorrect input buffer shape.");
            if (!m_fmodel)
            {
                std::vector<Tensor<BufferT> const *> ids;
                auto id_of = [&](Tensor<BufferT> const *t) {
                    for (size_t i = 0; i < ids.size(); ++i)
                        if (ids[i] == t) return (int)i;
                    ids.push_back(t);
                    return (int)ids.size() - 1;
                };
                std::vector<small_hip_flayer> recs(steps.size());
                for (size_t i = 0; i < steps.size(); ++i)
                {
                    if (!steps[i].layer->one_launch(recs[i])) { m_frefused = true; return false; }
                    recs[i].src = i == 0 ? SMALL_HIP_QM_INPUT : id_of(steps[i].src);
                    const int dst = id_of(steps[i].dst);
                    recs[i].dst = i + 1 == steps.size() ? SMALL_HIP_QM_OUTPUT : dst;
                }
                const int rc = small_hip_fmodel_create((int)recs.size(), recs.data(), &m_fmodel, detail::current_stream());
                if (rc == SMALL_HIP_EUNSUPPORTED)
                {
                    m_frefused = true;        // does not fit one launch: not an error, and not worth asking again
                    m_refusal = small_hip_last_error();
                    return false;
                }
                detail::hip_check(rc, "small_hip_fmodel_create");     // anything else is a genuine error: raised
            }
            Tensor<BufferT> *out = steps.back().dst;
            if (out->capacity() < steps.back().layer->output_size())
                throw std::invalid_argument("Model::forward_one_launch() ERROR: insufficient output buffer space.");
            detail::hip_check(small_hip_fmodel_forward(m_fmodel, (int)m_input_shape[BATCH], steps.front().src->buffer().device_in(),
                                                       out->buffer().device_out(), detail::current_stream()),
                              "small_hip_fmodel_forward");
            out->set_shape(steps.back().layer->output_shape());
            return true;
        }
    }

    shape_type m_input_shape;
    std::vector<Layer<BufferT> *> m_layers;

private:
    // QUInt8Buffer: on unless SMALL_HIP_TUNE="one_launch=0" (the launch is bit-identical to the layer calls).  FloatBuffer: off
    // unless SMALL_HIP_TUNE="one_launch=1" or set_one_launch(true): its sums run in another order, and callers (the reference's
    // own model tests among them) compare a model's output with the layer functions' bit for bit.
    static bool one_launch_default()
    {
        int const v = small_hip_tune_int("one_launch", -1);
        if (std::is_same<BufferT, QUInt8Buffer>::value) return v != 0;
        return v == 1;
    }
    bool m_one_launch = one_launch_default();
    small_hip_qmodel *m_qmodel = nullptr;
    std::vector<int32_t> m_qsig, m_qrefused;
    small_hip_fmodel *m_fmodel = nullptr;
    bool m_frefused = false;
    std::string m_refusal;
};

} // namespace small
