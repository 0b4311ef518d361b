// Test-only C entry points around the C++ Layer / Model classes of include/small/ so that the
// Python parity tests can drive them with numpy data (built by tests/test_cpp_layers.py with g++,
// linked against libsmall_hip.so).  oracle/ref_shim.cpp exports the same functions (prefix sref_)
// around the reference's own classes; the two are compared through the oracle.
//
// Tensors cross this boundary flat (NCHW / OIHW, unpacked): the shim packs inputs and unpacks
// outputs with pack_buffer / unpack_buffer, as a user of the Layer API would.
// Return value: 0 ok, 1 std::invalid_argument, 2 any other exception; stest_last_error() has the text.
#include <chrono>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include <small.h>
#include <small/AddLayer.hpp>
#include <small/AveragePool2DLayer.hpp>
#include <small/Conv1DLayer.hpp>
#include <small/Conv2DLayer.hpp>
#include <small/DepthwiseConv2DLayer.hpp>
#include <small/DummyLayer.hpp>
#include <small/LeakyReLULayer.hpp>
#include <small/MaxPool2DLayer.hpp>
#include <small/PartialConv2DLayer.hpp>
#include <small/ReLULayer.hpp>
#include <small/RouteLayer.hpp>
#include <small/SoftMaxLayer.hpp>
#include <small/UpSample2DLayer.hpp>
#include <small/models/AutoencoderTiny.hpp>
#include <small/models/AutoencoderTinyDAG.hpp>
#include <small/models/DSCNNSquareTinyDAG.hpp>
#include <small/models/DSCNNTinyDAG.hpp>
#include <small/models/MobileNetTinyDAG.hpp>
#include <small/models/Resnet8TinyDAG.hpp>
#include <small/models/TinyYoloV2DAG.hpp>
#include <small/models/DSCNNSquareTiny.hpp>
#include <small/models/DSCNNTiny.hpp>
#include <small/models/Darknet.hpp>
#include <small/models/MobileNetTiny.hpp>
#include <small/models/Resnet8Tiny.hpp>
#include <small/models/TinyYoloV2.hpp>

namespace
{
thread_local std::string g_err;

template <class Fn>
int guarded(Fn &&fn)
{
    try { fn(); return 0; }
    catch (std::invalid_argument const &e) { g_err = e.what(); return 1; }
    catch (std::exception const &e) { g_err = e.what(); return 2; }
    catch (...) { g_err = "unknown exception"; return 2; }
}

template <class BufferT>
BufferT from_host(typename BufferT::value_type const *p, size_t n)
{
    BufferT b(n);
    if (n) std::memcpy(b.data(), p, n * sizeof(typename BufferT::value_type));
    return b;
}

// flat [batch][C][H][W] -> packed tensor of that shape
template <class BufferT>
small::Tensor<BufferT> packed_tensor(typename BufferT::value_type const *flat, small::shape_type const &shape,
                                     size_t capacity = 0)
{
    const size_t per = shape[1] * shape[2] * shape[3], n = shape[0] * per;
    BufferT f = from_host<BufferT>(flat, n);
    BufferT p(std::max(n, capacity));
    // one call per image keeps this independent of the library's batched pack
    for (size_t i = 0; i < shape[0]; ++i)
    {
        BufferT fi = from_host<BufferT>(flat + i * per, per), pi(per);
        small::pack_buffer(fi, small::INPUT, 1U, (uint32_t)shape[1], (uint32_t)shape[2], (uint32_t)shape[3],
                           BufferT::C_ib, BufferT::C_ob, pi);
        std::memcpy(p.data() + i * per, pi.data(), per * sizeof(typename BufferT::value_type));
    }
    return small::Tensor<BufferT>(shape, std::move(p));
}

template <class BufferT>
void unpack_tensor(small::Tensor<BufferT> const &t, typename BufferT::value_type *flat, int *out_shape)
{
    auto const &s = t.shape();
    for (int i = 0; i < 4; ++i) out_shape[i] = (int)s[i];
    const size_t per = s[1] * s[2] * s[3];
    for (size_t i = 0; i < s[0]; ++i)
    {
        BufferT pi(per), fi(per);
        std::memcpy(pi.data(), t.buffer().data() + i * per, per * sizeof(typename BufferT::value_type));
        small::unpack_buffer(pi, small::OUTPUT, 1U, (uint32_t)s[1], (uint32_t)s[2], (uint32_t)s[3], BufferT::C_ib,
                             BufferT::C_ob, fi);
        std::memcpy(flat + i * per, fi.data(), per * sizeof(typename BufferT::value_type));
    }
}

void set_quant(small::QUInt8Buffer &b, int32_t const *q)
{
    b.m_zero = q[0];
    b.multiplier = q[1];
    b.lshift = q[2];
    b.rshift = q[3];
}

// kind: 0 Conv2DLayer, 1 PartialConv2DLayer, 2 DepthwiseConv2DLayer, 3 Conv1DLayer
template <class BufferT>
std::unique_ptr<small::Layer<BufferT>> make_conv_layer(int kind, small::shape_type const &in_shape, int kh, int kw,
                                                       int stride, int padding, int Co, BufferT const &filt,
                                                       BufferT const &bias, BufferT const *bn, float eps, int act,
                                                       float slope)
{
    const auto pad = padding ? small::PADDING_F : small::PADDING_V;
    const auto a = (small::ActivationType)act;
    small::Layer<BufferT> *l = nullptr;
    if (kind == 3)      // Conv1DLayer (float only): kh is ignored
    {
        if constexpr (std::is_same<BufferT, small::FloatBuffer>::value)
        {
            if (bn) l = new small::Conv1DLayer<BufferT>(in_shape, kw, stride, pad, Co, filt, bn[0], bn[1], bn[2], bn[3], eps, false, a, slope);
            else if (bias.size()) l = new small::Conv1DLayer<BufferT>(in_shape, kw, stride, pad, Co, filt, bias, false, a, slope);
            else l = new small::Conv1DLayer<BufferT>(in_shape, kw, stride, pad, Co, filt, false, a, slope);
        }
    }
    else if (kind == 2)
    {
        if (bn) l = new small::DepthwiseConv2DLayer<BufferT>(in_shape, kh, kw, stride, pad, filt, bias, bn[0], bn[1], bn[2], bn[3], eps, false, a, slope);
        else if (bias.size()) l = new small::DepthwiseConv2DLayer<BufferT>(in_shape, kh, kw, stride, pad, filt, bias, false, a, slope);
        else l = new small::DepthwiseConv2DLayer<BufferT>(in_shape, kh, kw, stride, pad, filt, false, a, slope);
    }
    else if (kind == 1)
    {
        if (bn) l = new small::PartialConv2DLayer<BufferT>(in_shape, kh, kw, stride, pad, Co, filt, bias, bn[0], bn[1], bn[2], bn[3], eps, false, a, slope);
        else if (bias.size()) l = new small::PartialConv2DLayer<BufferT>(in_shape, kh, kw, stride, pad, Co, filt, bias, false, a, slope);
        else l = new small::PartialConv2DLayer<BufferT>(in_shape, kh, kw, stride, pad, Co, filt, false, a, slope);
    }
    else
    {
        if (bn) l = new small::Conv2DLayer<BufferT>(in_shape, kh, kw, stride, pad, Co, filt, bias, bn[0], bn[1], bn[2], bn[3], eps, false, a, slope);
        else if (bias.size()) l = new small::Conv2DLayer<BufferT>(in_shape, kh, kw, stride, pad, Co, filt, bias, false, a, slope);
        else l = new small::Conv2DLayer<BufferT>(in_shape, kh, kw, stride, pad, Co, filt, false, a, slope);
    }
    return std::unique_ptr<small::Layer<BufferT>>(l);
}
} // namespace

using FB = small::FloatBuffer;
using QB = small::QUInt8Buffer;

extern "C"
{

const char *stest_last_error(void) { return g_err.c_str(); }

// Convolution-type layer on flat data.  filters: [Co][Ci][kh][kw] (depthwise: [C][kh][kw]); bias: Co or
// NULL; bn: 4 x Co (gamma, beta, mean, variance) or NULL.  out: in/out, flat [batch][Co_padded][Ho][Wo]
// (read first by the partial layer); out_shape receives the layer's output shape.
int stest_conv_layer_f32(int kind, int batch, int C, int H, int W, int kh, int kw, int stride, int padding, int Co,
                         const float *filters, const float *bias, const float *bn, float eps, int act, float slope,
                         const float *in, float *out, int *out_shape)
{
    return guarded([&] {
        const small::shape_type is{(size_t)batch, (size_t)C, (size_t)H, (size_t)W};
        const size_t nf = (kind == 2 ? (size_t)C : (size_t)Co * C) * kh * kw;
        const size_t nb = kind == 2 ? C : Co;
        FB f = from_host<FB>(filters, nf), b = bias ? from_host<FB>(bias, nb) : FB();
        FB bnb[4];
        if (bn)
            for (int i = 0; i < 4; ++i) bnb[i] = from_host<FB>(bn + i * nb, nb);
        auto layer = make_conv_layer<FB>(kind, is, kh, kw, stride, padding, Co, f, b, bn ? bnb : nullptr, eps, act, slope);
        auto x = packed_tensor<FB>(in, is);
        auto y = packed_tensor<FB>(out, layer->output_shape());
        layer->compute_output({&x}, &y);
        unpack_tensor<FB>(y, out, out_shape);
    });
}

// quantised: q = {zero, multiplier, lshift, rshift} for input, filter, output
int stest_conv_layer_u8(int kind, int batch, int C, int H, int W, int kh, int kw, int stride, int padding, int Co,
                        const uint8_t *filters, int act, const uint8_t *in, const int32_t *in_q,
                        const int32_t *filter_q, const int32_t *out_q, uint8_t *out, int *out_shape)
{
    return guarded([&] {
        const small::shape_type is{(size_t)batch, (size_t)C, (size_t)H, (size_t)W};
        const size_t nf = (kind == 2 ? (size_t)C : (size_t)Co * C) * kh * kw;
        QB f = from_host<QB>(filters, nf);
        set_quant(f, filter_q);
        auto layer = make_conv_layer<QB>(kind, is, kh, kw, stride, padding, Co, f, QB(), nullptr, 0.f, act, 0.f);
        auto x = packed_tensor<QB>(in, is);
        set_quant(x.buffer(), in_q);
        auto y = packed_tensor<QB>(out, layer->output_shape());
        set_quant(y.buffer(), out_q);
        layer->compute_output({&x}, &y);
        unpack_tensor<QB>(y, out, out_shape);
    });
}

// kind: 0 MaxPool2DLayer, 1 AveragePool2DLayer, 2 ReLULayer, 3 LeakyReLULayer(slope), 4 UpSample2DLayer(k = scale),
// 5 AddLayer (out += in), 6 RouteLayer(one input), 7 RouteLayer(in, in2 with C2 channels), 8 SoftMaxLayer
int stest_simple_layer_f32(int kind, int batch, int C, int H, int W, int k, int kw, int stride, int padding,
                           float slope, const float *in, const float *in2, int C2, float *out, int *out_shape)
{
    return guarded([&] {
        const small::shape_type is{(size_t)batch, (size_t)C, (size_t)H, (size_t)W};
        const small::shape_type is2{(size_t)batch, (size_t)C2, (size_t)H, (size_t)W};
        const auto pad = padding ? small::PADDING_F : small::PADDING_V;
        std::unique_ptr<small::Layer<FB>> layer;
        switch (kind)
        {
        case 0: layer.reset(new small::MaxPool2DLayer<FB>(is, k, kw, stride, pad)); break;
        case 1: layer.reset(new small::AveragePool2DLayer<FB>(is, k, kw, stride, pad)); break;
        case 2: layer.reset(new small::ReLULayer<FB>(is)); break;
        case 3: layer.reset(new small::LeakyReLULayer<FB>(is, slope)); break;
        case 4: layer.reset(new small::UpSample2DLayer<FB>(is, k)); break;
        case 5: layer.reset(new small::AddLayer<FB>(is, is)); break;
        case 6: layer.reset(new small::RouteLayer<FB>(is)); break;
        case 7: layer.reset(new small::RouteLayer<FB>(is, is2)); break;
        case 8: layer.reset(new small::SoftMaxLayer<FB>(is)); break;
        default: throw std::invalid_argument("stest_simple_layer_f32: unknown kind");
        }
        auto x = packed_tensor<FB>(in, is);
        auto y = packed_tensor<FB>(out, layer->output_shape());
        if (kind == 7)
        {
            auto x2 = packed_tensor<FB>(in2, is2);
            layer->compute_output({&x, &x2}, &y);
        }
        else
            layer->compute_output({&x}, &y);
        unpack_tensor<FB>(y, out, out_shape);
    });
}

// which: 0 MobileNetTiny, 1 Resnet8Tiny, 2 DSCNNTiny, 3 TinyYoloV2, built with the reference's defaults
// (variant 0) or as the benchmark topology (variant 1: MobileNet 1000 classes + average pooling; ResNet-8
// 10 classes; DS-CNN 10x4 stem, 12 classes, average pooling; Tiny-YOLOv2 LeakyReLU 0.1 with 125 linear outputs).
// filters: unpacked, in the model's filter order; sizes[i] elements each.
int stest_model_f32(int which, int variant, int batch, int C, int H, int W, const float *const *filters,
                    const size_t *sizes, int nfilters, const float *in, float *out, int *out_shape)
{
    return guarded([&] {
        const small::shape_type is{(size_t)batch, (size_t)C, (size_t)H, (size_t)W};
        std::vector<std::unique_ptr<FB>> own;
        std::vector<FB *> fl;
        for (int i = 0; i < nfilters; ++i)
        {
            own.emplace_back(new FB(from_host<FB>(filters[i], sizes[i])));
            fl.push_back(own.back().get());
        }
        std::unique_ptr<small::Model<FB>> m;
        switch (which)
        {
        case 0: m.reset(variant ? new small::MobileNetTiny<FB>(is, fl, false, 32, 1000, true)
                                : new small::MobileNetTiny<FB>(is, fl, false)); break;
        case 1: m.reset(variant ? new small::Resnet8Tiny<FB>(is, fl, false, 10) : new small::Resnet8Tiny<FB>(is, fl, false)); break;
        case 2: m.reset(variant ? new small::DSCNNTiny<FB>(is, fl, false, 10, 4, 12, true)
                                : new small::DSCNNTiny<FB>(is, fl, false)); break;
        case 3: m.reset(variant ? new small::TinyYoloV2<FB>(is, fl, false, small::LEAKY, 0.1f, 125, false)
                                : new small::TinyYoloV2<FB>(is, fl, false)); break;
        case 4: m.reset(new small::AutoencoderTiny<FB>(is, 16, fl, false)); break;
        case 5: m.reset(new small::DSCNNSquareTiny<FB>(is, fl, false)); break;
        // 10 + which: the same model on the DAG executor
        case 10: m.reset(new small::MobileNetTinyDAG<FB>(is, fl, false)); break;
        case 11: m.reset(new small::Resnet8TinyDAG<FB>(is, fl, false)); break;
        case 12: m.reset(new small::DSCNNTinyDAG<FB>(is, fl, false)); break;
        case 13: m.reset(new small::TinyYoloV2DAG<FB>(is, fl, false)); break;
        case 14: m.reset(new small::AutoencoderTinyDAG<FB>(is, 16, fl, false)); break;
        case 15: m.reset(new small::DSCNNSquareTinyDAG<FB>(is, fl, false)); break;
        default: throw std::invalid_argument("stest_model_f32: unknown model");
        }
        auto x = packed_tensor<FB>(in, is);
        if (which >= 10) m->inference(&x);       // the second pass of a DAG model runs on recycled pool tensors
        auto outs = m->inference(&x);
        unpack_tensor<FB>(*outs[0], out, out_shape);
    });
}

// Milliseconds per inference() call of a model class on a resident input (synthetic filters and input made
// here; `steps` timed calls after `warmup`, bracketed by stream synchronisation).  Same which / variant as above.
int stest_model_time_f32(int which, int variant, int batch, int C, int H, int W, const size_t *sizes, int nfilters,
                         int steps, int warmup, double *ms_per_call)
{
    return guarded([&] {
        const small::shape_type is{(size_t)batch, (size_t)C, (size_t)H, (size_t)W};
        std::vector<std::unique_ptr<FB>> own;
        std::vector<FB *> fl;
        for (int i = 0; i < nfilters; ++i)
        {
            own.emplace_back(new FB(sizes[i]));
            float *p = own.back()->data();
            for (size_t k = 0; k < sizes[i]; ++k) p[k] = 0.01f * float((int)((k * 2654435761u) >> 24) - 128) / 128.f;
            fl.push_back(own.back().get());
        }
        std::unique_ptr<small::Model<FB>> m;
        switch (which)
        {
        case 0: m.reset(variant ? new small::MobileNetTiny<FB>(is, fl, false, 32, 1000, true)
                                : new small::MobileNetTiny<FB>(is, fl, false)); break;
        case 1: m.reset(variant ? new small::Resnet8Tiny<FB>(is, fl, false, 10) : new small::Resnet8Tiny<FB>(is, fl, false)); break;
        case 2: m.reset(variant ? new small::DSCNNTiny<FB>(is, fl, false, 10, 4, 12, true)
                                : new small::DSCNNTiny<FB>(is, fl, false)); break;
        case 3: m.reset(variant ? new small::TinyYoloV2<FB>(is, fl, false, small::LEAKY, 0.1f, 125, false)
                                : new small::TinyYoloV2<FB>(is, fl, false)); break;
        default: throw std::invalid_argument("stest_model_time_f32: unknown model");
        }
        small::Tensor<FB> x(is);
        float *px = x.buffer().data();
        for (size_t k = 0; k < x.size(); ++k) px[k] = float((int)((k * 40503u) & 255) - 128) / 128.f;
        for (int i = 0; i < warmup; ++i) m->inference(&x);
        small::synchronize();
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < steps; ++i) m->inference(&x);
        small::synchronize();
        const auto t1 = std::chrono::steady_clock::now();
        *ms_per_call = std::chrono::duration<double, std::milli>(t1 - t0).count() / steps;
    });
}

// A caller that holds HOST buffers: every step a new batch sits in host memory, is uploaded, run, and the logits are read
// back on the host.  serial: one input tensor, upload -> inference -> read.  overlapped: two input tensors in turn,
// Tensor::prefetch() of batch i + 1 before inference() of batch i is issued, so the upload rides under the layers.
// Milliseconds per step of both forms; *mismatches counts overlapped steps whose logits differ from the serial run's
// logits for the same batch (two distinct batches alternate).
int stest_model_host_feed_f32(int batch, const size_t *sizes, int nfilters, int steps, int warmup, double *ms_serial,
                              double *ms_overlapped, int *mismatches)
{
    return guarded([&] {
        const small::shape_type is{(size_t)batch, 3, 224, 224};
        std::vector<std::unique_ptr<FB>> own;
        std::vector<FB *> fl;
        for (int i = 0; i < nfilters; ++i)
        {
            own.emplace_back(new FB(sizes[i]));
            float *p = own.back()->data();
            for (size_t k = 0; k < sizes[i]; ++k) p[k] = 0.05f * float((int)((k * 2654435761u) >> 24) - 128) / 128.f;
            fl.push_back(own.back().get());
        }
        small::MobileNetTiny<FB> m(is, fl, false, 32, 1000, true);
        small::Tensor<FB> x[2] = {small::Tensor<FB>(is), small::Tensor<FB>(is)};
        for (int b = 0; b < 2; ++b)
        {
            float *px = x[b].buffer().data();
            for (size_t k = 0; k < x[b].size(); ++k) px[k] = float((int)(((k + 977u * b) * 40503u) & 255) - 128) / 128.f;
        }
        // a new batch "arrives": the host block is written (one element is enough to make the whole tensor stale on the device)
        auto arrive = [&](int b, int step) { x[b].buffer().data()[0] = float((step & 1) ? 0.25f : -0.25f) + float(b); };
        std::vector<float> want[2];
        double total = 0.0;
        auto read = [&](small::Tensor<FB> const *t, std::vector<float> &dst) {
            float const *p = t->buffer().data();                // waits for the pass and downloads
            dst.assign(p, p + t->size());
        };
        // serial
        for (int i = 0; i < warmup + steps; ++i)
        {
            if (i == warmup) { small::synchronize(); total = 0.0; }
            const auto t0 = std::chrono::steady_clock::now();
            const int b = i & 1;
            arrive(b, b);
            auto outs = m.inference(&x[b]);
            read(outs[0], want[b]);
            total += std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
        }
        *ms_serial = total / steps;
        // overlapped
        *mismatches = 0;
        std::vector<float> got;
        arrive(0, 0);
        x[0].prefetch();
        for (int i = 0; i < warmup + steps; ++i)
        {
            if (i == warmup) total = 0.0;
            const auto t0 = std::chrono::steady_clock::now();
            const int b = i & 1, nb = b ^ 1;
            arrive(nb, nb);
            x[nb].prefetch();                                    // batch i + 1 goes up while batch i runs
            auto outs = m.inference(&x[b]);
            read(outs[0], got);
            total += std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
            if (got.size() != want[b].size() || std::memcmp(got.data(), want[b].data(), got.size() * sizeof(float)) != 0) ++*mismatches;
        }
        *ms_overlapped = total / steps;
    });
}

// Resnet8Tiny<QUInt8Buffer>: every tensor of the model shares one set of quantisation fields per role
// (input, filters, activations), enough to exercise the quantised layer classes end to end.
int stest_resnet8_u8(int batch, const uint8_t *const *filters, const size_t *sizes, int nfilters, const uint8_t *in,
                     const int32_t *in_q, const int32_t *filter_q, int one_launch, uint8_t *out, int *out_shape)
{
    return guarded([&] {
        const small::shape_type is{(size_t)batch, 3, 32, 32};
        std::vector<std::unique_ptr<QB>> own;
        std::vector<QB *> fl;
        for (int i = 0; i < nfilters; ++i)
        {
            own.emplace_back(new QB(from_host<QB>(filters[i], sizes[i])));
            set_quant(*own.back(), filter_q);
            fl.push_back(own.back().get());
        }
        small::Resnet8Tiny<QB> m(is, fl, false, 10);
        m.set_one_launch(one_launch != 0);
        auto x = packed_tensor<QB>(in, is);
        set_quant(x.buffer(), in_q);
        auto outs = m.inference(&x);
        outs = m.inference(&x);          // a second pass re-uses the planned launch
        if (m.one_launch_planned() != (one_launch != 0))
            throw std::runtime_error("Resnet8Tiny<QUInt8Buffer>: one-launch form requested and not used (or the reverse)");
        unpack_tensor<QB>(*outs[0], out, out_shape);
    });
}

// The reference-named two-layer functions of small/interface.hpp on PACKED batch-1 arrays.
// second 0: Conv2D_*_Maxpool2D, 1: Conv2D_*_DepthwiseConv2D_*; variant 0 plain, 1 ReLU, 2 bias + ReLU.
// inter / out: packed first-layer and second-layer outputs (inter is only defined where the library says so).
int stest_fused_two_layers_f32(int second, int variant, int ck, int cs, int ct, int cb, int cl, int cr, int k2, int s2,
                               int t2, int b2, int l2, int r2, int Co, int Ci, int H, int W, const float *in,
                               size_t n_in, const float *filt, size_t n_filt, const float *bias, const float *dwfilt,
                               size_t n_dwfilt, const float *dwbias, float *out, size_t n_out, size_t n_inter)
{
    using FB = small::FloatBuffer;
    return guarded([&] {
        FB x = from_host<FB>(in, n_in), f = from_host<FB>(filt, n_filt), b = from_host<FB>(bias, Co);
        FB df = from_host<FB>(dwfilt, n_dwfilt), db = from_host<FB>(dwbias, Co), inter(n_inter), o(n_out);
        if (second == 0 && variant == 0)
            small::Conv2D_Maxpool2D(ck, ck, cs, ct, cb, cl, cr, k2, k2, s2, t2, b2, l2, r2, Co, Ci, H, W, x, f, inter, o);
        else if (second == 0 && variant == 1)
            small::Conv2D_ReLU_Maxpool2D(ck, ck, cs, ct, cb, cl, cr, k2, k2, s2, t2, b2, l2, r2, Co, Ci, H, W, x, f,
                                         inter, o);
        else if (second == 0)
            small::Conv2D_Bias_ReLU_Maxpool2D(ck, ck, cs, ct, cb, cl, cr, k2, k2, s2, t2, b2, l2, r2, Co, Ci, H, W, x, f,
                                              b, inter, o);
        else if (variant == 0)
            small::Conv2D_DepthwiseConv2D(ck, ck, cs, ct, cb, cl, cr, k2, k2, s2, t2, b2, l2, r2, Co, Ci, H, W, x, f,
                                          inter, df, o);
        else if (variant == 1)
            small::Conv2D_ReLU_DepthwiseConv2D_ReLU(ck, ck, cs, ct, cb, cl, cr, k2, k2, s2, t2, b2, l2, r2, Co, Ci, H, W,
                                                    x, f, inter, df, o);
        else
            small::Conv2D_Bias_ReLU_DepthwiseConv2D_Bias_ReLU(ck, ck, cs, ct, cb, cl, cr, k2, k2, s2, t2, b2, l2, r2, Co,
                                                              Ci, H, W, x, f, b, inter, df, db, o);
        std::memcpy(out, o.data(), n_out * sizeof(float));
    });
}

// The 1-D functions of small/interface_1D.hpp on PACKED arrays (batch-1 signatures of the reference; rows = its
// batch_size).  kind 0 Conv1D, 1 PartialConv1D (out is in/out), 2 MaxPool1D, 3 AveragePool1D, 4 ReLUActivation1D,
// 5 UpSample1D (k = scale), 6 Conv1D_ReLU, 7 Conv1D_Bias_ReLU (bias = 4th array), 8 GroupConv1D, 9 PartialGroupConv1D
// (Co = groups, Ci = channels per group)
int stest_1d_f32(int kind, int k, int s, int l, int r, int Co, int Ci, int rows, int W, const float *in, size_t n_in,
                 const float *filt, size_t n_filt, const float *bias, float *out, size_t n_out)
{
    using FB = small::FloatBuffer;
    return guarded([&] {
        FB x = from_host<FB>(in, n_in), f = from_host<FB>(filt, n_filt), b = from_host<FB>(bias, bias && kind == 7 ? Co : 0);
        FB o = from_host<FB>(out, n_out);
        switch (kind)
        {
        case 0: small::Conv1D(k, s, l, r, Co, Ci, rows, W, x, f, o); break;
        case 1: small::PartialConv1D(k, s, l, r, Co, Ci, rows, W, x, f, o); break;
        case 2: small::MaxPool1D(k, s, l, r, Ci, rows, W, x, o); break;
        case 3: small::AveragePool1D(k, s, l, r, Ci, rows, W, x, o); break;
        case 4: small::ReLUActivation1D(Ci, rows, W, x, o); break;
        case 5: small::UpSample1D(k, Ci, rows, W, x, o); break;
        case 6: small::Conv1D_ReLU(k, s, l, r, Co, Ci, rows, W, x, f, o); break;
        case 8: small::GroupConv1D(k, s, Co, l, r, Ci, rows, W, x, f, o); break;          // Co = groups
        case 9: small::PartialGroupConv1D(k, s, Co, l, r, Ci, rows, W, x, f, o); break;
        default: small::Conv1D_Bias_ReLU(k, s, l, r, Co, Ci, rows, W, x, f, b, o); break;
        }
        std::memcpy(out, o.data(), n_out * sizeof(float));
    });
}

// variant 0: DepthwiseConv2D_ReLU, 1: DepthwiseConv2D_Bias_ReLU, 2: Conv2D_ReLU, 3: Conv2D_Bias_ReLU (packed arrays)
int stest_fused_single_f32(int variant, int k, int s, int t, int b, int l, int r, int Co, int Ci, int H, int W,
                           const float *in, size_t n_in, const float *filt, size_t n_filt, const float *bias,
                           float *out, size_t n_out)
{
    using FB = small::FloatBuffer;
    return guarded([&] {
        FB x = from_host<FB>(in, n_in), f = from_host<FB>(filt, n_filt), bb = from_host<FB>(bias, variant < 2 ? Ci : Co);
        FB o(n_out);
        if (variant == 0) small::DepthwiseConv2D_ReLU(k, k, s, t, b, l, r, Ci, H, W, x, f, o);
        else if (variant == 1) small::DepthwiseConv2D_Bias_ReLU(k, k, s, t, b, l, r, Ci, H, W, x, f, bb, o);
        else if (variant == 2) small::Conv2D_ReLU(k, k, s, t, b, l, r, Co, Ci, H, W, x, f, o);
        else small::Conv2D_Bias_ReLU(k, k, s, t, b, l, r, Co, Ci, H, W, x, f, bb, o);
        std::memcpy(out, o.data(), n_out * sizeof(float));
    });
}

// ---- Darknet cfg / weights model, YOLO decode, non-maximum suppression -------------------------------------------
// Runs the model the two files describe on one flat [C][H][W] image.  out receives the YOLO heads' records one
// after the other (each head is [predictions][5 + classes]); out_preds[i] = predictions of head i.
// det (may be NULL): detections after process_outputs(conf, iou), 7 floats each {x, y, w, h, objectness, class
// score, class id}; *n_det in: capacity, out: count.
int stest_darknet_f32(const char *cfg, const char *weights, const float *in, size_t n_in, float *out, size_t out_cap,
                       int *out_preds, int *n_heads, int *record_len, float conf, float iou, float *det, int *n_det)
{
    return guarded([&] {
        small::Darknet<FB> model(cfg, weights);
        auto const &is = model.get_input_shape();
        if (small::compute_size(is) != n_in) throw std::invalid_argument("darknet shim: input size mismatch");
        auto x = packed_tensor<FB>(in, is);
        model.inference(&x);                     // the second pass runs on recycled pool tensors
        auto outs = model.inference(&x);
        size_t at = 0;
        *n_heads = (int)outs.size();
        for (size_t i = 0; i < outs.size(); ++i)
        {
            auto const &s = outs[i]->shape();
            out_preds[i] = (int)s[2];
            *record_len = (int)s[3];
            const size_t n = s[2] * s[3];
            if (at + n > out_cap) throw std::invalid_argument("darknet shim: output capacity");
            for (size_t k = 0; k < n; ++k) out[at + k] = outs[i]->buffer()[k];
            at += n;
        }
        if (det)
        {
            auto d = model.process_outputs(outs, conf, iou);
            const int cap = *n_det;
            *n_det = (int)d.size();
            for (int i = 0; i < (int)d.size() && i < cap; ++i)
            {
                float *r = det + 7 * i;
                r[0] = d[i].bbox.x; r[1] = d[i].bbox.y; r[2] = d[i].bbox.w; r[3] = d[i].bbox.h;
                r[4] = d[i].objectness; r[5] = d[i].class_score; r[6] = (float)d[i].class_id;
            }
        }
    });
}

// basic_nms on n records of 7 floats (layout as above); kept records are written to out, their count returned in *n_out
int stest_nms(const float *pred, int n, float iou, float *out, int *n_out)
{
    return guarded([&] {
        std::vector<small::Detection> p;
        for (int i = 0; i < n; ++i)
        {
            const float *r = pred + 7 * i;
            p.push_back(small::Detection{{r[0], r[1], r[2], r[3]}, r[4], r[5], (size_t)r[6]});
        }
        auto k = small::basic_nms(p, iou);
        *n_out = (int)k.size();
        for (size_t i = 0; i < k.size(); ++i)
        {
            float *r = out + 7 * i;
            r[0] = k[i].bbox.x; r[1] = k[i].bbox.y; r[2] = k[i].bbox.w; r[3] = k[i].bbox.h;
            r[4] = k[i].objectness; r[5] = k[i].class_score; r[6] = (float)k[i].class_id;
        }
    });
}

// YOLOLayer on a flat [C][H][W] input (C is padded to the channel block with zeros by the caller)
int stest_yolo_layer_f32(int C, int H, int W, const uint32_t *anchors_wh, int num_anchors, int classes, int image_size,
                          const float *in, float *out)
{
    return guarded([&] {
        const small::shape_type is{1UL, (size_t)C, (size_t)H, (size_t)W};
        std::vector<std::pair<uint32_t, uint32_t>> an;
        for (int a = 0; a < num_anchors; ++a) an.emplace_back(anchors_wh[2 * a], anchors_wh[2 * a + 1]);
        small::YOLOLayer<FB> layer(is, an, classes, image_size);
        auto x = packed_tensor<FB>(in, is);
        small::Tensor<FB> y(layer.output_shape());
        layer.compute_output({&x}, &y);
        for (size_t k = 0; k < layer.output_size(); ++k) out[k] = y.buffer()[k];
    });
}

// Milliseconds per Darknet::inference() call at `batch` images (input left as allocated; resident on the device).
int stest_darknet_time(const char *cfg, const char *weights, int batch, int steps, int warmup, double *ms_per_call)
{
    return guarded([&] {
        small::Darknet<FB> model(cfg, weights, false, (uint32_t)batch);
        small::Tensor<FB> x(model.get_input_shape());
        for (int i = 0; i < warmup; ++i) model.inference(&x);
        small::synchronize();
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < steps; ++i) model.inference(&x);
        small::synchronize();
        *ms_per_call = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / steps;
    });
}

} // extern "C"
