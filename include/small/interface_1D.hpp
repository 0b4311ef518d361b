// The 1-D layer functions of the reference (include/small/interface_abstract_1D.hpp:47-1700 and the single-launch
// members of fused_interface_abstract_1D.hpp), same names and argument order.
//
// A 1-D tensor is the packed 2-D tensor [C/16][rows][W][16] whose rows are independent signals: the
// reference's `batch_size` argument is that row count (its Conv1DLayer passes shape[HEIGHT],
// Conv1DLayer.hpp:671-690).  Every function here is therefore the 2-D kernel with a 1 x kernel_width window
// and no vertical padding.  The 2-D entry points stride both axes alike; several rows together with a stride other
// than 1 go through the 1-D entry points (small_hip_conv1d_* / small_hip_pool1d_*), which stride along the width only.
// small::batched::<Fn>(batch, ...) takes `batch` such tensors back to back.
// The QUInt8Buffer forms (Conv1D, MaxPool1D, ReLUActivation1D) are the quantised 2-D functions on the same
// 1 x kernel_width window; the reference's own quantised 1-D functions write unrelated bytes on its scalar build
// (its only quantised platform), so there is nothing to compare them with.
#pragma once

#include "interface.hpp"

namespace small
{
namespace detail
{
// several rows AND a stride other than 1: the case the 1-D entry points exist for
inline bool rows_need_1d(int stride, int rows) { return rows > 1 && stride != 1; }

template <class BufferT>
inline void conv1d_rows(const char *op, int batch, int k, int stride, uint8_t l_pad, uint8_t r_pad, int groups, int Co,
                        int Ci, int rows, int width, BufferT const &in, BufferT const &filt, BufferT const &bias,
                        ActivationType act, float slope, bool accumulate, BufferT &out)
{
    int rc;
    if constexpr (std::is_same<BufferT, FloatBuffer>::value)
        rc = small_hip_conv1d_f32(batch, k, stride, l_pad, r_pad, groups, Co, Ci, rows, width, in.device_in(), filt.device_in(),
                                  bias.size() > 0 ? bias.device_in() : nullptr, (int)act, slope, accumulate ? 1 : 0,
                                  out.device_out(), st());
    else
    {
        const small_hip_quant iq = in.quant(), fq = filt.quant(), oq = out.quant();
        rc = small_hip_conv1d_u8(batch, k, stride, l_pad, r_pad, groups, Co, Ci, rows, width, in.device_in(), &iq,
                                 filt.device_in(), &fq, out.device_out(), &oq, st());
    }
    raise<BufferT>(rc, op);
}

template <class BufferT>
inline void pool1d_rows(const char *op, bool is_max, int batch, int k, int stride, uint8_t l_pad, uint8_t r_pad, int C,
                        int rows, int width, BufferT const &in, BufferT &out)
{
    int rc;
    if constexpr (std::is_same<BufferT, FloatBuffer>::value)
        rc = small_hip_pool1d_f32(is_max ? 1 : 0, batch, k, stride, l_pad, r_pad, C, rows, width, in.device_in(),
                                  out.device_out(), st());
    else
    {
        const small_hip_quant iq = in.quant(), oq = out.quant();
        rc = small_hip_pool1d_u8(is_max ? 1 : 0, batch, k, stride, l_pad, r_pad, C, rows, width, in.device_in(), &iq,
                                 out.device_out(), &oq, st());
    }
    raise<BufferT>(rc, op);
}
} // namespace detail

namespace batched
{
// interface_abstract_1D.hpp:47 (float), :229 (quint8)
template <class BufferT>
void Conv1D(int batch, int kernel_width, int stride, uint8_t l_pad, uint8_t r_pad, int output_channels,
            int input_channels, int batch_size, int input_width, BufferT const &input_buf, BufferT const &filter_buf,
            BufferT &output_buf)
{
    if (detail::rows_need_1d(stride, batch_size))
        return detail::conv1d_rows("Conv1D", batch, kernel_width, stride, l_pad, r_pad, 0, output_channels, input_channels,
                                   batch_size, input_width, input_buf, filter_buf, BufferT(), NONE, 0.f, false, output_buf);
    try
    {
        Conv2D(batch, 1, kernel_width, stride, 0, 0, l_pad, r_pad, output_channels, input_channels, batch_size,
               input_width, input_buf, filter_buf, output_buf);
    }
    catch (std::invalid_argument const &e) { throw std::invalid_argument(detail::rename_op(e.what(), "Conv2D", "Conv1D")); }
}

// interface_abstract_1D.hpp:415
template <class BufferT, detail::if_float<BufferT> = true>
void PartialConv1D(int batch, int kernel_width, int stride, uint8_t l_pad, uint8_t r_pad, int output_channels,
                   int input_channels, int batch_size, int input_width, BufferT const &input_buf,
                   BufferT const &filter_buf, BufferT &output_buf)
{
    if (detail::rows_need_1d(stride, batch_size))
        return detail::conv1d_rows("PartialConv1D", batch, kernel_width, stride, l_pad, r_pad, 0, output_channels,
                                   input_channels, batch_size, input_width, input_buf, filter_buf, BufferT(), NONE, 0.f, true,
                                   output_buf);
    try
    {
        PartialConv2D(batch, 1, kernel_width, stride, 0, 0, l_pad, r_pad, output_channels, input_channels, batch_size,
                      input_width, input_buf, filter_buf, output_buf);
    }
    catch (std::invalid_argument const &e)
    {
        throw std::invalid_argument(detail::rename_op(e.what(), "PartialConv2D", "PartialConv1D"));
    }
}

// interface_abstract_1D.hpp:1255 (float), :1320 (quint8): output_groups convolutions of input_channels -> input_channels,
// one per slab of input_channels channels
template <class BufferT>
void GroupConv1D(int batch, int kernel_width, int stride, int output_groups, uint8_t l_pad, uint8_t r_pad,
                 int input_channels, int batch_size, int input_width, BufferT const &input_buf,
                 BufferT const &filter_buf, BufferT &output_buf)
{
    if (detail::rows_need_1d(stride, batch_size))
        return detail::conv1d_rows("GroupConv1D", batch, kernel_width, stride, l_pad, r_pad, output_groups, input_channels,
                                   input_channels, batch_size, input_width, input_buf, filter_buf, BufferT(), NONE, 0.f, false,
                                   output_buf);
    try
    {
        GroupConv2D(batch, 1, kernel_width, stride, output_groups, 0, 0, l_pad, r_pad, input_channels, batch_size,
                    input_width, input_buf, filter_buf, output_buf);
    }
    catch (std::invalid_argument const &e) { throw std::invalid_argument(detail::rename_op(e.what(), "GroupConv2D", "GroupConv1D")); }
}

// interface_abstract_1D.hpp:1388
template <class BufferT, detail::if_float<BufferT> = true>
void PartialGroupConv1D(int batch, int kernel_width, int stride, int output_groups, uint8_t l_pad, uint8_t r_pad,
                        int input_channels, int batch_size, int input_width, BufferT const &input_buf,
                        BufferT const &filter_buf, BufferT &output_buf)
{
    if (detail::rows_need_1d(stride, batch_size))
        return detail::conv1d_rows("PartialGroupConv1D", batch, kernel_width, stride, l_pad, r_pad, output_groups,
                                   input_channels, input_channels, batch_size, input_width, input_buf, filter_buf, BufferT(),
                                   NONE, 0.f, true, output_buf);
    try
    {
        PartialGroupConv2D(batch, 1, kernel_width, stride, output_groups, 0, 0, l_pad, r_pad, input_channels,
                           batch_size, input_width, input_buf, filter_buf, output_buf);
    }
    catch (std::invalid_argument const &e)
    {
        throw std::invalid_argument(detail::rename_op(e.what(), "PartialGroupConv2D", "PartialGroupConv1D"));
    }
}

// bias + convolution + activation in one launch (Conv1D_ReLU / Conv1D_Bias_ReLU, fused_interface_abstract_1D.hpp:55, 216,
// and what Conv1DLayer::compute_output issues as three calls); bias_buf may be empty
template <class BufferT, detail::if_float<BufferT> = true>
void Conv1D_Bias_Act(int batch, int kernel_width, int stride, uint8_t l_pad, uint8_t r_pad, int output_channels,
                     int input_channels, int batch_size, int input_width, BufferT const &input_buf,
                     BufferT const &filter_buf, BufferT const &bias_buf, ActivationType act, float negative_slope,
                     BufferT &output_buf)
{
    if (detail::rows_need_1d(stride, batch_size))
        return detail::conv1d_rows("Conv1D", batch, kernel_width, stride, l_pad, r_pad, 0, output_channels, input_channels,
                                   batch_size, input_width, input_buf, filter_buf, bias_buf, act,
                                   negative_slope, false, output_buf);
    Conv2D_Bias_Act(batch, 1, kernel_width, stride, 0, 0, l_pad, r_pad, output_channels, input_channels, batch_size,
                    input_width, input_buf, filter_buf, bias_buf, act, negative_slope, output_buf);
}

// interface_abstract_1D.hpp:776 (float), :840 (quint8)
template <class BufferT>
void MaxPool1D(int batch, int kernel_width, int stride, uint8_t l_pad, uint8_t r_pad, int input_channels,
               int batch_size, int input_width, BufferT const &input_buf, BufferT &output_buf)
{
    if (detail::rows_need_1d(stride, batch_size))
        return detail::pool1d_rows("MaxPool1D", true, batch, kernel_width, stride, l_pad, r_pad, input_channels, batch_size,
                                   input_width, input_buf, output_buf);
    try
    {
        MaxPool2D(batch, 1, kernel_width, stride, 0, 0, l_pad, r_pad, input_channels, batch_size, input_width,
                  input_buf, output_buf);
    }
    catch (std::invalid_argument const &e) { throw std::invalid_argument(detail::rename_op(e.what(), "MaxPool2D", "MaxPool1D")); }
}

// interface_abstract_1D.hpp:906
template <class BufferT, detail::if_float<BufferT> = true>
void AveragePool1D(int batch, int kernel_width, int stride, uint8_t l_pad, uint8_t r_pad, int input_channels,
                   int batch_size, int input_width, BufferT const &input_buf, BufferT &output_buf)
{
    if (detail::rows_need_1d(stride, batch_size))
        return detail::pool1d_rows("AveragePool1D", false, batch, kernel_width, stride, l_pad, r_pad, input_channels, batch_size,
                                   input_width, input_buf, output_buf);
    try
    {
        AveragePool2D(batch, 1, kernel_width, stride, 0, 0, l_pad, r_pad, input_channels, batch_size, input_width,
                      input_buf, output_buf);
    }
    catch (std::invalid_argument const &e)
    {
        throw std::invalid_argument(detail::rename_op(e.what(), "AveragePool2D", "AveragePool1D"));
    }
}

// interface_abstract_1D.hpp:1526 (float), :1562 (quint8)
template <class BufferT>
void ReLUActivation1D(int batch, int input_channels, int batch_size, int input_width, BufferT const &input_buf,
                      BufferT &output_buf)
{
    ReLUActivation(batch, input_channels, batch_size, input_width, input_buf, output_buf);
}

// interface_abstract_1D.hpp:1614: nearest neighbour along the width
template <class BufferT, detail::if_float<BufferT> = true>
void UpSample1D(int batch, int scale_factor, int input_channels, int batch_size, int input_width,
                BufferT const &input_buf, BufferT &output_buf)
{
    detail::raise<BufferT>(small_hip_upsample1d_f32(batch, scale_factor, input_channels, batch_size, input_width,
                                                    input_buf.device_in(), output_buf.device_out(), detail::st()),
                           "Upsample");
}
} // namespace batched

// ---- the reference's signatures ---------------------------------------------------------------------------------
template <class BufferT>
void Conv1D(int kernel_width, int stride, uint8_t l_pad, uint8_t r_pad, int output_channels, int input_channels,
            int batch_size, int input_width, BufferT const &input_buf, BufferT const &filter_buf, BufferT &output_buf)
{
    batched::Conv1D(1, kernel_width, stride, l_pad, r_pad, output_channels, input_channels, batch_size, input_width,
                    input_buf, filter_buf, output_buf);
}

template <class BufferT>
void PartialConv1D(int kernel_width, int stride, uint8_t l_pad, uint8_t r_pad, int output_channels,
                   int input_channels, int batch_size, int input_width, BufferT const &input_buf,
                   BufferT const &filter_buf, BufferT &output_buf)
{
    batched::PartialConv1D(1, kernel_width, stride, l_pad, r_pad, output_channels, input_channels, batch_size,
                           input_width, input_buf, filter_buf, output_buf);
}

template <class BufferT>
void GroupConv1D(int kernel_width, int stride, int output_groups, uint8_t l_pad, uint8_t r_pad, int input_channels,
                 int batch_size, int input_width, BufferT const &input_buf, BufferT const &filter_buf,
                 BufferT &output_buf)
{
    batched::GroupConv1D(1, kernel_width, stride, output_groups, l_pad, r_pad, input_channels, batch_size,
                         input_width, input_buf, filter_buf, output_buf);
}

template <class BufferT>
void PartialGroupConv1D(int kernel_width, int stride, int output_groups, uint8_t l_pad, uint8_t r_pad,
                        int input_channels, int batch_size, int input_width, BufferT const &input_buf,
                        BufferT const &filter_buf, BufferT &output_buf)
{
    batched::PartialGroupConv1D(1, kernel_width, stride, output_groups, l_pad, r_pad, input_channels, batch_size,
                                input_width, input_buf, filter_buf, output_buf);
}

template <class BufferT>
void MaxPool1D(int kernel_width, int stride, uint8_t l_pad, uint8_t r_pad, int input_channels, int batch_size,
               int input_width, BufferT const &input_buf, BufferT &output_buf)
{
    batched::MaxPool1D(1, kernel_width, stride, l_pad, r_pad, input_channels, batch_size, input_width, input_buf,
                       output_buf);
}

template <class BufferT>
void AveragePool1D(int kernel_width, int stride, uint8_t l_pad, uint8_t r_pad, int input_channels, int batch_size,
                   int input_width, BufferT const &input_buf, BufferT &output_buf)
{
    batched::AveragePool1D(1, kernel_width, stride, l_pad, r_pad, input_channels, batch_size, input_width, input_buf,
                           output_buf);
}

template <class BufferT>
void ReLUActivation1D(int input_channels, int batch_size, int input_width, BufferT const &input_buf,
                      BufferT &output_buf)
{
    batched::ReLUActivation1D(1, input_channels, batch_size, input_width, input_buf, output_buf);
}

template <class BufferT>
void UpSample1D(int scale_factor, int input_channels, int batch_size, int input_width, BufferT const &input_buf,
                BufferT &output_buf)
{
    batched::UpSample1D(1, scale_factor, input_channels, batch_size, input_width, input_buf, output_buf);
}

// fused_interface_abstract_1D.hpp:55, 216: one launch
template <class BufferT>
void Conv1D_ReLU(int kernel_width, int stride, uint8_t l_pad, uint8_t r_pad, int output_channels, int input_channels,
                 int batch_size, int input_width, BufferT const &input_buf, BufferT const &filter_buf,
                 BufferT &output_buf)
{
    batched::Conv1D_Bias_Act(1, kernel_width, stride, l_pad, r_pad, output_channels, input_channels, batch_size,
                             input_width, input_buf, filter_buf, BufferT(), RELU, 0.f, output_buf);
}

template <class BufferT>
void Conv1D_Bias_ReLU(int kernel_width, int stride, uint8_t l_pad, uint8_t r_pad, int output_channels,
                      int input_channels, int batch_size, int input_width, BufferT const &input_buf,
                      BufferT const &filter_buf, BufferT const &bias_buf, BufferT &output_buf)
{
    batched::Conv1D_Bias_Act(1, kernel_width, stride, l_pad, r_pad, output_channels, input_channels, batch_size,
                             input_width, input_buf, filter_buf, bias_buf, RELU, 0.f, output_buf);
}

} // namespace small
