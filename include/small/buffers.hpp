// Packed-layout index maps, pack/unpack and test initialisers of the SMaLL layer API
// (same names, arguments and results as the reference's include/small/buffers.hpp:22-607;
// re-stated, not copied).
#pragma once

#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <stdexcept>
#include <string>
#include <type_traits>

#include "Buffer.hpp"

namespace small
{

enum BufferTypeEnum
{
    INPUT,       // activations read by a layer:   [C/C_ib][H][W][C_ib]
    OUTPUT,      // activations written by a layer: [C/C_ob][H][W][C_ob]
    FILTER_DW,   // depthwise filter   [C/C_ob][Fh][Fw][1][C_ob]
    FILTER_CONV, // convolution filter [Co/C_ob][Ci/C_ib][Fh][Fw][C_ib][C_ob]
    FILTER_FC    // fully connected = FILTER_CONV with a 1x1 window
};

namespace detail
{
// the input-channel block actually used: the platform block, or the channel count itself for
// 1, 2 and 3 channel first layers (reference buffers.hpp:52-67)
inline uint32_t effective_block(uint32_t num_channels, uint32_t blocking, char const *too_small_msg)
{
    if (num_channels < blocking)
    {
        if (num_channels == 1 || num_channels == 2 || num_channels == 3) return num_channels;
        throw std::runtime_error(too_small_msg);
    }
    if (num_channels % blocking != 0) throw std::runtime_error("num_channels %% channel_blocking != 0");
    return blocking;
}
} // namespace detail

inline size_t packed_weight_index(uint32_t num_filters, uint32_t num_channels, uint32_t num_rows,
                                  uint32_t num_cols, uint32_t filter_blocking, uint32_t channel_blocking,
                                  size_t filter_idx, size_t channel_idx, size_t height_idx, size_t width_idx)
{
    (void)num_filters;
    const size_t cib = detail::effective_block(
        num_channels, channel_blocking, "num_channels < channel_blocking && num_channels not in {1, 2, 3}");
    const size_t cob = filter_blocking;
    const size_t tile = cib * cob;                      // one filter tap of one (co, ci) block pair
    const size_t ci_block = (size_t)num_rows * num_cols * tile;
    const size_t co_block = (num_channels / cib) * ci_block;
    return (filter_idx / cob) * co_block + (channel_idx / cib) * ci_block +
           (height_idx * num_cols + width_idx) * tile + (channel_idx % cib) * cob + (filter_idx % cob);
}

inline size_t packed_buffer_index(uint32_t num_channels, uint32_t num_rows, uint32_t num_cols,
                                  uint32_t channel_blocking, size_t channel_idx, size_t height_idx,
                                  size_t width_idx)
{
    const size_t cb = detail::effective_block(num_channels, channel_blocking,
                                              "num_channels < channel_blocking && num_channels != 3");
    return (channel_idx / cb) * ((size_t)num_rows * num_cols * cb) +
           (height_idx * num_cols + width_idx) * cb + (channel_idx % cb);
}

namespace detail
{
// Walks every element of a flat [C_o][C_i][H][W] tensor in packed order and calls
// visit(packed_offset, flat_offset).  Returns the element count, 0 on an unsupported type.
template <class Visit>
uint32_t walk_packed(BufferTypeEnum type, uint32_t C_o, uint32_t C_i, uint32_t H, uint32_t W, uint32_t C_ib,
                     uint32_t C_ob, Visit visit)
{
    if (type == FILTER_FC) H = W = 1;
    if (type == FILTER_DW) C_ib = 1;
    if ((type == FILTER_CONV || type == INPUT) && C_i < C_ib) C_ib = C_i;   // 1/2/3-channel first layer
    uint32_t in_block, out_block;
    switch (type)
    {
    case INPUT: in_block = C_ib; out_block = 1; break;
    case OUTPUT: in_block = C_ob; out_block = 1; break;
    case FILTER_DW:
    case FILTER_CONV:
    case FILTER_FC: in_block = C_ib; out_block = C_ob; break;
    default: std::printf("ERROR: unsupported tensor buffer type\n"); return 0;
    }
    size_t packed = 0;
    for (uint32_t o0 = 0; o0 < C_o; o0 += out_block)
        for (uint32_t i0 = 0; i0 < C_i; i0 += in_block)
            for (uint32_t h = 0; h < H; ++h)
                for (uint32_t w = 0; w < W; ++w)
                    for (uint32_t i = 0; i < in_block; ++i)
                        for (uint32_t o = 0; o < out_block; ++o)
                            visit(packed++, (((size_t)(o0 + o) * C_i + (i0 + i)) * H + h) * W + w);
    return C_o * C_i * H * W;
}
} // namespace detail

template <class ScalarT>
uint32_t convert_tensor2dc(ScalarT const *flat_t, BufferTypeEnum type, uint32_t C_o, uint32_t C_i, uint32_t H,
                           uint32_t W, uint32_t _C_ib, uint32_t _C_ob, ScalarT *dc_array)
{
    return detail::walk_packed(type, C_o, C_i, H, W, _C_ib, _C_ob,
                               [&](size_t p, size_t f) { dc_array[p] = flat_t[f]; });
}

template <class ScalarT>
uint32_t convert_dc2tensor(ScalarT const *dc_array, BufferTypeEnum type, uint32_t C_o, uint32_t C_i, uint32_t H,
                           uint32_t W, uint32_t _C_ib, uint32_t _C_ob, ScalarT *flat_t)
{
    return detail::walk_packed(type, C_o, C_i, H, W, _C_ib, _C_ob,
                               [&](size_t p, size_t f) { flat_t[f] = dc_array[p]; });
}

namespace detail
{
// pack_buffer / unpack_buffer run on the device (small_hip_pack / small_hip_unpack): the source is
// uploaded if its newest copy is on the host, the result stays on the device for the layer call that
// follows.  An unknown tensor type prints the reference's message and returns 0 as the reference does;
// extents that do not fill their channel blocks (the reference then indexes past the tensor) throw.
template <class BufferT, class Fn>
uint32_t repack_on_device(Fn fn, BufferT const &src, BufferTypeEnum type, uint32_t dim0, uint32_t dim1,
                          uint32_t dim2, uint32_t dim3, uint32_t c_ib, uint32_t c_ob, BufferT &dst, char const *who)
{
    if (type < INPUT || type > FILTER_FC)
    {
        std::printf("ERROR: unsupported tensor buffer type\n");
        return 0;
    }
    const size_t n = (size_t)dim0 * dim1 * (type == FILTER_FC ? 1 : (size_t)dim2 * dim3);
    if (n == 0) return 0;
    if (src.size() < n || dst.size() < n) throw std::invalid_argument(std::string(who) + " ERROR: buffer too small.");
    const int rc = fn((int)type, 1, dim0, dim1, dim2, dim3, c_ib, c_ob, src.device_in(), dst.device_out(),
                      sizeof(typename BufferT::value_type), current_stream());
    if (rc == SMALL_HIP_EINVAL) throw std::invalid_argument(std::string(who) + " ERROR: " + small_hip_last_error());
    hip_check(rc, who);
    return (uint32_t)((size_t)dim0 * dim1 * dim2 * dim3);
}
} // namespace detail

template <class BufferT>
uint32_t pack_buffer(BufferT const &flat_t, BufferTypeEnum type, uint32_t dim0, uint32_t dim1, uint32_t dim2,
                     uint32_t dim3, uint32_t _C_ib, uint32_t _C_ob, BufferT &dc_array)
{
    return detail::repack_on_device(small_hip_pack, flat_t, type, dim0, dim1, dim2, dim3, _C_ib, _C_ob, dc_array,
                                    "pack_buffer");
}

template <class BufferT>
uint32_t unpack_buffer(BufferT const &dc_array, BufferTypeEnum type, uint32_t dim0, uint32_t dim1,
                       uint32_t dim2, uint32_t dim3, uint32_t _C_ib, uint32_t _C_ob, BufferT &flat_t)
{
    return detail::repack_on_device(small_hip_unpack, dc_array, type, dim0, dim1, dim2, dim3, _C_ib, _C_ob, flat_t,
                                    "unpack_buffer");
}

//****************************************************************************
// test initialisers (reference buffers.hpp:420-556)
template <class BufferT>
void init(BufferT &ptr, uint32_t numel)
{
    if (numel > ptr.size()) throw std::invalid_argument("init ERROR: buffer too small.");
    auto *p = ptr.data();
    if constexpr (std::is_same<float, typename BufferT::value_type>::value)
    {
        for (size_t i = 0; i < numel; ++i) p[i] = 2.0 * ((float)rand() / RAND_MAX) - 1;
    }
    else
    {
        srand(42);
        for (size_t i = 0; i < numel; ++i) p[i] = rand() % 10;
    }
}

template <class BufferT>
void init_ones(BufferT &ptr, uint32_t numel)
{
    if (numel > ptr.size()) throw std::invalid_argument("init_ones ERROR: buffer too small.");
    auto *p = ptr.data();
    for (size_t i = 0; i < numel; ++i) p[i] = (typename BufferT::value_type)1;
}

template <class BufferT>
void init_zeros(BufferT &ptr, uint32_t numel)
{
    if (numel > ptr.size()) throw std::invalid_argument("init_zeroes ERROR: buffer too small.");
    auto *p = ptr.data();
    for (size_t i = 0; i < numel; ++i) p[i] = (typename BufferT::value_type)0;
}

template <class BufferT, uint32_t _C_ob>
void init_arange(BufferT &ptr, uint32_t H, uint32_t W, uint32_t C)
{
    if ((size_t)C * H * W > ptr.size()) throw std::invalid_argument("init_arange ERROR: buffer too small.");
    auto *p = ptr.data();
    size_t at = 0;
    for (size_t c0 = 0; c0 < C; c0 += _C_ob)
        for (size_t h = 0; h < H; ++h)
            for (size_t w = 0; w < W; ++w)
                for (size_t c = 0; c < _C_ob; ++c)
                    p[at++] = (typename BufferT::value_type)(c + c0 + w * C + h * (W * C));
}

template <class BufferT>
void init_norm(BufferT &ptr, uint32_t numel, uint32_t C_o)
{
    if (numel > ptr.size()) throw std::invalid_argument("init_norm ERROR: buffer too small.");
    auto *p = ptr.data();
    if constexpr (std::is_same<float, typename BufferT::value_type>::value)
    {
        const float norm = (1.0 * C_o) / (1.0 * ptr.size());
        for (size_t i = 0; i < ptr.size(); ++i) p[i] = norm;
    }
    else
    {
        const typename BufferT::value_type norm = (1.0 * C_o) / (1.0 * numel);
        for (size_t i = 0; i < numel; ++i) p[i] = norm;
    }
}

// absolute-difference comparison (reference buffers.hpp:561-607)
template <class BufferT>
bool equals(uint32_t numel, BufferT const &buf1, BufferT const &buf2, float tolerance = 1.0e-8)
{
    if (buf1.size() < numel || buf2.size() < numel) return false;
    auto const *a = buf1.data();
    auto const *b = buf2.data();
    bool same = true;
    for (size_t i = 0; i < numel; ++i)
    {
        if constexpr (std::is_same<float, typename BufferT::value_type>::value)
        {
            if (std::fabs(b[i] - a[i]) > tolerance)
            {
                std::printf("equals ERROR: %zu, buf2/buf1 %.4f/%.4f, diff %.4f\n", i, b[i], a[i], b[i] - a[i]);
                same = false;
            }
        }
        else if (a[i] != b[i])
        {
            std::cout << "equals ERROR: i=" << i << ", buf1[i]=" << (int)a[i] << ", buf2[i]=" << (int)b[i] << std::endl;
            same = false;
        }
    }
    return same;
}

} // namespace small
