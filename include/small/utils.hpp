// Shape arithmetic of the SMaLL layer API (same names and results as the reference's
// include/small/utils.hpp:20-231; re-stated, not copied).
#pragma once

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <stdexcept>

namespace small
{

typedef uint32_t index_t;
typedef uint32_t dim_t;

enum PaddingEnum
{
    PADDING_V, // "valid": no padding
    PADDING_F  // "full": pad so that every input pixel is covered (TensorFlow-"same" split)
};

// front/back padding of one dimension for PADDING_F (reference utils.hpp:43-64)
inline void calc_padding(size_t I_dim, uint32_t K_dim, uint16_t stride, uint8_t &padding_front,
                         uint8_t &padding_back)
{
    const size_t rem = I_dim % stride;
    const size_t covered = (rem == 0) ? stride : rem;
    const uint32_t total = (K_dim > covered) ? static_cast<uint32_t>(K_dim - covered) : 0u;
    padding_front = static_cast<uint8_t>(total / 2);
    padding_back = static_cast<uint8_t>(total - total / 2);
}

inline uint8_t calc_front_padding(PaddingEnum padding_type, uint32_t I_dim, uint32_t K_dim, uint16_t stride)
{
    if (padding_type == PADDING_V) return 0;
    uint8_t f, b;
    calc_padding(I_dim, K_dim, stride, f, b);
    return f;
}

inline uint8_t calc_back_padding(PaddingEnum padding_type, uint32_t I_dim, uint32_t K_dim, uint16_t stride)
{
    if (padding_type == PADDING_V) return 0;
    uint8_t f, b;
    calc_padding(I_dim, K_dim, stride, f, b);
    return b;
}

// number of window positions of an un-padded extent (reference utils.hpp:159-165); 0 if none fit
inline dim_t output_dim(dim_t input_dim, dim_t stride, dim_t kernel_dim)
{
    if (kernel_dim > input_dim || stride == 0) return 0;
    return (input_dim - kernel_dim) / stride + 1;
}

inline dim_t output_dim_new(dim_t input_dim, dim_t stride, dim_t kernel_dim)
{
    return output_dim(input_dim, stride, kernel_dim);
}

inline size_t compute_output_dim(size_t input_dim, size_t kernel_dim, size_t stride, PaddingEnum padding)
{
    if (padding == PADDING_V && input_dim >= kernel_dim) return (input_dim - kernel_dim) / stride + 1;
    if (padding == PADDING_F)
    {
        uint8_t f, b;
        calc_padding(input_dim, static_cast<uint32_t>(kernel_dim), static_cast<uint16_t>(stride), f, b);
        return 1 + (input_dim + f + b - kernel_dim) / stride;
    }
    throw std::invalid_argument("compute_output_dim: Bad kernel and image size combination.");
}

inline void compute_padding_output_dim(size_t unpadded_input_dim, uint32_t kernel_dim, uint32_t stride,
                                       PaddingEnum padding_type, uint8_t &front_pad, uint8_t &back_pad,
                                       size_t &output_dim)
{
    front_pad = back_pad = 0;
    output_dim = 0;
    if (padding_type == PADDING_F)
        calc_padding(unpadded_input_dim, kernel_dim, static_cast<uint16_t>(stride), front_pad, back_pad);
    const size_t padded = unpadded_input_dim + front_pad + back_pad;
    if (padded < kernel_dim)
        throw std::invalid_argument("compute_padding_output_dim() ERROR: Bad combination, kernel too large.");
    output_dim = 1 + (padded - kernel_dim) / stride;
}

} // namespace small
