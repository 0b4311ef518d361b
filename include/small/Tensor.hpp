// Tensor: a shape {batch, channels, height, width} over a buffer whose capacity may exceed it
// (same public surface as the reference's include/small/Tensor.hpp:22-143).  The buffer is a
// FloatBuffer / QUInt8Buffer of this build, i.e. host block + device mirror: tensors handed from
// layer to layer stay on the device.
#pragma once

#include <array>
#include <ostream>
#include <stdexcept>
#include <utility>

#include "Buffer.hpp"
#include "buffers.hpp"

namespace small
{

typedef std::array<size_t, 4UL> shape_type;   // {batch_size, num_channels, H, W}

enum ShapeFields
{
    BATCH = 0,
    CHANNEL = 1,
    HEIGHT = 2,
    WIDTH = 3
};

inline size_t compute_size(shape_type const &shape) { return shape[0] * shape[1] * shape[2] * shape[3]; }

} // namespace small

inline std::ostream &operator<<(std::ostream &ostr, small::shape_type const &shape)
{
    return ostr << "(" << shape[0] << ", " << shape[1] << ", " << shape[2] << ", " << shape[3] << ")";
}

namespace small
{

template <typename BufferT>
class Tensor
{
public:
    typedef typename BufferT::value_type value_type;

    Tensor() = delete;

    // capacity only; the shape is set by the layer that writes the tensor
    Tensor(size_t capacity) : m_shape({capacity, 1, 1, 1}), m_buffer(capacity) {}

    Tensor(shape_type const &shape) : m_shape(shape), m_buffer(compute_size(shape))
    {
        if (compute_size(shape) == 0) throw std::invalid_argument("Tensor ctor ERROR: invalid shape.");
    }

    Tensor(shape_type const &shape, BufferT const &buffer) : m_shape(shape)
    {
        require_room(buffer.size());
        m_buffer = buffer;
    }

    Tensor(shape_type const &shape, BufferT &&buffer) : m_shape(shape)
    {
        require_room(buffer.size());
        m_buffer = std::move(buffer);
    }

    void set_shape(shape_type const &new_shape)
    {
        if (compute_size(new_shape) > m_buffer.size())
            throw std::invalid_argument("Tensor::set_shape() ERROR: insufficient buffer size.");
        m_shape = new_shape;
        m_buffer.set_extent(compute_size(new_shape));      // a download to the host moves the tensor, not the capacity
    }

    shape_type const &shape() const { return m_shape; }
    size_t size() const { return compute_size(m_shape); }
    size_t capacity() const { return m_buffer.size(); }
    BufferT &buffer() { return m_buffer; }
    BufferT const &buffer() const { return m_buffer; }

    // Not in the reference (whose tensors are host memory): start uploading the host-side contents now, overlapped with
    // the layer calls that follow; the first layer that reads the tensor waits for the upload on its stream.  Feed a
    // model from two input tensors in turn: fill and prefetch one while inference() runs on the other.
    void prefetch() const { m_buffer.prefetch(); }

    void swap(Tensor<BufferT> &other) noexcept
    {
        if (this == &other) return;
        m_shape.swap(other.m_shape);
        m_buffer.swap(other.m_buffer);
    }

private:
    void require_room(size_t have) const
    {
        if (compute_size(m_shape) > have) throw std::invalid_argument("Tensor ctor ERROR: insufficient buffer size.");
    }

    shape_type m_shape;
    BufferT m_buffer;
};

} // namespace small
