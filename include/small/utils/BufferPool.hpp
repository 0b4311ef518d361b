// Pool of equally sized tensors for DAGModel (reference include/small/utils/BufferPool.hpp:30-106): pop hands out
// a pooled tensor, or a new one when the pool is empty; push returns it.  Device and pinned host memory of a
// tensor are allocated once and recycled, so a model's inference() allocates nothing after the first pass.
#pragma once

#include <memory>
#include <stdexcept>
#include <vector>

#include "../Tensor.hpp"

namespace small
{

template <class BufferT>
class BufferPool
{
public:
    BufferPool() : m_buffer_size(0) {}
    BufferPool(size_t buffer_size, size_t num_buffers) : m_buffer_size(buffer_size)
    {
        for (size_t i = 0; i < num_buffers; ++i) m_pool.emplace_back(new Tensor<BufferT>(m_buffer_size));
    }
    BufferPool(BufferPool const &) = delete;
    BufferPool &operator=(BufferPool const &) = delete;
    BufferPool(BufferPool &&) = default;
    BufferPool &operator=(BufferPool &&) = default;

    size_t buffer_size() const { return m_buffer_size; }
    size_t available() const { return m_pool.size(); }

    // the caller owns the tensor until it pushes it back
    Tensor<BufferT> *pop_buffer()
    {
        if (m_pool.empty()) return new Tensor<BufferT>(m_buffer_size);
        Tensor<BufferT> *t = m_pool.back().release();
        m_pool.pop_back();
        return t;
    }

    void push_buffer(Tensor<BufferT> *t)
    {
        if (t->capacity() != m_buffer_size)
            throw std::invalid_argument("BufferPool::push_buffer ERROR: tensor of another size.");
        m_pool.emplace_back(t);
    }

private:
    size_t m_buffer_size;
    std::vector<std::unique_ptr<Tensor<BufferT>>> m_pool;
};

} // namespace small
