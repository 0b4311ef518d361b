// FloatBuffer / QUInt8Buffer for the MI355X build of the SMaLL layer API.
//
// Same public surface as the reference's buffers
// (include/small/platforms/reference/FloatBuffer.hpp:42-167, QUInt8Buffer.hpp:31-276,
// Buffer.hpp:37-61): static blocking parameters, value_type / accum_type, value semantics
// (deep copy, move, swap), size(), data(), operator[], zero(), and for the quantised buffer the
// public fields scale, offset, multiplier, lshift, rshift, m_zero, min_val, max_val, b.
//
// Storage is a pinned host block plus a device mirror with validity tracking:
//   - data() / operator[] give HOST access, exactly as callers of the reference expect; a
//     non-const access makes the host copy the newest one.
//   - the layer functions use device_in() / device_out(); back-to-back layer calls never touch
//     the host.  Results reach the host when the caller next reads the buffer.
// The blocking of this platform is C_ob = C_ib = 16 for both element types (the reference's ZEN2
// float blocking, so its packed float tensors are layout-identical).
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>
#include <new>
#include <string>
#include <stdexcept>
#include <type_traits>
#include <utility>

#include "../small_hip.h"

#define SMALL_HAS_FLOAT_SUPPORT 1
#define SMALL_HAS_QUINT8_SUPPORT 1

#define FLOAT_W_ob 6
#define FLOAT_C_ob 16
#define FLOAT_SIMD 64
#define FLOAT_UNROLL 1
#define FLOAT_C_ib FLOAT_C_ob
#define FLOAT_NUM_FMA 1
#define FLOAT_NUM_MAX 1
#define FLOAT_NUM_LOAD 1
#define FLOAT_NUM_STORE 1

#define QUINT8_W_ob 2
#define QUINT8_C_ob 16
#define QUINT8_SIMD 64
#define QUINT8_UNROLL 1
#define QUINT8_C_ib QUINT8_C_ob
#define QUINT8_NUM_FMA 1
#define QUINT8_NUM_MAX 1
#define QUINT8_NUM_LOAD 1
#define QUINT8_NUM_STORE 1

namespace small
{

namespace detail
{

// stream used by every layer call of this thread's buffers (nullptr = default stream)
inline small_hip_stream_t &current_stream()
{
    static thread_local small_hip_stream_t s = nullptr;
    return s;
}

inline void hip_check(int status, const char *what)
{
    if (status == SMALL_HIP_OK) return;
    if (status == SMALL_HIP_ENOMEM) throw std::bad_alloc();
    throw std::runtime_error(std::string(what) + ": " + small_hip_last_error());
}

// host + device storage with validity flags
template <class T>
class MirroredStorage
{
public:
    MirroredStorage() = default;
    explicit MirroredStorage(size_t n) : m_n(n) { allocate(); }
    MirroredStorage(MirroredStorage const &o) : m_n(o.m_n), m_extent(o.m_extent)
    {
        allocate();
        if (m_n == 0) return;
        if (o.m_host_valid)
            std::memcpy(m_host, o.m_host, m_n * sizeof(T));
        else
        {
            hip_check(small_hip_memcpy_d2d(m_dev, o.m_dev, m_n * sizeof(T), current_stream()), "buffer copy");
            m_host_valid = false;
            m_dev_valid = true;
        }
    }
    MirroredStorage(MirroredStorage &&o) noexcept { swap(o); }
    MirroredStorage &operator=(MirroredStorage o) noexcept
    {
        swap(o);
        return *this;
    }
    ~MirroredStorage() { release(); }

    void swap(MirroredStorage &o) noexcept
    {
        std::swap(m_upload, o.m_upload);
        std::swap(m_extent, o.m_extent);
        std::swap(m_n, o.m_n);
        std::swap(m_host, o.m_host);
        std::swap(m_dev, o.m_dev);
        std::swap(m_host_valid, o.m_host_valid);
        std::swap(m_dev_valid, o.m_dev_valid);
    }

    size_t size() const { return m_n; }

    T *host_rw()
    {
        finish_upload();       // the host block is about to change: a copy in flight must have read it
        pull();
        m_dev_valid = false;
        return m_host;
    }
    T const *host_ro() const
    {
        pull();
        return m_host;
    }
    T const *device_in() const
    {
        push();
        return m_dev;
    }
    T *device_out()
    {
        push();                // partial / accumulating layers read what is already there
        m_host_valid = false;
        return m_dev;
    }
    // The elements [0, n) are the ones in use (a tensor's shape inside a larger buffer): a download to the host copies
    // only those.  Model classes ping-pong between two tensors sized for their largest activation; reading 64 x 1000
    // logits back must not move 200 MB.  Growing the extent makes a host copy that was downloaded at the smaller
    // extent stale again.
    void set_extent(size_t n)
    {
        if (n > m_extent && m_dev_valid) m_host_valid = false;
        m_extent = n;
    }
    // Starts the upload of host-side contents now, on the library's copy stream, behind the layer calls queued so far
    // and without blocking the host: the layer calls that follow run while it is in flight, and the first call that
    // uses this buffer makes its stream wait for it.  A caller that feeds batches from host memory fills and prefetches
    // input tensor B while the model runs on input tensor A.
    void prefetch() const
    {
        if (m_dev_valid || m_n == 0 || m_upload) return;
        hip_check(small_hip_upload_begin(m_dev, m_host, m_n * sizeof(T), current_stream(), &m_upload), "prefetch");
        m_dev_valid = true;
    }

private:
    void allocate()
    {
        if (m_n == 0) return;
        void *h = nullptr, *d = nullptr;
        hip_check(small_hip_host_malloc(&h, m_n * sizeof(T)), "host allocation");
        int rc = small_hip_malloc(&d, m_n * sizeof(T));
        if (rc != SMALL_HIP_OK)
        {
            small_hip_host_free(h);
            hip_check(rc, "device allocation");
        }
        m_host = static_cast<T *>(h);
        m_dev = static_cast<T *>(d);
    }
    void finish_upload() const
    {
        if (!m_upload) return;
        small_hip_event_t ev = m_upload;
        m_upload = nullptr;
        hip_check(small_hip_upload_finish(ev), "prefetch");
    }
    void release() noexcept
    {
        if (m_upload) (void)small_hip_upload_finish(m_upload);
        m_upload = nullptr;
        if (m_dev) small_hip_free(m_dev);
        if (m_host) small_hip_host_free(m_host);
        m_dev = nullptr;
        m_host = nullptr;
        m_n = 0;
    }
    void pull() const
    {
        if (m_host_valid || m_n == 0) return;
        const size_t n = m_extent < m_n ? m_extent : m_n;
        hip_check(small_hip_memcpy_d2h(m_host, m_dev, n * sizeof(T), current_stream()), "device to host");
        hip_check(small_hip_stream_synchronize(current_stream()), "synchronize");
        m_host_valid = true;
    }
    void push() const
    {
        if (m_upload)
        {
            // a prefetch is in flight: the layer call that is about to use the buffer waits for it on its stream
            small_hip_event_t ev = m_upload;
            m_upload = nullptr;
            hip_check(small_hip_upload_wait(ev, current_stream()), "prefetch");
        }
        if (m_dev_valid || m_n == 0) return;
        hip_check(small_hip_memcpy_h2d(m_dev, m_host, m_n * sizeof(T), current_stream()), "host to device");
        // the pinned block may be rewritten by the caller as soon as this returns
        hip_check(small_hip_stream_synchronize(current_stream()), "synchronize");
        m_dev_valid = true;
    }

    size_t m_n = 0;
    size_t m_extent = ~size_t(0);                      // elements in use (downloads stop there)
    T *m_host = nullptr;
    T *m_dev = nullptr;
    mutable bool m_host_valid = true;
    mutable bool m_dev_valid = false;
    mutable small_hip_event_t m_upload = nullptr;      // a prefetch whose completion no stream has waited for yet
};

} // namespace detail

// Route the layer calls of this thread onto a HIP stream (hipStream_t); nullptr = default stream.
inline void set_stream(void *hip_stream) { detail::current_stream() = hip_stream; }
// Wait until every layer call issued so far has finished.
inline void synchronize() { detail::hip_check(small_hip_stream_synchronize(detail::current_stream()), "synchronize"); }

//****************************************************************************
class FloatBuffer
{
public:
    static uint32_t const W_ob{FLOAT_W_ob};
    static uint32_t const C_ob{FLOAT_C_ob};
    static uint32_t const SIMD{FLOAT_SIMD};
    static uint32_t const UNROLL{FLOAT_UNROLL};
    static uint32_t const C_ib{FLOAT_C_ib};
    static uint32_t const NUM_FMA{FLOAT_NUM_FMA};
    static uint32_t const NUM_MAX{FLOAT_NUM_MAX};
    static uint32_t const NUM_LOAD{FLOAT_NUM_LOAD};
    static uint32_t const NUM_STORE{FLOAT_NUM_STORE};

    typedef float value_type;
    typedef float accum_type;

    FloatBuffer() = default;
    FloatBuffer(size_t num_elts) : m_store(num_elts) {}
    FloatBuffer(FloatBuffer const &) = default;
    FloatBuffer(FloatBuffer &&) noexcept = default;
    FloatBuffer &operator=(FloatBuffer const &other)
    {
        if (this != &other)
        {
            FloatBuffer tmp(other);   // strong exception guarantee, as in the reference
            swap(tmp);
        }
        return *this;
    }
    FloatBuffer &operator=(FloatBuffer &&other) noexcept
    {
        if (this != &other)
        {
            FloatBuffer tmp(std::move(other));
            swap(tmp);
        }
        return *this;
    }

    size_t size() const { return m_store.size(); }
    value_type *data() { return m_store.host_rw(); }
    value_type const *data() const { return m_store.host_ro(); }
    value_type &operator[](size_t index) { return m_store.host_rw()[index]; }
    value_type const &operator[](size_t index) const { return m_store.host_ro()[index]; }
    void swap(FloatBuffer &other) { m_store.swap(other.m_store); }
    accum_type zero() const { return (accum_type)0; }

    // device side, used by the layer functions
    value_type const *device_in() const { return m_store.device_in(); }
    value_type *device_out() { return m_store.device_out(); }
    // start uploading host-side contents now, overlapped with the layer calls that follow (see MirroredStorage::prefetch)
    void prefetch() const { m_store.prefetch(); }
    // only the first n elements are in use: downloads to the host stop there (Tensor::set_shape calls this)
    void set_extent(size_t n) { m_store.set_extent(n); }

private:
    detail::MirroredStorage<float> m_store;
};

//****************************************************************************
class QUInt8Buffer
{
public:
    static uint32_t const W_ob{QUINT8_W_ob};
    static uint32_t const C_ob{QUINT8_C_ob};
    static uint32_t const SIMD{QUINT8_SIMD};
    static uint32_t const UNROLL{QUINT8_UNROLL};
    static uint32_t const C_ib{QUINT8_C_ib};
    static uint32_t const NUM_FMA{QUINT8_NUM_FMA};
    static uint32_t const NUM_MAX{QUINT8_NUM_MAX};
    static uint32_t const NUM_LOAD{QUINT8_NUM_LOAD};
    static uint32_t const NUM_STORE{QUINT8_NUM_STORE};

    typedef uint8_t value_type;
    typedef int32_t accum_type;

    QUInt8Buffer() { quantized_init(); }
    QUInt8Buffer(size_t num_elts) : m_store(num_elts) { quantized_init(); }
    QUInt8Buffer(QUInt8Buffer const &) = default;
    QUInt8Buffer(QUInt8Buffer &&other) noexcept
    {
        quantized_init();
        swap(other);
    }
    QUInt8Buffer &operator=(QUInt8Buffer const &other)
    {
        if (this != &other)
        {
            QUInt8Buffer tmp(other);
            swap(tmp);
        }
        return *this;
    }
    QUInt8Buffer &operator=(QUInt8Buffer &&other) noexcept
    {
        if (this != &other)
        {
            QUInt8Buffer tmp(std::move(other));
            swap(tmp);
        }
        return *this;
    }

    size_t size() const { return m_store.size(); }
    value_type *data() { return m_store.host_rw(); }
    value_type const *data() const { return m_store.host_ro(); }
    value_type &operator[](size_t index) { return m_store.host_rw()[index]; }
    value_type const &operator[](size_t index) const { return m_store.host_ro()[index]; }

    void swap(QUInt8Buffer &other)
    {
        if (this == &other) return;
        std::swap(scale, other.scale);
        std::swap(offset, other.offset);
        std::swap(multiplier, other.multiplier);
        std::swap(lshift, other.lshift);
        std::swap(rshift, other.rshift);
        std::swap(m_zero, other.m_zero);
        std::swap(min_val, other.min_val);
        std::swap(max_val, other.max_val);
        std::swap(b, other.b);
        m_store.swap(other.m_store);
    }

    accum_type zero() const { return m_zero; }

    value_type const *device_in() const { return m_store.device_in(); }
    value_type *device_out() { return m_store.device_out(); }
    void prefetch() const { m_store.prefetch(); }
    void set_extent(size_t n) { m_store.set_extent(n); }
    small_hip_quant quant() const { return small_hip_quant{m_zero, multiplier, lshift, rshift}; }

public:
    // quantisation parameters travel with the buffer, as in the reference
    float scale;
    int32_t offset;
    int32_t multiplier;
    int lshift;
    int rshift;
    accum_type m_zero;
    int min_val;
    int max_val;
    uint8_t b;

private:
    // Default parameters of a buffer that represents reals in [-1, 1] with 8 bits
    // (reference QUInt8Buffer.hpp:234-272): scale = 2/255, zero = 128, and the scale expressed
    // as a Q31 multiplier with a power-of-two shift  ->  multiplier 1077952576, rshift 6.
    void quantized_init()
    {
        const double lo = -1.0, hi = 1.0;
        b = 8;
        const double qmax = 255.0, qmin = 0.0;
        const double real_scale = (hi - lo) / (qmax - qmin) + 1e-17;
        int exponent = 0;
        const double mantissa = std::frexp(real_scale, &exponent);
        long long fixed = std::llround(mantissa * 2147483648.0);
        if (fixed == (1LL << 31))
        {
            fixed >>= 1;
            ++exponent;
        }
        if (exponent < -31)
        {
            exponent = 0;
            fixed = 0;
        }
        if (exponent > 30)
        {
            exponent = 30;
            fixed = (1LL << 31) - 1;
        }
        multiplier = static_cast<int32_t>(fixed);
        m_zero = static_cast<accum_type>(std::rint((hi * qmin - lo * qmax) / (hi - lo)));
        scale = static_cast<float>(real_scale);
        lshift = exponent > 0 ? exponent : 0;
        rshift = exponent > 0 ? 0 : -exponent;
        min_val = 0;
        max_val = 255;
        offset = 0;
    }

    detail::MirroredStorage<uint8_t> m_store;
};

//**********************************************************************
// reference Buffer.hpp:37-61
template <class BufferT>
inline BufferT *alloc_buffer(size_t num_elts)
{
    static_assert(std::is_same<BufferT, FloatBuffer>::value || std::is_same<BufferT, QUInt8Buffer>::value,
                  "small::alloc_buffer: unsupported buffer type");
    return new BufferT(num_elts);
}

template <class BufferT>
inline void free_buffer(BufferT *buffer)
{
    delete buffer;
}

} // namespace small
