// Shared host-side helpers for libsmall_hip (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <mutex>

#include "../../include/small_hip.h"

namespace shp
{

constexpr int CB = SMALL_HIP_CB;          // channel block of every packed tensor
constexpr int WAVE = 64;                  // gfx950 wavefront
constexpr int NUM_XCD = 8;                // MI355X: 8 XCDs x 32 CUs, one L2 per XCD
constexpr int NUM_CU = 256;

void set_error(const char *fmt, ...);

inline int fail_hip(hipError_t e, const char *what)
{
    set_error("%s: %s", what, hipGetErrorString(e));
    return SMALL_HIP_EHIP;
}

#define SHP_HIP(call)                                                                             \
    do                                                                                            \
    {                                                                                             \
        hipError_t e__ = (call);                                                                  \
        if (e__ != hipSuccess) return shp::fail_hip(e__, #call);                                  \
    } while (0)

#define SHP_LAUNCH_CHECK(name)                                                                    \
    do                                                                                            \
    {                                                                                             \
        hipError_t e__ = hipGetLastError();                                                       \
        if (e__ != hipSuccess) return shp::fail_hip(e__, name);                                   \
    } while (0)

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int einval(const char *msg)
{
    set_error("%s", msg);
    return SMALL_HIP_EINVAL;
}

// include/small/utils.hpp:159-165 applied to the padded extent; 0 when the kernel does not fit
inline int out_dim(int in, int pad_front, int pad_back, int k, int stride)
{
    long padded = (long)in + pad_front + pad_back;
    if (k > padded) return 0;
    return (int)((padded - k) / stride + 1);
}

// window geometry shared by convolution, depthwise and pooling kernels
struct Geom
{
    int H, W, Ho, Wo, kh, kw, stride, pt, pl;
    int stride_h;      // vertical stride: `stride` for the 2-D layers, 1 for the 1-D layers (rows are independent signals)
};

// Position of a flat pixel index in [planes][Ho][Wo].  Tensors of fewer than 2^32 pixels (all that
// fit in practice) take the 32-bit division, a quarter of the instructions of the 64-bit one.
struct PixelPos
{
    int ow, oh;
    size_t plane;
};

#ifdef __HIPCC__
__device__ __forceinline__ PixelPos split_pixel(size_t pix, int Wo, int Ho)
{
    PixelPos r;
    if (pix <= 0xffffffffull)
    {
        const uint32_t p = (uint32_t)pix;
        const uint32_t row = p / (uint32_t)Wo;
        r.ow = (int)(p - row * (uint32_t)Wo);
        const uint32_t pl = row / (uint32_t)Ho;
        r.oh = (int)(row - pl * (uint32_t)Ho);
        r.plane = pl;
    }
    else
    {
        r.ow = (int)(pix % (size_t)Wo);
        pix /= (size_t)Wo;
        r.oh = (int)(pix % (size_t)Ho);
        r.plane = pix / (size_t)Ho;
    }
    return r;
}

// pix / d and pix % d for a row-less split (columns of planes)
__device__ __forceinline__ size_t split_col(size_t col, int Wo, int *ow)
{
    if (col <= 0xffffffffull)
    {
        const uint32_t c = (uint32_t)col;
        const uint32_t pl = c / (uint32_t)Wo;
        *ow = (int)(c - pl * (uint32_t)Wo);
        return pl;
    }
    *ow = (int)(col % (size_t)Wo);
    return col / (size_t)Wo;
}
#endif

// Library-owned device scratch of (current device, stream): grows on demand and is re-used by later calls on the
// same stream; other streams get their own block.  The lease holds the pool's lock: keep it alive until the last
// launch that uses `ptr` has been enqueued (a regrow on another thread frees blocks only under that lock, with a
// call that waits for the device).
struct WorkspaceLease
{
    std::unique_lock<std::mutex> lock;
    void *ptr = nullptr;
};
int lease_workspace(size_t bytes, hipStream_t stream, WorkspaceLease *lease);

// uint8 convolution filter pre-pass (conv_u8.hip): packed filter [Co/16][Ci/16][tap][16 ci][16 co] -> signed bytes in
// MFMA operand order [Co/16][S_pad][16 co][16 ci] (S = taps * Ci/16 steps, padded to a multiple of 4 with zeros),
// followed at prepared_table_offset_u8() by the int32 prefix table P[(kh+1)*(kw+1)][Co] of the per-tap filter sums
size_t prepared_bytes_u8(int kh, int kw, int Co, int Ci);
size_t prepared_table_offset_u8(int kh, int kw, int Co, int Ci);
int prepare_filter_u8(int kh, int kw, int Co, int Ci, const uint8_t *filt, void *ws, hipStream_t s);

inline hipStream_t as_stream(small_hip_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline bool pads_ok(int t, int b, int l, int r)
{
    return t >= 0 && b >= 0 && l >= 0 && r >= 0 && t < 256 && b < 256 && l < 256 && r < 256;
}

} // namespace shp
