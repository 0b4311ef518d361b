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

// Measurement switches, all in ONE environment variable read once per process: SMALL_HIP_TUNE="key=value,key=value".
// Nothing in production needs it; every default is the measured best.  Keys (integers unless noted):
//   conv_tile=CxP     force the float32 convolution's wave tile (1x1 1x2 2x1 2x2)
//   conv_tail=0|2     never / always cut left-over tiles into split-K pieces        conv_pw=0   general K loop for 1x1
//   conv_buf=0        operand streams through flat addresses instead of buffer loads (then conv_pw picks the 1x1 loop)
//   conv_splitk=0|1   force the split-K kernel off / on                             conv_streamk=0|N  equal-share split off / N per CU
//   conv_streamk_min  least K-steps for the equal-share split                       stem_lds=0  first layers without the LDS kernel
//   stem_vec=0|1      16-byte staging of first-layer patches                        smallci_valu=1  vector-ALU first layers
//   pwdw_cot=1|2      channels (x32) per workgroup of the LDS-parked pointwise + depthwise kernel
//   fuse_form=3       convolution + depthwise pairs through an intermediate buffer: always the two launches
//   dw_tile=0         depthwise without the LDS tile kernel                         dw_shape=N  force its tile shape
//   convq_min_wg, convq_table_min_wg   workgroup targets of the uint8 convolution   fmodel_fuse=0  whole-model kernel without dw + 1x1 fusion
//   fuse_conv_dw=0|2, fuse_pool=0, one_launch=0|1   the C++ wrappers' choices (read through small_hip_tune_int)
int tune_int(const char *key, int dflt);
bool tune_pair(const char *key, int *a, int *b);

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

// p / d for 0 <= p < 2^31 as one 64-bit multiply and a shift: with L = ceil(log2 d) and m = floor(2^(31+L) / d) + 1 (fits 32
// bits), p * m / 2^(31+L) = p / d + (an error below 2^-L <= 1/d), which cannot carry the quotient over an integer.  The
// run-time division it replaces is about 25 vector instructions.
struct FastDiv
{
    unsigned m;
    int sh;
};
inline FastDiv make_fast_div(unsigned d)
{
    int L = 0;
    while ((1ull << L) < d) ++L;
    FastDiv f;
    f.m = (unsigned)((1ull << (31 + L)) / d + 1);
    f.sh = 31 + L;
    return f;
}
#ifdef __HIPCC__
__device__ __forceinline__ int fast_div(int p, FastDiv f) { return (int)(((unsigned long long)(unsigned)p * f.m) >> f.sh); }
#endif

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

// Library-owned device scratch of (current device, stream): grows on demand (a larger request allocates a new block
// and keeps the old one allocated, so pointers handed out earlier stay valid) and is re-used by later calls on the
// same stream; other streams get their own block.  Blocks are freed only by small_hip_workspace_release().  The
// lease holds the pool's lock: keep it alive until the last launch that uses `ptr` has been enqueued (a release on
// another thread waits for that lock).
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
