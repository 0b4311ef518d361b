// DepthwiseConv2D / PartialDepthwiseConv2D (float32, optional fused bias + activation) and
// DepthwiseConv2D (uint8).  Bandwidth-bound, no MFMA: a lane owns four channels of one output
// pixel, so the four lanes of a (pixel, channel-block) touch one 64-byte line per tap and a wave
// covers 16 neighbouring output pixels.  Three float32 kernels, picked by shape:
//   - 3x3 on images of at least 7x7 (28x28 at stride 2) outputs: input tile staged in LDS
//   - other 3x3: a lane loads a strip of rows into registers
//   - any other window: one output per lane, taps read through the vector cache
#include "common.h"
#include "quant.h"

#include <cstdlib>

using namespace shp;

namespace
{

constexpr int TPB = 256;

struct Epi
{
    const float4 *bias;   // may be null
    int act;
    float slope;
    int accumulate;
};

__device__ __forceinline__ float act1(float v, int act, float slope)
{
    if (act == SMALL_HIP_ACT_RELU) return v > 0.f ? v : 0.f;
    if (act == SMALL_HIP_ACT_LEAKY) return v > 0.f ? v : v * slope;
    return v;
}

// The same without a branch on the activation kind (a branch per output row splits the unrolled
// compute loop into blocks the compiler cannot schedule across): negative inputs are multiplied by
// 1 (none), 0 (ReLU) or the slope (LeakyReLU); "+ 0.f" turns the -0 of x * 0 into the +0 ReLU gives.
__device__ __forceinline__ float act_scale(int act, float slope)
{
    return act == SMALL_HIP_ACT_RELU ? 0.f : act == SMALL_HIP_ACT_LEAKY ? slope : 1.f;
}
__device__ __forceinline__ float act_bf(float v, float neg_scale)
{
    const float n = fmaf(v, neg_scale, 0.f);
    return v > 0.f ? v : n;
}

// KH/KW == 0: run-time window size
template <int KH, int KW>
__global__ __launch_bounds__(TPB) void dw_f32_kernel(const float4 *__restrict__ in,
                                                     const float4 *__restrict__ filt, float4 *out,
                                                     size_t total4, int cblocks, Geom g, Epi e)
{
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= total4) return;
    const int kh = KH ? KH : g.kh, kw = KW ? KW : g.kw;
    const int q = (int)(i & 3);
    const PixelPos pp = split_pixel(i >> 2, g.Wo, g.Ho);
    const int ow = pp.ow, oh = pp.oh;
    const size_t plane = pp.plane;                        // n * cblocks + cb
    const int cbk = (int)((uint32_t)plane % (uint32_t)cblocks);   // planes < 2^31 (checked by the launcher)
    const float4 *src = in + plane * (size_t)g.H * g.W * 4 + q;
    const float4 *f = filt + (size_t)cbk * kh * kw * 4 + q;
    const int ih0 = oh * g.stride - g.pt, iw0 = ow * g.stride - g.pl;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (e.accumulate) acc = out[i];
    else if (e.bias) acc = e.bias[cbk * 4 + q];
#pragma unroll
    for (int a = 0; a < kh; ++a)
    {
        const int ih = ih0 + a;
        if (ih < 0 || ih >= g.H) continue;
#pragma unroll
        for (int b = 0; b < kw; ++b)
        {
            const int iw = iw0 + b;
            if (iw < 0 || iw >= g.W) continue;
            const float4 v = src[((size_t)ih * g.W + iw) * 4];
            const float4 w = f[(a * kw + b) * 4];
            acc.x = fmaf(v.x, w.x, acc.x); acc.y = fmaf(v.y, w.y, acc.y);
            acc.z = fmaf(v.z, w.z, acc.z); acc.w = fmaf(v.w, w.w, acc.w);
        }
    }
    acc.x = act1(acc.x, e.act, e.slope); acc.y = act1(acc.y, e.act, e.slope);
    acc.z = act1(acc.z, e.act, e.slope); acc.w = act1(acc.w, e.act, e.slope);
    out[i] = acc;
}

// 3x3 depthwise, the shape every MobileNet / DS-CNN block uses.  A lane owns one output column,
// four channels and ROWS consecutive output rows.  It first issues every 16-byte load of the
// (ROWS-1)*STRIDE+3 input rows x 3 columns it needs (all in flight together), then computes the
// ROWS outputs from registers: 4.5 loads per output at stride 1 instead of 9, the nine filter taps
// are loaded once per lane, and the memory latency is paid once per lane instead of once per tap.
// Neighbouring lanes are neighbouring columns, so each row access of a wave is one contiguous
// kilobyte (stride 1).
template <int STRIDE, int ROWS, bool ACC>
__global__ __launch_bounds__(TPB) void dw3x3_f32_strip_kernel(const float4 *__restrict__ in,
                                                              const float4 *__restrict__ filt, float4 *out,
                                                              size_t ncols4, int cblocks, int nstrips,
                                                              int nblocks, int per_xcd, Geom g, Epi e)
{
    constexpr int NR = (ROWS - 1) * STRIDE + 3;
    // XCD-aware id: consecutive logical ids share an XCD, and the strips of one column block are
    // consecutive, so the two halo rows between neighbouring strips are served by that XCD's L2
    const int bid = blockIdx.x;
    const int lid = (bid % NUM_XCD) * per_xcd + bid / NUM_XCD;
    if (lid >= nblocks) return;
    const int strip = lid % nstrips;
    const size_t i = (size_t)(lid / nstrips) * TPB + threadIdx.x;  // (plane, ow, quad)
    if (i >= ncols4) return;
    const int q = (int)(i & 3);
    int ow;
    const size_t plane = split_col(i >> 2, g.Wo, &ow);              // n * cblocks + cb
    const int cbk = (int)((uint32_t)plane % (uint32_t)cblocks);     // planes < 2^31 (checked by the launcher)
    const float4 *src = in + plane * (size_t)g.H * g.W * 4 + q;
    float4 *dst = out + plane * (size_t)g.Ho * g.Wo * 4 + (size_t)ow * 4 + q;
    const float4 *f = filt + (size_t)cbk * 36 + q;

    const int oh_lo = strip * ROWS;
    const int ih_lo = oh_lo * STRIDE - g.pt;
    const int iw0 = ow * STRIDE - g.pl;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);

    float4 x[NR][3];
#pragma unroll
    for (int r = 0; r < NR; ++r)
    {
        const int ih = ih_lo + r;
        const bool rv = ih >= 0 && ih < g.H;
        const float4 *p = src + ((size_t)(rv ? ih : 0) * g.W) * 4;
#pragma unroll
        for (int c = 0; c < 3; ++c)
        {
            const int iw = iw0 + c;
            const bool ok = rv && iw >= 0 && iw < g.W;
            x[r][c] = p[(size_t)(ok ? iw : 0) * 4];
            if (!ok) x[r][c] = zero;
        }
    }
    float4 w[9];
#pragma unroll
    for (int t = 0; t < 9; ++t) w[t] = f[t * 4];
    float4 bias = zero;
    if (e.bias) bias = e.bias[cbk * 4 + q];
    const float nscale = act_scale(e.act, e.slope);

    // no branch inside the unrolled rows: rows past the end are computed and not stored
#pragma unroll
    for (int o = 0; o < ROWS; ++o)
    {
        const int oh = oh_lo + o;
        const bool ok = oh < g.Ho;
        float4 acc = bias;
        if (ACC) { acc = zero; if (ok) acc = dst[(size_t)oh * g.Wo * 4]; }
#pragma unroll
        for (int a = 0; a < 3; ++a)
#pragma unroll
            for (int c = 0; c < 3; ++c)
            {
                const float4 v = x[o * STRIDE + a][c];
                const float4 k = w[a * 3 + c];
                acc.x = fmaf(v.x, k.x, acc.x); acc.y = fmaf(v.y, k.y, acc.y);
                acc.z = fmaf(v.z, k.z, acc.z); acc.w = fmaf(v.w, k.w, acc.w);
            }
        if (ACC) { acc.x += bias.x; acc.y += bias.y; acc.z += bias.z; acc.w += bias.w; }   // bias is zero without one
        acc.x = act_bf(acc.x, nscale); acc.y = act_bf(acc.y, nscale);
        acc.z = act_bf(acc.z, nscale); acc.w = act_bf(acc.w, nscale);
        if (ok) dst[(size_t)oh * g.Wo * 4] = acc;
    }
}

// 3x3 depthwise through LDS.  A workgroup owns a TW x TH tile of output pixels of one (image,
// channel block) plane.  The input pixels under it (64 bytes each) are fetched from memory exactly
// once, in row-contiguous 16-byte pieces, and parked in LDS with zeros where the tile hangs over
// the image; the nine filter taps of the block go to LDS too.  The staging is done by the memory
// pipeline (global_load_lds_dwordx4: a wave's 64 lanes write one KiB of consecutive LDS, each lane
// gives its own global address; pieces outside the image come from a block of zeros): no lane holds
// the pieces in registers or waits for them before it can issue an LDS store (against staging
// through registers, batch 64: 512 channels on 14x14 13.0 -> 10.0 us, 256 on 28x28 21.1 -> 17.4,
// 128 on 56x56 32.7 -> 30.3).  A lane then owns one output column, four channels and R consecutive
// rows.  At stride 1 it slides a three-row register window down the staged tile (three 16-byte LDS
// reads per output); at stride 2 it reads its nine taps per output.  The strip kernel issued 4.5
// (stride 1) to 7 (stride 2) vector-cache loads per output plus nine tap loads per lane, and that
// cache, not HBM, was its limit.
__device__ __align__(16) const float g_dw_zero[4] = {0.f, 0.f, 0.f, 0.f};

template <int S, int TW, int R, bool ACC, int SRU = 0>
__global__ __launch_bounds__(TPB) void dw3x3_f32_tile_kernel(const float4 *__restrict__ in,
                                                             const float4 *__restrict__ filt, float4 *out,
                                                             int cblocks, int tiles_x, int tiles_y,
                                                             int nblocks, int per_xcd, Geom g, Epi e)
{
    constexpr int SR = SRU ? SRU : 64 / TW;
    constexpr int TH = SR * R;
    constexpr int IW = (TW - 1) * S + 3, IH = (TH - 1) * S + 3;
    constexpr int ROW4 = IW * 4;
    constexpr int E = IH * ROW4;
    constexpr int NLD = (E + TPB - 1) / TPB;
    constexpr int EP = NLD * TPB;                            // every lane writes a piece in every round
    __shared__ float4 sX[EP];
    __shared__ float4 sW[64];

    const int bid = blockIdx.x;
    const int lid = (bid % NUM_XCD) * per_xcd + bid / NUM_XCD;
    if (lid >= nblocks) return;              // the whole workgroup leaves, before any barrier
    const int tiles = tiles_x * tiles_y;
    const int plane = lid / tiles, tile = lid - plane * tiles;
    const int tyi = tile / tiles_x, txi = tile - tyi * tiles_x;
    const int cbk = plane % cblocks;
    const int oh0 = tyi * TH, ow0 = txi * TW;
    const int ih0 = oh0 * S - g.pt, iw0 = ow0 * S - g.pl;
    const float4 *src = in + (size_t)plane * g.H * g.W * 4;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    const float4 *gzero = reinterpret_cast<const float4 *>(g_dw_zero);
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

#pragma unroll
    for (int k = 0; k < NLD; ++k)
    {
        const int el = tid + k * TPB;
        const int r = el / ROW4, c4 = el - r * ROW4;
        const int ih = ih0 + r, iw = iw0 + (c4 >> 2);
        const bool ok = el < E && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
        const float4 *gp = ok ? src + ((size_t)ih * g.W + iw) * 4 + (c4 & 3) : gzero;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                         (__attribute__((address_space(3))) void *)&sX[k * TPB + wave * 64], 16, 0, 0);
    }
    if (wave == 0)
    {
        const float4 *gp = filt + (size_t)cbk * 36 + (tid < 36 ? tid : 35);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                         (__attribute__((address_space(3))) void *)&sW[0], 16, 0, 0);
    }

    const int q = tid & 3, slot = tid >> 2;
    const int tx = slot % TW, sy_raw = slot / TW;
    const bool slot_on = sy_raw < SR;
    const int sy = slot_on ? sy_raw : 0;      // idle slots read in bounds and store nothing
    const int ow = ow0 + tx;
    float4 bias = zero;
    if (e.bias) bias = e.bias[cbk * 4 + q];
    const float nscale = act_scale(e.act, e.slope);
    const float4 *xs = sX + ((sy * R * S) * IW + tx * S) * 4 + q;
    float4 *dst = out + (size_t)plane * g.Ho * g.Wo * 4 + (size_t)ow * 4 + q;
    const bool col_ok = slot_on && ow < g.Wo;

    __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0): this lane's pieces have landed
    __syncthreads();                         // everyone's have

    float4 w[9];
#pragma unroll
    for (int t = 0; t < 9; ++t) w[t] = sW[t * 4 + q];
    float4 win[3][3];
    if (S == 1)
    {
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int c = 0; c < 3; ++c) win[a][c] = xs[(a * IW + c) * 4];
    }
#pragma unroll
    for (int o = 0; o < R; ++o)
    {
        if (S == 1)
        {
#pragma unroll
            for (int c = 0; c < 3; ++c) win[(o + 2) % 3][c] = xs[((o + 2) * IW + c) * 4];
        }
        else
        {
#pragma unroll
            for (int a = 0; a < 3; ++a)
#pragma unroll
                for (int c = 0; c < 3; ++c) win[(o + a) % 3][c] = xs[((o * S + a) * IW + c) * 4];
        }
        const int oh = oh0 + sy * R + o;
        const bool ok = col_ok && oh < g.Ho;
        float4 acc = bias;
        if (ACC) { acc = zero; if (ok) acc = dst[(size_t)oh * g.Wo * 4]; }
#pragma unroll
        for (int a = 0; a < 3; ++a)
#pragma unroll
            for (int c = 0; c < 3; ++c)
            {
                const float4 x = win[(o + a) % 3][c];
                const float4 k = w[a * 3 + c];
                acc.x = fmaf(x.x, k.x, acc.x); acc.y = fmaf(x.y, k.y, acc.y);
                acc.z = fmaf(x.z, k.z, acc.z); acc.w = fmaf(x.w, k.w, acc.w);
            }
        if (ACC) { acc.x += bias.x; acc.y += bias.y; acc.z += bias.z; acc.w += bias.w; }
        acc.x = act_bf(acc.x, nscale); acc.y = act_bf(acc.y, nscale);
        acc.z = act_bf(acc.z, nscale); acc.w = act_bf(acc.w, nscale);
        if (ok) dst[(size_t)oh * g.Wo * 4] = acc;
    }
}

// tile shapes of the LDS kernel: (TW, R) -> a TW x (64/TW)*R tile of output pixels
struct TileShape { int tw, th; };
constexpr TileShape TILE_SHAPES_S1[] = {{16, 16}, {8, 28}, {16, 28}, {32, 8}, {8, 8}};
constexpr TileShape TILE_SHAPES_S2[] = {{8, 8}, {4, 16}, {16, 4}};


__global__ __launch_bounds__(TPB) void dw_u8_kernel(const uint32_t *__restrict__ in,
                                                    const uint32_t *__restrict__ filt,
                                                    uint32_t *__restrict__ out, size_t total,
                                                    int cblocks, Geom g, int32_t zi, int32_t zf, QOut qo)
{
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= total) return;
    const int q = (int)(i & 3);
    const PixelPos pp = split_pixel(i >> 2, g.Wo, g.Ho);
    const int ow = pp.ow, oh = pp.oh;
    const size_t plane = pp.plane;
    const int cbk = (int)((uint32_t)plane % (uint32_t)cblocks);   // planes < 2^31 (checked by the launcher)
    const uint32_t *src = in + plane * (size_t)g.H * g.W * 4 + q;
    const uint32_t *f = filt + (size_t)cbk * g.kh * g.kw * 4 + q;
    const int ih0 = oh * g.stride - g.pt, iw0 = ow * g.stride - g.pl;
    uint32_t acc[4] = {0, 0, 0, 0};
    for (int a = 0; a < g.kh; ++a)
    {
        const int ih = ih0 + a;
        if (ih < 0 || ih >= g.H) continue;
        for (int b = 0; b < g.kw; ++b)
        {
            const int iw = iw0 + b;
            if (iw < 0 || iw >= g.W) continue;
            const uint32_t v = src[((size_t)ih * g.W + iw) * 4];
            const uint32_t w = f[(a * g.kw + b) * 4];
#pragma unroll
            for (int c = 0; c < 4; ++c)
                acc[c] += (uint32_t)((int32_t)((v >> (8 * c)) & 0xffu) + zi) *
                          (uint32_t)((int32_t)((w >> (8 * c)) & 0xffu) + zf);
        }
    }
    uint32_t packed = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) packed |= requant_u8((int32_t)acc[c], qo) << (8 * c);
    out[i] = packed;
}

int dw_check(const char *op, int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int C,
             int H, int W, const void *in, const void *filt, const void *out, Geom *g)
{
    // interface_abstract.hpp:1013-1050: channel test first, then stride
    if (C <= 0 || C % CB != 0) return SMALL_HIP_ECHANNELS;
    if (stride != 1 && stride != 2) return SMALL_HIP_ESTRIDE;
    if (batch <= 0 || kh <= 0 || kw <= 0 || H <= 0 || W <= 0 || !pads_ok(pt, pb, pl, pr))
    { set_error("%s: bad size", op); return SMALL_HIP_EINVAL; }
    if (!in || !filt || !out || !aligned16(in) || !aligned16(filt) || !aligned16(out))
    { set_error("%s: null or misaligned pointer", op); return SMALL_HIP_EINVAL; }
    if (in == out) { set_error("%s: in-place convolution is not supported", op); return SMALL_HIP_EINVAL; }
    if ((long)batch * (C / CB) > 0x7fffffffL) { set_error("%s: batch * C / 16 too large", op); return SMALL_HIP_EINVAL; }
    g->H = H; g->W = W; g->kh = kh; g->kw = kw; g->stride = stride; g->pt = pt; g->pl = pl;
    g->stride_h = stride;
    g->Ho = out_dim(H, pt, pb, kh, stride);
    g->Wo = out_dim(W, pl, pr, kw, stride);
    return SMALL_HIP_OK;
}

int dw_f32(const char *op, int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int C, int H,
           int W, const float *in, const float *filt, const float *bias, int act, float slope, int accumulate,
           float *out, small_hip_stream_t stream)
{
    Geom g;
    if (int rc = dw_check(op, batch, kh, kw, stride, pt, pb, pl, pr, C, H, W, in, filt, out, &g)) return rc;
    if (bias && !aligned16(bias)) { set_error("%s: misaligned bias", op); return SMALL_HIP_EINVAL; }
    if (act < SMALL_HIP_ACT_NONE || act > SMALL_HIP_ACT_LEAKY) { set_error("%s: bad activation", op); return SMALL_HIP_EINVAL; }
    const size_t total4 = (size_t)batch * C * g.Ho * g.Wo / 4;
    if (total4 == 0) return SMALL_HIP_OK;
    const Epi e{reinterpret_cast<const float4 *>(bias), act, slope, accumulate};
    if (kh == 3 && kw == 3)
    {
        constexpr int R1 = 4, R2 = 3;      // output rows per lane at stride 1 / stride 2
        static const bool tile_off = tune_int("dw_tile", 1) == 0;
        // measured: the strip kernel wins below 7x7 outputs at stride 1 and below 14x14 at stride 2 (256 channels 28x28 -> 14x14,
        // batch 64: tile kernel 11.4 us, strip kernel 14.0 us; 512 channels 14x14 -> 7x7: 7.0 us either way)
        const int min_side = stride == 1 ? 7 : 14;
        if (g.Ho >= min_side && g.Wo >= min_side && !tile_off)
        {
            // the tile shape that wastes the fewest lanes on this image; ties go to the first
            const TileShape *shapes = stride == 1 ? TILE_SHAPES_S1 : TILE_SHAPES_S2;
            int best = -1;
            double best_util = 0.7;        // below that the strip kernel is the better choice
            const int nshapes = stride == 1 ? 5 : 3;
            for (int t = 0; t < nshapes; ++t)
            {
                const int tx = (g.Wo + shapes[t].tw - 1) / shapes[t].tw;
                const int ty = (g.Ho + shapes[t].th - 1) / shapes[t].th;
                double util = (double)g.Wo * g.Ho / ((double)tx * shapes[t].tw * ty * shapes[t].th);
                // measured corrections: the 8x28 tile leaves one slot row of eight idle but still wins at 56x56
                // (128 channels: 37 us against 46 us for the exact-fit 8x8 tile); the 8x8 tile re-reads 56% of
                // its input as halo and does one row per lane
                if (stride == 1 && t == 1) util *= 0.95;
                if (stride == 1 && t == 4) util *= 0.92;
                if (util > best_util + 1e-9) { best_util = util; best = t; }
            }
            // SMALL_HIP_TUNE key dw_shape: force a shape of the table
            {
                static const int f = tune_int("dw_shape", -1);
                if (f >= 0 && f < nshapes) best = f;
            }
            if (best >= 0)
            {
                const int tiles_x = (g.Wo + shapes[best].tw - 1) / shapes[best].tw;
                const int tiles_y = (g.Ho + shapes[best].th - 1) / shapes[best].th;
                const size_t nb = (size_t)batch * (C / CB) * tiles_x * tiles_y;
                if (nb > 0x7fffffff / 2) { set_error("%s: too many blocks for one launch", op); return SMALL_HIP_EINVAL; }
                const int nblocks = (int)nb;
                const int per_xcd = (nblocks + NUM_XCD - 1) / NUM_XCD;
                decltype(&dw3x3_f32_tile_kernel<1, 16, 4, false>) tk;
#define SHP_DW_TILE(S_, TW_, R_) (accumulate ? dw3x3_f32_tile_kernel<S_, TW_, R_, true> : dw3x3_f32_tile_kernel<S_, TW_, R_, false>)
                if (stride == 1)
                    tk = best == 0 ? SHP_DW_TILE(1, 16, 4)
                       : best == 1 ? (accumulate ? dw3x3_f32_tile_kernel<1, 8, 4, true, 7> : dw3x3_f32_tile_kernel<1, 8, 4, false, 7>)
                       : best == 2 ? SHP_DW_TILE(1, 16, 7) : best == 3 ? SHP_DW_TILE(1, 32, 4) : SHP_DW_TILE(1, 8, 1);
                else
                    tk = best == 0 ? SHP_DW_TILE(2, 8, 1) : best == 1 ? SHP_DW_TILE(2, 4, 1) : SHP_DW_TILE(2, 16, 1);
#undef SHP_DW_TILE
                hipLaunchKernelGGL(tk, dim3(per_xcd * NUM_XCD), dim3(TPB), 0, as_stream(stream),
                                   reinterpret_cast<const float4 *>(in), reinterpret_cast<const float4 *>(filt),
                                   reinterpret_cast<float4 *>(out), C / CB, tiles_x, tiles_y, nblocks, per_xcd, g, e);
                SHP_LAUNCH_CHECK(op);
                return SMALL_HIP_OK;
            }
        }
        const int rows = stride == 1 ? R1 : R2;
        const size_t ncols4 = (size_t)batch * C * g.Wo / 4;
        const int nstrips = (g.Ho + rows - 1) / rows;
        const size_t nb = ((ncols4 + TPB - 1) / TPB) * (size_t)nstrips;
        if (nb > 0x7fffffff / 2) { set_error("%s: too many blocks for one launch", op); return SMALL_HIP_EINVAL; }
        const int nblocks = (int)nb, per_xcd = (nblocks + NUM_XCD - 1) / NUM_XCD;
        auto sk = stride == 1 ? (accumulate ? dw3x3_f32_strip_kernel<1, R1, true> : dw3x3_f32_strip_kernel<1, R1, false>)
                              : (accumulate ? dw3x3_f32_strip_kernel<2, R2, true> : dw3x3_f32_strip_kernel<2, R2, false>);
        hipLaunchKernelGGL(sk, dim3(per_xcd * NUM_XCD), dim3(TPB), 0, as_stream(stream),
                           reinterpret_cast<const float4 *>(in), reinterpret_cast<const float4 *>(filt),
                           reinterpret_cast<float4 *>(out), ncols4, C / CB, nstrips, nblocks, per_xcd, g, e);
        SHP_LAUNCH_CHECK(op);
        return SMALL_HIP_OK;
    }
    const dim3 grid((unsigned)((total4 + TPB - 1) / TPB)), block(TPB);
    auto k = (kh == 3 && kw == 3) ? dw_f32_kernel<3, 3> : dw_f32_kernel<0, 0>;
    hipLaunchKernelGGL(k, grid, block, 0, as_stream(stream), reinterpret_cast<const float4 *>(in),
                       reinterpret_cast<const float4 *>(filt), reinterpret_cast<float4 *>(out), total4,
                       C / CB, g, e);
    SHP_LAUNCH_CHECK(op);
    return SMALL_HIP_OK;
}

} // namespace

extern "C" {

int small_hip_depthwise_conv2d_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                                   int C, int H, int W, const float *in, const float *filt, float *out,
                                   small_hip_stream_t stream)
{
    return dw_f32("small_hip_depthwise_conv2d_f32", batch, kh, kw, stride, pt, pb, pl, pr, C, H, W, in, filt,
                  nullptr, SMALL_HIP_ACT_NONE, 0.f, 0, out, stream);
}

int small_hip_partial_depthwise_conv2d_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl,
                                           int pr, int C, int H, int W, const float *in, const float *filt,
                                           float *out, small_hip_stream_t stream)
{
    return dw_f32("small_hip_partial_depthwise_conv2d_f32", batch, kh, kw, stride, pt, pb, pl, pr, C, H, W, in,
                  filt, nullptr, SMALL_HIP_ACT_NONE, 0.f, 1, out, stream);
}

int small_hip_depthwise_conv2d_bias_act_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl,
                                            int pr, int C, int H, int W, const float *in, const float *filt,
                                            const float *bias, int act, float slope, float *out,
                                            small_hip_stream_t stream)
{
    return dw_f32("small_hip_depthwise_conv2d_bias_act_f32", batch, kh, kw, stride, pt, pb, pl, pr, C, H, W, in,
                  filt, bias, act, slope, 0, out, stream);
}

int small_hip_dense_literal_f32(int No, int Ni, const float *in, const float *filt, float *out,
                                small_hip_stream_t stream)
{
    // interface_abstract.hpp:2113-2132: a 1x1 depthwise over a 1 x Ni image with No channels;
    // no channel-count check there, but the packed layout needs whole blocks
    if (No <= 0 || No % CB != 0) return einval("small_hip_dense_literal_f32: output_elements must be a multiple of 16");
    return dw_f32("small_hip_dense_literal_f32", 1, 1, 1, 1, 0, 0, 0, 0, No, 1, Ni, in, filt, nullptr,
                  SMALL_HIP_ACT_NONE, 0.f, 0, out, stream);
}

int small_hip_depthwise_conv2d_u8(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int C,
                                  int H, int W, const uint8_t *in, const small_hip_quant *iq,
                                  const uint8_t *filt, const small_hip_quant *fq, uint8_t *out,
                                  const small_hip_quant *oq, small_hip_stream_t stream)
{
    const char *op = "small_hip_depthwise_conv2d_u8";
    if (!iq || !fq || !oq) return einval("small_hip_depthwise_conv2d_u8: null quantisation parameters");
    Geom g;
    if (int rc = dw_check(op, batch, kh, kw, stride, pt, pb, pl, pr, C, H, W, in, filt, out, &g)) return rc;
    const size_t total = (size_t)batch * C * g.Ho * g.Wo / 4;
    if (total == 0) return SMALL_HIP_OK;
    const QOut q = make_qout(oq->multiplier, oq->lshift, oq->rshift);
    hipLaunchKernelGGL(dw_u8_kernel, dim3((unsigned)((total + TPB - 1) / TPB)), dim3(TPB), 0, as_stream(stream),
                       reinterpret_cast<const uint32_t *>(in), reinterpret_cast<const uint32_t *>(filt),
                       reinterpret_cast<uint32_t *>(out), total, C / CB, g, iq->zero, fq->zero, q);
    SHP_LAUNCH_CHECK(op);
    return SMALL_HIP_OK;
}

} // extern "C"
