// Conv2D / PartialConv2D / Dense (float32) for gfx950.
//
// input_channels % 16 == 0: implicit GEMM on v_mfma_f32_32x32x2_f32,
//      D[co][px] += sum_k  F[co][k] * I[k][px],   k = (tap, ci)
// MFMA rows are output channels, MFMA columns are output pixels flattened over (image, oh, ow).
// With the packed layouts a K-step of 16 (one input-channel block at one filter tap) needs no
// shuffling at all:
//   - B operand: lane (px = lane%32, half = lane/32) reads 8 consecutive floats of its pixel's
//     64-byte channel block: two 16-byte loads straight from global memory into the register the
//     MFMA consumes.  The two wave halves take channels 0-7 and 8-15, so MFMA number kk of the
//     step contracts channels {kk, 8+kk}; the pairing of k inside an MFMA is free as long as A
//     and B agree.  Padded taps load a block of zeros.
//   - A operand: F[ci = 8*half+kk][co%16] of the channel block's [16 ci][16 co] tile, staged
//     through LDS once per workgroup (conv_lds_tile) or read directly (conv_splitk_tile).
//   - D: a lane holds 4 consecutive output channels of one pixel per register quad, i.e. 16-byte
//     stores into the packed [px][16] output, after accumulate / bias / activation in registers.
// Addresses: tensors of at most 1 GiB (every case that occurs in practice) are read and written through buffer
// resources, so that a K-step and a store need no address arithmetic on the vector ALU, whose instructions cost
// the SIMD's matrix pipe their issue time (BUF template parameter); larger tensors take the flat-address forms.
// A wave owns COT x PXT tiles of 32 x 32; the four waves of a workgroup share the output channel
// group and take consecutive pixel tiles.  Workgroup ids are re-mapped so that all channel groups
// of a pixel range run on one XCD and share its L2.  Kernels:
//   conv_mfma_f32_lds_kernel      every workgroup runs conv_lds_tile
//   conv_mfma_f32_hybrid_kernel   whole rounds of conv_lds_tile + the remainder as split-K tiles
//   conv_mfma_f32_splitk_kernel   small outputs: one 32x32 tile per workgroup, K split over its waves
//
// input_channels in {1,2,3} (first layers): conv_smallci_mfma_f32_kernel (3x3 and 10x4 windows,
// at least 32 output channels) and conv_smallci_f32_kernel (vector ALU, everything else).
#include "common.h"

#include <cstdlib>

using namespace shp;

namespace
{

typedef float floatx16 __attribute__((ext_vector_type(16)));

struct ConvArgs
{
    const float *in;
    const float *filt;
    const float *bias;   // may be null
    float *out;
    int batch, Co, Ci, H, W, Ho, Wo, kh, kw, stride, pt, pl;
    int stride_h;        // vertical stride: `stride`, or 1 for the 1-D layers (the rows are independent signals)
    int act;
    float slope;
    int accumulate;
    // derived
    int P;               // batch * Ho * Wo
    int n_co_groups;     // ceil(Co / (32*COT))
    int n_px_blocks;     // ceil(P / (32*PXT*4))
    int n_blocks;        // n_co_groups * n_px_blocks
    int per_xcd;         // ceil(n_blocks / 8)
    int n_main;          // hybrid kernel: workgroups that run whole tiles (multiple of the CU count)
    // grouped convolution: blockIdx.y walks `slabs` (image, group) slabs of Ci channels that lie in_slab / out_slab
    // floats apart; slab y uses filter block (slab0 + y) % groups.  slabs == 0: an ordinary convolution.
    int slabs, groups, slab0;
    long long in_slab, out_slab, filt_slab;
    // equal-share split of the reduction (conv_mfma_f32_streamk_kernel): the launch's K-steps, tile after tile, are cut into
    // sk_chunks runs of sk_chunk steps; a run that does not cover a whole tile leaves raw accumulators in sk_scratch
    // ([tile][part < sk_parts][SK_PART_FLOATS]) for conv_streamk_fixup_kernel to add up in run order
    int sk_chunk, sk_chunks, sk_parts;
    float *sk_scratch;
    // pixel index -> (image, row, column) without run-time divisions (conv_lds_tile, conv_splitk_tile): by Ho*Wo and Wo, in
    // the pooling form by (Ho/2)*(Wo/2) and Wo/2
    FastDiv fd_plane, fd_row;
};

void set_pixel_divisors(ConvArgs &a, bool pool)
{
    const int Wr = pool ? a.Wo >> 1 : a.Wo, Hr = pool ? a.Ho >> 1 : a.Ho;
    a.fd_plane = make_fast_div((unsigned)(Hr * Wr > 0 ? Hr * Wr : 1));
    a.fd_row = make_fast_div((unsigned)(Wr > 0 ? Wr : 1));
}

// the arguments of this workgroup's slab (uniform per workgroup: three scalar pointer additions)
__device__ __forceinline__ ConvArgs slab_args(ConvArgs a)
{
    if (a.slabs > 0)
    {
        const int y = blockIdx.y;
        a.in += (long long)y * a.in_slab;
        a.out += (long long)y * a.out_slab;
        a.filt += (long long)((a.slab0 + y) % a.groups) * a.filt_slab;
    }
    return a;
}

// 64 bytes of zeros.  A masked tap (padding, a pixel past the end, a step past the last) loads from
// here instead of being zeroed after the load: a select on the loaded value sits in the step that
// issued the load and makes the wave wait for data it only needs a step later.
__device__ __align__(64) float g_zero_block[CB];

__device__ __forceinline__ float act1(float v, int act, float slope)
{
    if (act == SMALL_HIP_ACT_RELU) return v > 0.f ? v : 0.f;
    if (act == SMALL_HIP_ACT_LEAKY) return v > 0.f ? v : v * slope;
    return v;
}

// negative inputs are multiplied by 1 (no activation), 0 (ReLU) or the slope (LeakyReLU): the
// activation without a branch on its kind; "+ 0.f" turns the -0 of x * 0 into the +0 ReLU gives
__device__ __forceinline__ float act_scale(int act, float slope)
{
    return act == SMALL_HIP_ACT_RELU ? 0.f : act == SMALL_HIP_ACT_LEAKY ? slope : 1.f;
}
__device__ __forceinline__ float act_bf(float v, float neg_scale)
{
    const float n = fmaf(v, neg_scale, 0.f);
    return v > 0.f ? v : n;
}
// The same with the kind known at compile time: ReLU is one instruction (a maximum) instead of three, and gives the
// same bits as act_bf(v, 0) for every input that is a number (negative and -0 -> +0).  A vector instruction costs the
// matrix pipe of its SIMD about eight cycles whichever wave issues it, so the epilogues' instruction count is launch time.
template <bool RELU>
__device__ __forceinline__ float act_k(float v, float neg_scale)
{
    return RELU ? fmaxf(v, 0.f) : act_bf(v, neg_scale);
}

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
constexpr unsigned BUF_OUT_OF_RANGE = 0x80000000u;
constexpr long long BUF_MAX_BYTES = 1ll << 30;
constexpr int BUF_RSRC_FLAGS = 0x00020000;            // raw buffer of 32-bit elements
constexpr unsigned BUF_SCALAR_OUT_OF_RANGE = 1u << 30; // a scalar offset that puts every lane out of range (>= BUF_MAX_BYTES)

// accumulate / bias / activation in registers, then 16-byte stores: a lane holds channels
// 8q + 4*half + {0..3} of its pixel in accumulator registers 4q .. 4q+3.  Straight-line code:
// pixels past the end and channels past Co are computed and not stored, the bias is loaded once
// per channel quad, PartialConv2D (ACC) is a compile-time variant.
template <int COT, int PXT, bool ACC, bool RELU>
__device__ __forceinline__ void conv_epilogue_impl(const ConvArgs &a, floatx16 (&acc)[COT][PXT], int cg, int half,
                                                   int HoWo, const bool (&pvalid)[PXT], const size_t (&out_pix)[PXT],
                                                   const float *lds_bias)
{
    const float nscale = act_scale(a.act, a.slope);
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 bb[COT][4];
#pragma unroll
    for (int c = 0; c < COT; ++c)
#pragma unroll
        for (int q = 0; q < 4; ++q) bb[c][q] = zero;
    if (lds_bias)
    {
        // the workgroup's bias values (zeros without a bias or past the last channel), parked in LDS before the K loop
#pragma unroll
        for (int c = 0; c < COT; ++c)
#pragma unroll
            for (int q = 0; q < 4; ++q) bb[c][q] = *reinterpret_cast<const float4 *>(lds_bias + c * 32 + 8 * q + 4 * half);
    }
    else if (a.bias)
    {
#pragma unroll
        for (int c = 0; c < COT; ++c)
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const int co4 = (cg * COT + c) * 32 + 8 * q + 4 * half;
                if (co4 < a.Co) bb[c][q] = *reinterpret_cast<const float4 *>(a.bias + co4);
            }
    }
#pragma unroll
    for (int c = 0; c < COT; ++c)
    {
        const int co_tile = (cg * COT + c) * 32;
#pragma unroll
        for (int t = 0; t < PXT; ++t)
        {
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const int co4 = co_tile + 8 * q + 4 * half;
                const bool ok = pvalid[t] && co4 < a.Co;
                float4 v = make_float4(acc[c][t][4 * q + 0], acc[c][t][4 * q + 1],
                                       acc[c][t][4 * q + 2], acc[c][t][4 * q + 3]);
                float4 *o = reinterpret_cast<float4 *>(a.out + out_pix[t] +
                                                       (size_t)(co4 / CB) * HoWo * CB + (co4 % CB));
                if (ACC)
                {
                    float4 old = zero;
                    if (ok) old = *o;
                    v.x += old.x; v.y += old.y; v.z += old.z; v.w += old.w;
                }
                v.x += bb[c][q].x; v.y += bb[c][q].y; v.z += bb[c][q].z; v.w += bb[c][q].w;
                v.x = act_k<RELU>(v.x, nscale); v.y = act_k<RELU>(v.y, nscale);
                v.z = act_k<RELU>(v.z, nscale); v.w = act_k<RELU>(v.w, nscale);
                if (ok) *o = v;
            }
        }
    }
}

template <int COT, int PXT>
__device__ __forceinline__ void conv_epilogue(const ConvArgs &a, floatx16 (&acc)[COT][PXT], int cg, int half,
                                              int HoWo, const bool (&pvalid)[PXT], const size_t (&out_pix)[PXT],
                                              const float *lds_bias = nullptr)
{
    // the epilogue runs once per workgroup: a uniform branch picks the straight-line variant (ReLU is one instruction
    // per value instead of three, and the epilogue's vector instructions are time the matrix pipe stands still)
    if (a.accumulate) conv_epilogue_impl<COT, PXT, true, false>(a, acc, cg, half, HoWo, pvalid, out_pix, lds_bias);
    else if (a.act == SMALL_HIP_ACT_RELU) conv_epilogue_impl<COT, PXT, false, true>(a, acc, cg, half, HoWo, pvalid, out_pix, lds_bias);
    else conv_epilogue_impl<COT, PXT, false, false>(a, acc, cg, half, HoWo, pvalid, out_pix, lds_bias);
}

// The same through buffer stores (conv_lds_tile's BUF form).  ovoff: the lane's byte offset of (pixel, channel 4 * half of
// channel block 0) in the output tensor, or BUF_OUT_OF_RANGE for a lane that stores nothing; the channel quad's offset
// is wave-uniform, channels past Co get one that is out of range for every lane.  One vector addition per store and no
// predicate: nine vector instructions (offset, bias, activation) per 16-byte store.
// The uniform offset is added to the lane offset and NOT passed as the store's scalar offset: a 16-byte buffer store must
// be followed by a wait state before a vector instruction overwrites its data registers, the compiler inserts that wait
// state only for stores without a scalar-offset register, and this hardware needs it with one as well (seen here: the
// second data register of the one store whose next instruction rewrote it reached memory with the new value in four
// lanes of every sixteen, in some waves).
template <int COT, int PXT, bool ACC, bool RELU>
__device__ __forceinline__ void conv_epilogue_buf_impl(const ConvArgs &a, floatx16 (&acc)[COT][PXT], int cg, int half,
                                                       int HoWo, const unsigned (&ovoff)[PXT], const float *lds_bias)
{
    const float nscale = act_scale(a.act, a.slope);
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        a.out, 0, (int)((size_t)a.batch * a.Co * HoWo * sizeof(float)), BUF_RSRC_FLAGS);
#pragma unroll
    for (int c = 0; c < COT; ++c)
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const int co8 = (cg * COT + c) * 32 + 8 * q;                        // wave-uniform; Co is a multiple of 16
            const unsigned soff = co8 < a.Co ? (unsigned)(((co8 / CB) * HoWo * CB + (co8 % CB)) * (int)sizeof(float))
                                             : BUF_SCALAR_OUT_OF_RANGE;
            const float4 bb = *reinterpret_cast<const float4 *>(lds_bias + c * 32 + 8 * q + 4 * half);
#pragma unroll
            for (int t = 0; t < PXT; ++t)
            {
                float4 v = make_float4(acc[c][t][4 * q + 0], acc[c][t][4 * q + 1], acc[c][t][4 * q + 2], acc[c][t][4 * q + 3]);
                if (ACC)
                {
                    const float4 old = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, ovoff[t], soff, 0));
                    v.x += old.x; v.y += old.y; v.z += old.z; v.w += old.w;
                }
                v.x += bb.x; v.y += bb.y; v.z += bb.z; v.w += bb.w;
                v.x = act_k<RELU>(v.x, nscale); v.y = act_k<RELU>(v.y, nscale);
                v.z = act_k<RELU>(v.z, nscale); v.w = act_k<RELU>(v.w, nscale);
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), rsrc, ovoff[t] + soff, 0, 0);
            }
        }
}

template <int COT, int PXT>
__device__ __forceinline__ void conv_epilogue_buf(const ConvArgs &a, floatx16 (&acc)[COT][PXT], int cg, int half, int HoWo,
                                                  const unsigned (&ovoff)[PXT], const float *lds_bias)
{
    if (a.accumulate) conv_epilogue_buf_impl<COT, PXT, true, false>(a, acc, cg, half, HoWo, ovoff, lds_bias);
    else if (a.act == SMALL_HIP_ACT_RELU) conv_epilogue_buf_impl<COT, PXT, false, true>(a, acc, cg, half, HoWo, ovoff, lds_bias);
    else conv_epilogue_buf_impl<COT, PXT, false, false>(a, acc, cg, half, HoWo, ovoff, lds_bias);
}

// Epilogue with MaxPool2D 2x2 stride 2 (no padding) fused: the wave's 32-pixel tiles are 8 pooling windows of
// four pixels (pool_tile_pixel), so a window is this lane, lane ^ 1 (next column) and lanes ^ 2 (next row): bias
// and activation, two shuffles and maxima per value, and the first lane of each window stores the pooled pixel
// into [N][Co/16][Ho/2][Wo/2][16].
// BUFS: the store goes through a buffer resource (pvoff: the lane's byte offset of (pooled pixel, channel 4 * half of
// channel block 0), or BUF_OUT_OF_RANGE for the three lanes of a window that store nothing), as in conv_epilogue_buf_impl.
template <int COT, int PXT, bool BUFS = false>
__device__ __forceinline__ void conv_epilogue_pool(const ConvArgs &a, floatx16 (&acc)[COT][PXT], int cg, int half,
                                                   const bool (&pool_ok)[PXT], const size_t (&pool_pix)[PXT],
                                                   const float *lds_bias = nullptr, const unsigned *pvoff = nullptr)
{
    const float nscale = act_scale(a.act, a.slope);
    const int HpWp = (a.Ho >> 1) * (a.Wo >> 1);
    __amdgpu_buffer_rsrc_t rsrc;
    if (BUFS) rsrc = __builtin_amdgcn_make_buffer_rsrc(a.out, 0, (int)((size_t)a.batch * a.Co * HpWp * sizeof(float)), BUF_RSRC_FLAGS);
#pragma unroll
    for (int c = 0; c < COT; ++c)
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const int co4 = (cg * COT + c) * 32 + 8 * q + 4 * half;
            float4 bb = make_float4(0.f, 0.f, 0.f, 0.f);
            if (lds_bias) bb = *reinterpret_cast<const float4 *>(lds_bias + c * 32 + 8 * q + 4 * half);
            else if (a.bias && co4 < a.Co) bb = *reinterpret_cast<const float4 *>(a.bias + co4);
            const float b4[4] = {bb.x, bb.y, bb.z, bb.w};
#pragma unroll
            for (int t = 0; t < PXT; ++t)
            {
                float m[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    float v = act_bf(acc[c][t][4 * q + e] + b4[e], nscale);
                    const float u = __shfl_xor(v, 1, WAVE);
                    v = v > u ? v : u;
                    const float w = __shfl_xor(v, 2, WAVE);
                    m[e] = v > w ? v : w;
                }
                if (BUFS)
                {
                    const int co8 = co4 - 4 * half;                              // wave-uniform
                    const unsigned soff = co8 < a.Co ? (unsigned)(((co8 / CB) * HpWp * CB + (co8 % CB)) * (int)sizeof(float))
                                                     : BUF_SCALAR_OUT_OF_RANGE;
                    // (lane offset + uniform offset as the vector offset: see conv_epilogue_buf_impl)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, make_float4(m[0], m[1], m[2], m[3])), rsrc,
                                                           pvoff[t] + soff, 0, 0);
                }
                else if (pool_ok[t] && co4 < a.Co)
                    *reinterpret_cast<float4 *>(a.out + pool_pix[t] + (size_t)(co4 / CB) * HpWp * CB + (co4 % CB)) =
                        make_float4(m[0], m[1], m[2], m[3]);
            }
        }
}

// The pooling form's pixel order: pooling windows (image, pooled row, pooled column) counted straight through, four
// pixels each; lane column `col` = (window of the tile) * 4 + (row in the window) * 2 + (column in the window), a.P = 4 x
// the number of windows.  No slot is lost to ragged patches (a 26x26 map cut into 4 x 8 patches computed 32% more pixels
// than it has), and convolution rows / columns that no window covers (odd extents) are not computed at all.  pool_ok:
// this lane stores the pooled pixel of its window at pool_pix (element offset of channel 0 of channel block 0 in
// [N][Co/16][Ho/2][Wo/2][16]).
__device__ __forceinline__ void pool_tile_pixel(const ConvArgs &a, const int tile, const int col, int &n, int &oh, int &ow,
                                                bool &pvalid, bool &pool_ok, size_t &pool_pix)
{
    const int Wp = a.Wo >> 1, HpWp = (a.Ho >> 1) * Wp;
    const int p = tile * 32 + col;
    pvalid = p < a.P;
    const int w = pvalid ? p >> 2 : 0;
    n = fast_div(w, a.fd_plane);
    const int r = w - n * HpWp;
    const int ph = fast_div(r, a.fd_row), pw = r - ph * Wp;
    oh = 2 * ph + ((col >> 1) & 1);
    ow = 2 * pw + (col & 1);
    pool_ok = pvalid && (col & 3) == 0;
    pool_pix = ((size_t)n * (a.Co / CB) * HpWp + r) * CB;
}

// ---------------------------------------------------------------------------------------------
// The main kernel body: filter operand staged through LDS.  The four waves of a workgroup
// multiply the same output-channel group, so the step's [16 ci][16 co] filter tiles (COT*2 KiB)
// are fetched once per workgroup with fully coalesced 16-byte loads, written to LDS (double
// buffered, one barrier per K-step) and read back by every wave in MFMA operand order: a quarter
// of the vector-cache accesses of per-wave filter reads, and one 16-byte load per lane instead
// of 8 strided dword loads per tile.  The activation operand goes straight from global memory to
// the MFMA register, two 16-byte loads per lane and tile.
constexpr int A_TILE_FLOATS = 272;   // 256 + 16 pad: consecutive channel blocks start 16 banks apart

// s_begin / s_count: only K-steps [s_begin, s_begin + s_count) of the tile (s_count < 0: all of them); raw != nullptr: the
// accumulators go there as they are ([wave][tile of the wave][register quad][lane] float4) instead of through the epilogue
// PW: a pointwise convolution (1x1 window, stride 1, no padding): the activation operand of a lane is its own pixel's
// channel vector, channel block after channel block, so a K-step needs one address instruction per pixel tile where the
// general form needs about ten (window position, bounds, select).  Every vector instruction between the MFMAs takes an
// issue slot of the SIMD away from them (measured on a loop of this shape: 12 vector instructions per 16 MFMAs = 4%).
// BLDS: the workgroup runs this body once; its bias values are requested first of all and parked in LDS under the K loop, so
// the epilogue does not wait for memory once more (a caller that runs several tiles per workgroup would overwrite them
// while another wave still reads)
// BUF: both operand streams come through buffer loads (a resource descriptor per tensor, a 32-bit byte offset per lane, the
// channel block's offset in a scalar register).  A tap outside the image, a pixel past the end and a step past the last
// are then an offset the hardware finds out of range and answers with zeros, and a lane's offsets change only when the
// window position does (once in Ci/16 steps): a K-step issues no vector-ALU instruction for its addresses.  The
// launcher allows it for tensors of at most 1 GiB (lane offset + scalar offset + 16 stays below 2^31 on either side of
// the range check, whether or not the hardware adds the scalar offset before it checks).

template <int COT, int PXT, bool POOL = false, bool PW = false, bool BLDS = false, bool BUF = false>
__device__ __forceinline__ void conv_lds_tile(const ConvArgs &a, float (&lds_a)[2][COT * 2 * A_TILE_FLOATS],
                                              const int cg, const int pxb, const int s_begin = 0, const int s_count = -1,
                                              float *raw = nullptr)
{
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int col = lane & 31;
    const int half = lane >> 5;
    __shared__ __align__(16) float s_bias[BLDS ? COT * 32 : 4];
    float my_bias = 0.f;
    if (BLDS && tid < COT * 32)
    {
        const int co = cg * COT * 32 + tid;
        if (a.bias && co < a.Co) my_bias = a.bias[co];
    }

    const int HoWo = a.Ho * a.Wo;
    const int CiB = a.Ci / CB;
    const int CoB = a.Co / CB;
    const int taps = a.kh * a.kw;
    const size_t in_blk = (size_t)a.H * a.W * CB;
    const float *zero_half = g_zero_block + half * 8;

    const float *in_img[PXT];
    unsigned lane_base[PXT];     // BUF: byte offset of (image, channel half) in the input tensor
    unsigned ovoff[PXT];         // BUF: byte offset of (output pixel, channel 4 * half) in the output tensor, or out of range
    int ih0[PXT], iw0[PXT];
    bool pvalid[PXT];
    size_t out_pix[PXT];
    bool pool_ok[PXT];           // POOL: this lane stores the pooled pixel of its window
#pragma unroll
    for (int t = 0; t < PXT; ++t)
    {
        int n, oh, ow, rem;
        if (POOL)
            pool_tile_pixel(a, (pxb * 4 + wave) * PXT + t, col, n, oh, ow, pvalid[t], pool_ok[t], out_pix[t]);
        else
        {
            const int p = ((pxb * 4 + wave) * PXT + t) * 32 + col;
            pvalid[t] = p < a.P;
            const int pc = pvalid[t] ? p : 0;
            n = fast_div(pc, a.fd_plane);
            rem = pc - n * HoWo;
            oh = fast_div(rem, a.fd_row);
            ow = rem - oh * a.Wo;
            pool_ok[t] = false;
            out_pix[t] = ((size_t)n * CoB * HoWo + rem) * CB;
        }
        ih0[t] = oh * a.stride_h - a.pt;
        iw0[t] = ow * a.stride - a.pl;
        in_img[t] = a.in + (size_t)n * CiB * in_blk + half * 8;
        lane_base[t] = (unsigned)(((size_t)n * CiB * in_blk + half * 8) * sizeof(float));
        ovoff[t] = (POOL ? pool_ok[t] : pvalid[t]) ? (unsigned)((out_pix[t] + 4 * half) * sizeof(float)) : BUF_OUT_OF_RANGE;
        // PW: the pixel's own position (a pixel past the end reads pixel 0 of image 0 and stores nothing)
        if (PW) in_img[t] += (size_t)(oh * a.W + ow) * CB;
    }

    // ---- cooperative filter fetch: COT*2 tiles of 64 float4 each -----------------------------
    constexpr int A_VECS = COT * 2 * 64;                 // float4 per step and workgroup
    constexpr int A_PER_THREAD = (A_VECS + 255) / 256;   // 1 for COT <= 2, 2 for COT == 4
    // Every thread loads and stores (no predicate): with fewer vectors than threads (COT == 1) the
    // upper threads repeat a lower thread's vector and write the same value to the same place.  A
    // predicated load would put the wait of the staging store inside a branch, and the compiler
    // would then have to wait at the top of the loop for loads issued only a step earlier.
    static_assert(A_VECS >= 256 ? A_VECS % 256 == 0 : 256 % A_VECS == 0, "filter vectors vs workgroup size");
    const float *a_src[A_PER_THREAD];
    unsigned a_voff[A_PER_THREAD];
    int a_dst[A_PER_THREAD];
#pragma unroll
    for (int j = 0; j < A_PER_THREAD; ++j)
    {
        const int vc = (tid + j * 256) % A_VECS;
        const int blk = vc >> 6, within = vc & 63;
        int cob = cg * COT * 2 + blk;
        cob = cob < CoB ? cob : CoB - 1;                  // rows past Co: garbage, never stored
        a_src[j] = a.filt + (size_t)cob * CiB * taps * (CB * CB) + within * 4;
        a_voff[j] = (unsigned)(((size_t)cob * CiB * taps * (CB * CB) + within * 4) * sizeof(float));
        a_dst[j] = blk * A_TILE_FLOATS + within * 4;
    }
    // read position of this lane inside a staged tile pair
    int a_rd[COT];
#pragma unroll
    for (int c = 0; c < COT; ++c) a_rd[c] = (c * 2 + (col >> 4)) * A_TILE_FLOATS + half * 8 * CB + (col & 15);

    floatx16 acc[COT][PXT];
#pragma unroll
    for (int c = 0; c < COT; ++c)
#pragma unroll
        for (int t = 0; t < PXT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[c][t][r] = 0.f;

    // first step: channel block fastest, then the window column, then the row
    const int tap0 = s_begin / CiB;
    int cib = s_begin - tap0 * CiB, ta = tap0 / a.kw, tb = tap0 - (tap0 / a.kw) * a.kw;
    const int nsteps = s_count < 0 ? taps * CiB : s_count;
    bool live = true;

    // issues the global loads of the step at (ta, tb, cib) and advances the position
    // Straight-line on purpose (selects, no branches; 32-bit element offsets inside an image, which the
    // launcher guarantees fit): a K-step is then one basic block and the compiler can slot this
    // address arithmetic between the MFMAs instead of running it after them.
    const int in_blk32 = a.H * a.W * CB;
    // BUF: the window position's lane offsets, recomputed only when the position moves
    unsigned voff[PXT];
    auto tap_offsets = [&]() {
#pragma unroll
        for (int t = 0; t < PXT; ++t)
        {
            const int ih = ih0[t] + ta, iw = iw0[t] + tb;
            const bool ok = live && pvalid[t] && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
            voff[t] = ok ? lane_base[t] + (unsigned)((ih * a.W + iw) * (CB * (int)sizeof(float))) : BUF_OUT_OF_RANGE;
        }
    };
    __amdgpu_buffer_rsrc_t rsrc_in, rsrc_f;
    if (BUF)
    {
        rsrc_in = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a.in), 0,
                                                    (int)((size_t)a.batch * a.Ci * a.H * a.W * sizeof(float)), 0x00020000);
        rsrc_f = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a.filt), 0,
                                                   (int)((size_t)CoB * CiB * taps * (CB * CB) * sizeof(float)), 0x00020000);
        tap_offsets();
    }
    auto fetch = [&](float4 (&Areg)[A_PER_THREAD], float4 (&B)[PXT][2]) {
        if (BUF)
        {
            const int soff_a = (cib * taps + ta * a.kw + tb) * (CB * CB * (int)sizeof(float));
#pragma unroll
            for (int j = 0; j < A_PER_THREAD; ++j)
                Areg[j] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_f, a_voff[j], soff_a, 0));
            const int soff_b = cib * (in_blk32 * (int)sizeof(float));
#pragma unroll
            for (int t = 0; t < PXT; ++t)
            {
                B[t][0] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_in, voff[t], soff_b, 0));
                B[t][1] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_in, voff[t] + 16, soff_b, 0));
            }
            // next (tap, channel block); the wave-uniform branch is taken once in Ci/16 steps.  Past the last step the
            // position stays and the lanes' offsets go out of range (zeros that are staged and never multiplied)
            if (++cib == CiB)
            {
                cib = 0;
                if (++tb == a.kw)
                {
                    tb = 0;
                    ++ta;
                }
                if (ta >= a.kh)
                {
                    ta = a.kh - 1;
                    tb = a.kw - 1;
                    cib = CiB - 1;
                    live = false;
                }
                tap_offsets();
            }
            return;
        }
        if (PW)
        {
            const int woff = cib * (CB * CB);
#pragma unroll
            for (int j = 0; j < A_PER_THREAD; ++j) Areg[j] = *reinterpret_cast<const float4 *>(a_src[j] + woff);
            const int cib_off = cib * in_blk32;              // wave-uniform
#pragma unroll
            for (int t = 0; t < PXT; ++t)
            {
                const float4 *p = reinterpret_cast<const float4 *>(in_img[t] + cib_off);
                B[t][0] = p[0];
                B[t][1] = p[1];
            }
            cib = cib + 1 < CiB ? cib + 1 : cib;             // the two fetches past the last step repeat it
            return;
        }
        const int tap = ta * a.kw + tb;
        // filter first: its staging store is the first consumer, so it can wait for these loads
        // alone and leave the activation loads of the same step in flight
        const int woff = (cib * taps + tap) * (CB * CB);
#pragma unroll
        for (int j = 0; j < A_PER_THREAD; ++j) Areg[j] = *reinterpret_cast<const float4 *>(a_src[j] + woff);
        const int cib_off = cib * in_blk32;
#pragma unroll
        for (int t = 0; t < PXT; ++t)
        {
            const int ih = ih0[t] + ta, iw = iw0[t] + tb;
            const bool ok = live && pvalid[t] && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
            const int off = cib_off + (ih * a.W + iw) * CB;
            const float *pp = in_img[t] + off;
            const float4 *p = reinterpret_cast<const float4 *>(ok ? pp : zero_half);
            B[t][0] = p[0];
            B[t][1] = p[1];
        }
        // next (tap, channel block): channel block fastest, then the window column, then the row
        const bool w1 = cib + 1 == CiB;
        const int ncib = w1 ? 0 : cib + 1;
        const bool w2 = w1 && tb + 1 == a.kw;
        const int ntb = w2 ? 0 : tb + (w1 ? 1 : 0);
        const int nta = ta + (w2 ? 1 : 0);
        const bool more = nta < a.kh;
        cib = more ? ncib : cib;
        tb = more ? ntb : tb;
        ta = more ? nta : ta;
        live = live && more;
    };
    auto stage = [&](int buf, const float4 (&Areg)[A_PER_THREAD]) {
#pragma unroll
        for (int j = 0; j < A_PER_THREAD; ++j) *reinterpret_cast<float4 *>(&lds_a[buf][a_dst[j]]) = Areg[j];
    };
    auto multiply = [&](int buf, const float4 (&B)[PXT][2]) {
        float A[COT][8];
#pragma unroll
        for (int c = 0; c < COT; ++c)
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) A[c][kk] = lds_a[buf][a_rd[c] + kk * CB];
#pragma unroll
        for (int kk = 0; kk < 8; ++kk)
#pragma unroll
            for (int t = 0; t < PXT; ++t)
            {
                const float4 bv = B[t][kk >> 2];
                const float b = (kk & 3) == 0 ? bv.x : (kk & 3) == 1 ? bv.y : (kk & 3) == 2 ? bv.z : bv.w;
#pragma unroll
                for (int c = 0; c < COT; ++c)
                    acc[c][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(A[c][kk], b, acc[c][t], 0, 0, 0);
            }
    };

    // Schedule per step s:  multiply(s) | stage filter(s+1) into the other LDS buffer | fetch(s+2)
    // | barrier.  The loads of a step are issued a whole step before they are consumed.
    float4 Areg[A_PER_THREAD];
    float4 B0[PXT][2], B1[PXT][2];
    fetch(Areg, B0);                 // step 0
    stage(0, Areg);
    if (BLDS && tid < COT * 32) s_bias[tid] = my_bias;      // requested before the filter, so it is here by now
    fetch(Areg, B1);                 // step 1
    __syncthreads();
    const int npairs = nsteps >> 1;
    for (int it = 0; it < npairs; ++it)
    {
        multiply(0, B0);             // step 2*it
        stage(1, Areg);              // filter of step 2*it + 1
        fetch(Areg, B0);             // step 2*it + 2
        __syncthreads();
        multiply(1, B1);             // step 2*it + 1
        stage(0, Areg);              // filter of step 2*it + 2
        fetch(Areg, B1);             // step 2*it + 3
        __syncthreads();
    }
    // an odd step count leaves the last step staged in buffer 0 / B0 (the loop's invariant)
    if (nsteps & 1) multiply(0, B0);

    if (raw)
    {
        float4 *r4 = reinterpret_cast<float4 *>(raw) + (size_t)wave * (COT * PXT * 4 * WAVE) + lane;
#pragma unroll
        for (int c = 0; c < COT; ++c)
#pragma unroll
            for (int t = 0; t < PXT; ++t)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    r4[((c * PXT + t) * 4 + q) * WAVE] = make_float4(acc[c][t][4 * q], acc[c][t][4 * q + 1], acc[c][t][4 * q + 2], acc[c][t][4 * q + 3]);
        return;
    }
    if (BUF && BLDS)
    {
        if (POOL) conv_epilogue_pool<COT, PXT, true>(a, acc, cg, half, pool_ok, out_pix, s_bias, ovoff);
        else conv_epilogue_buf<COT, PXT>(a, acc, cg, half, HoWo, ovoff, s_bias);
        return;
    }
    if (POOL) conv_epilogue_pool<COT, PXT>(a, acc, cg, half, pool_ok, out_pix, BLDS ? s_bias : nullptr);
    else conv_epilogue<COT, PXT>(a, acc, cg, half, HoWo, pvalid, out_pix, BLDS ? s_bias : nullptr);
}

// The second launch bound (minimum waves per SIMD: 6 / 5 / 2 for one / two / four MFMA tiles per
// wave) makes the compiler keep the accumulators in the unified register file and pack tighter
// (2x1: 108 -> 76 registers, 2x2: 184 -> 131, no spills); measured 1-3% faster, tighter bounds spill.
template <int COT, int PXT, bool POOL = false, bool PW = false, bool BUF = false>
__global__ __launch_bounds__(256, (COT * PXT == 2 ? 5 : COT * PXT == 1 ? 6 : 2)) void conv_mfma_f32_lds_kernel(const ConvArgs a0)
{
    const ConvArgs a = slab_args(a0);
    __shared__ float lds_a[2][COT * 2 * A_TILE_FLOATS];
    const int bid = blockIdx.x;
    const int lid = (bid % NUM_XCD) * a.per_xcd + bid / NUM_XCD;
    if (lid >= a.n_blocks) return;            // whole workgroup leaves together: no barrier is skipped
    conv_lds_tile<COT, PXT, POOL, PW, true, BUF>(a, lds_a, lid % a.n_co_groups, lid / a.n_co_groups);
}

// ---------------------------------------------------------------------------------------------
// Small outputs (few 32x32 tiles per SIMD: fully connected layers, 7x7 / 13x13 feature maps,
// batch 1): the four waves of a workgroup take the SAME output tile and one quarter of the K-steps
// each, then waves 1..3 hand their partial accumulators to wave 0 through LDS, which adds them in
// the fixed order 0+1+2+3 (deterministic) and runs the epilogue.  Operands go straight from global
// memory to the MFMA registers (nothing is shared between the waves until the reduction).
// POOL: the 32-pixel tiles are the pooling form's groups of 8 windows and the epilogue pools (pool_tile_pixel)
// BUF: operands through buffer loads, as in conv_lds_tile (each wave has its own K range, so its window position and
// scalar offsets are the wave's)
template <int COT, int PXT, bool POOL = false, bool BUF = false>
__device__ __forceinline__ void conv_splitk_tile(const ConvArgs &a, float (&red)[3][COT * PXT][16][64],
                                                 const int cg, const int pxb)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col = lane & 31;
    const int half = lane >> 5;

    const int HoWo = a.Ho * a.Wo;
    const int CiB = a.Ci / CB;
    const int CoB = a.Co / CB;
    const int taps = a.kh * a.kw;
    const size_t in_blk = (size_t)a.H * a.W * CB;
    const float *zero_half = g_zero_block + half * 8;

    const float *in_img[PXT];
    unsigned lane_base[PXT];     // BUF: byte offset of (image, channel half) in the input tensor
    int ih0[PXT], iw0[PXT];
    bool pvalid[PXT];
    size_t out_pix[PXT];
    bool pool_ok[PXT];
#pragma unroll
    for (int t = 0; t < PXT; ++t)
    {
        int n, oh, ow, rem;
        if (POOL)
            pool_tile_pixel(a, pxb * PXT + t, col, n, oh, ow, pvalid[t], pool_ok[t], out_pix[t]);
        else
        {
            const int p = (pxb * PXT + t) * 32 + col;
            pvalid[t] = p < a.P;
            const int pc = pvalid[t] ? p : 0;
            n = fast_div(pc, a.fd_plane);
            rem = pc - n * HoWo;
            oh = fast_div(rem, a.fd_row);
            ow = rem - oh * a.Wo;
            pool_ok[t] = false;
            out_pix[t] = ((size_t)n * CoB * HoWo + rem) * CB;
        }
        ih0[t] = oh * a.stride_h - a.pt;
        iw0[t] = ow * a.stride - a.pl;
        in_img[t] = a.in + (size_t)n * CiB * in_blk + half * 8;
        lane_base[t] = (unsigned)(((size_t)n * CiB * in_blk + half * 8) * sizeof(float));
    }
    const float *w_row[COT];
    unsigned w_voff[COT];        // BUF: byte offset of this lane's filter row in the filter tensor
#pragma unroll
    for (int c = 0; c < COT; ++c)
    {
        const int co = (cg * COT + c) * 32 + col;
        const int cc = co < a.Co ? co : a.Co - 1;
        w_row[c] = a.filt + (size_t)(cc / CB) * CiB * taps * (CB * CB) + (cc % CB) + half * 8 * CB;
        w_voff[c] = (unsigned)(((size_t)(cc / CB) * CiB * taps * (CB * CB) + (cc % CB) + half * 8 * CB) * sizeof(float));
    }

    floatx16 acc[COT][PXT];
#pragma unroll
    for (int c = 0; c < COT; ++c)
#pragma unroll
        for (int t = 0; t < PXT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[c][t][r] = 0.f;

    // this wave's K range: steps [s_lo, s_hi) of the (tap outer, channel block inner) order
    const int nsteps = taps * CiB;
    const int per = (nsteps + 3) >> 2;
    const int s_lo = wave * per;
    const int s_hi = (s_lo + per < nsteps) ? s_lo + per : nsteps;
    const int mine = s_hi > s_lo ? s_hi - s_lo : 0;
    int tap0 = (s_lo < nsteps ? s_lo : 0) / CiB;
    int cib = (s_lo < nsteps ? s_lo : 0) - tap0 * CiB;
    int ta = tap0 / a.kw, tb = tap0 - (tap0 / a.kw) * a.kw;
    int left = mine;                 // steps still to be loaded

    // BUF: the window position's lane offsets (out of range for a masked tap, and for every lane once the wave's steps
    // have all been requested)
    const int in_blk32 = a.H * a.W * CB;
    unsigned voff[PXT];
    auto tap_offsets = [&]() {
#pragma unroll
        for (int t = 0; t < PXT; ++t)
        {
            const int ih = ih0[t] + ta, iw = iw0[t] + tb;
            const bool ok = left > 0 && pvalid[t] && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
            voff[t] = ok ? lane_base[t] + (unsigned)((ih * a.W + iw) * (CB * (int)sizeof(float))) : BUF_OUT_OF_RANGE;
        }
    };
    __amdgpu_buffer_rsrc_t rsrc_in, rsrc_f;
    if (BUF)
    {
        rsrc_in = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a.in), 0,
                                                    (int)((size_t)a.batch * a.Ci * a.H * a.W * sizeof(float)), BUF_RSRC_FLAGS);
        rsrc_f = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a.filt), 0,
                                                   (int)((size_t)CoB * CiB * taps * (CB * CB) * sizeof(float)), BUF_RSRC_FLAGS);
        tap_offsets();
    }
    auto load_step = [&](float (&A)[COT][8], float4 (&B)[PXT][2]) {
        if (BUF)
        {
            const int soff_b = cib * (in_blk32 * (int)sizeof(float));
#pragma unroll
            for (int t = 0; t < PXT; ++t)
            {
                B[t][0] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_in, voff[t], soff_b, 0));
                B[t][1] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_in, voff[t] + 16, soff_b, 0));
            }
            const int soff_a = (cib * taps + ta * a.kw + tb) * (CB * CB * (int)sizeof(float));
#pragma unroll
            for (int c = 0; c < COT; ++c)
#pragma unroll
                for (int kk = 0; kk < 8; ++kk)
                    A[c][kk] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                             rsrc_f, w_voff[c] + kk * (CB * (int)sizeof(float)), soff_a, 0));
            --left;
            if (left <= 0) tap_offsets();          // nothing more to request: every lane out of range
            else if (++cib == CiB)                 // the next window position (wave-uniform, once in Ci/16 steps)
            {
                cib = 0;
                if (++tb == a.kw) { tb = 0; ++ta; }
                tap_offsets();
            }
            return;
        }
        const bool live = left > 0;
        const int tap = ta * a.kw + tb;
#pragma unroll
        for (int t = 0; t < PXT; ++t)
        {
            const int ih = ih0[t] + ta, iw = iw0[t] + tb;
            const bool ok = live && pvalid[t] && ih >= 0 && ih < a.H && iw >= 0 && iw < a.W;
            const size_t off = (size_t)cib * in_blk + ((size_t)ih * a.W + iw) * CB;
            const float4 *p = reinterpret_cast<const float4 *>(ok ? in_img[t] + off : zero_half);
            B[t][0] = p[0];
            B[t][1] = p[1];
        }
#pragma unroll
        for (int c = 0; c < COT; ++c)
        {
            const float *w = w_row[c] + ((size_t)cib * taps + tap) * (CB * CB);
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) A[c][kk] = w[kk * CB];
        }
        if (left > 1)                // stay on a valid position after the last step
        {
            if (++cib == CiB)
            {
                cib = 0;
                if (++tb == a.kw) { tb = 0; ++ta; }
            }
        }
        --left;
    };
    auto compute_step = [&](const float (&A)[COT][8], const float4 (&B)[PXT][2]) {
#pragma unroll
        for (int kk = 0; kk < 8; ++kk)
#pragma unroll
            for (int t = 0; t < PXT; ++t)
            {
                const float4 bv = B[t][kk >> 2];
                const float b = (kk & 3) == 0 ? bv.x : (kk & 3) == 1 ? bv.y : (kk & 3) == 2 ? bv.z : bv.w;
#pragma unroll
                for (int c = 0; c < COT; ++c)
                    acc[c][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(A[c][kk], b, acc[c][t], 0, 0, 0);
            }
    };

    float A0[COT][8], A1[COT][8];
    float4 B0[PXT][2], B1[PXT][2];
    load_step(A0, B0);
    const int npairs = (per + 1) >> 1;           // uniform over the workgroup
    for (int it = 0; it < npairs; ++it)
    {
        load_step(A1, B1);
        compute_step(A0, B0);
        load_step(A0, B0);
        compute_step(A1, B1);
    }

    // ---- reduction over the four K quarters --------------------------------------------------
    if (wave > 0)
    {
#pragma unroll
        for (int c = 0; c < COT; ++c)
#pragma unroll
            for (int t = 0; t < PXT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) red[wave - 1][c * PXT + t][r][lane] = acc[c][t][r];
    }
    __syncthreads();
    if (wave == 0)
    {
#pragma unroll
        for (int w = 0; w < 3; ++w)
#pragma unroll
            for (int c = 0; c < COT; ++c)
#pragma unroll
                for (int t = 0; t < PXT; ++t)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[c][t][r] += red[w][c * PXT + t][r][lane];
        if (POOL) conv_epilogue_pool<COT, PXT>(a, acc, cg, half, pool_ok, out_pix);
        else conv_epilogue<COT, PXT>(a, acc, cg, half, HoWo, pvalid, out_pix);
    }
}

template <int COT, int PXT, bool BUF = false>
__global__ __launch_bounds__(256) void conv_mfma_f32_splitk_kernel(const ConvArgs a0)
{
    const ConvArgs a = slab_args(a0);
    __shared__ float red[3][COT * PXT][16][64];
    const int bid = blockIdx.x;
    const int lid = (bid % NUM_XCD) * a.per_xcd + bid / NUM_XCD;
    if (lid >= a.n_blocks) return;
    conv_splitk_tile<COT, PXT, false, BUF>(a, red, lid % a.n_co_groups, lid / a.n_co_groups);
}

// ---------------------------------------------------------------------------------------------
// Whole rounds + balanced tail in one launch.  The MFMA pipes are the bound, so a launch whose
// workgroup count is not a multiple of the CU count ends with a round in which a few CUs work and
// the rest idle for a whole workgroup time.  Here the first n_main workgroups (a multiple of the
// CU count) run the LDS-staged kernel on their COT x (4*PXT) tiles; what is left over is cut into
// single 32x32 tiles, each multiplied by one workgroup whose four waves split the reduction, i.e.
// 4*COT*PXT times as many workgroups that each last 1/(4*COT*PXT) as long and spread over every CU.
// The hardware starts workgroups in block-id order, so the tail follows the whole rounds.
template <int COT, int PXT, bool POOL = false, bool PW = false, bool BUF = false>
__global__ __launch_bounds__(256, (COT * PXT == 2 ? 5 : COT * PXT == 1 ? 6 : 2)) void conv_mfma_f32_hybrid_kernel(const ConvArgs a0)
{
    const ConvArgs a = slab_args(a0);
    __shared__ float lds_a[2][COT * 2 * A_TILE_FLOATS];
    __shared__ float red[3][1][16][64];
    const int bid = blockIdx.x;
    if (bid < a.n_main)
    {
        // n_main is a multiple of NUM_XCD: consecutive logical ids share an XCD
        const int lid = (bid % NUM_XCD) * (a.n_main / NUM_XCD) + bid / NUM_XCD;
        conv_lds_tile<COT, PXT, POOL, PW, true, BUF>(a, lds_a, lid % a.n_co_groups, lid / a.n_co_groups);
        return;
    }
    constexpr int SUB = 4 * COT * PXT;            // 32x32 tiles per whole workgroup tile
    const int j = bid - a.n_main;
    const int lid = a.n_main + j / SUB;
    if (lid >= a.n_blocks) return;
    const int sub = j % SUB;
    const int co32 = (lid % a.n_co_groups) * COT + sub % COT;
    const int px32 = (lid / a.n_co_groups) * (4 * PXT) + sub / COT;
    if (co32 * 32 >= a.Co || px32 * 32 >= a.P) return;     // uniform over the workgroup
    conv_splitk_tile<1, 1, POOL, BUF>(a, red, co32, px32);
}

// ---------------------------------------------------------------------------------------------
// Equal shares of the reduction for launches with few tiles and a long reduction (3x3 convolutions with 512 / 1024
// channels on a 13x13 map: 352 workgroup tiles for 256 compute units, 288 or 576 K-steps each).  Whole tiles leave a
// second round in which a third of the machine works; cutting only the left-over tiles four ways (the hybrid kernel) leaves
// the first round with one wave per SIMD.  Here all K-steps of the launch, tile after tile, are cut into 3 x 256 equal runs;
// a workgroup multiplies its run (the end of one tile and the start of the next, as a rule) with the LDS-staged body, three
// workgroups per compute unit, all finishing together.  A run that is not a whole tile leaves its raw accumulators in a
// scratch block; conv_streamk_fixup_kernel adds the runs of a tile in run order (deterministic) and applies
// accumulate / bias / activation.
template <int COT, int PXT>
constexpr int sk_part_floats() { return 4 * COT * PXT * 16 * WAVE; }

template <int COT, int PXT, bool BUF = false>
__global__ __launch_bounds__(256, (COT * PXT == 2 ? 5 : COT * PXT == 1 ? 6 : 2)) void conv_mfma_f32_streamk_kernel(const ConvArgs a)
{
    __shared__ float lds_a[2][COT * 2 * A_TILE_FLOATS];
    const int bid = blockIdx.x;
    const int lid = (bid % NUM_XCD) * a.per_xcd + bid / NUM_XCD;      // consecutive runs (the same tiles) on one XCD
    if (lid >= a.sk_chunks) return;
    const int nsteps = a.kh * a.kw * (a.Ci / CB);
    const long total = (long)a.n_blocks * nsteps;
    long k0 = (long)lid * a.sk_chunk;
    const long k1 = k0 + a.sk_chunk < total ? k0 + a.sk_chunk : total;
    while (k0 < k1)                                                   // uniform over the workgroup
    {
        const int tile = (int)(k0 / nsteps);
        const int sb = (int)(k0 - (long)tile * nsteps);
        const int cnt = (int)(nsteps - sb < k1 - k0 ? nsteps - sb : k1 - k0);
        float *raw = nullptr;
        if (cnt != nsteps)
        {
            const int first = (int)(((long)tile * nsteps) / a.sk_chunk);          // the run that starts the tile
            raw = a.sk_scratch + ((size_t)tile * a.sk_parts + (lid - first)) * sk_part_floats<COT, PXT>();
        }
        conv_lds_tile<COT, PXT, false, false, false, BUF>(a, lds_a, tile % a.n_co_groups, tile / a.n_co_groups, sb, cnt, raw);
        k0 += cnt;
        __syncthreads();                                              // the next tile stages into the same LDS buffers
    }
}

template <int COT, int PXT>
__global__ __launch_bounds__(256) void conv_streamk_fixup_kernel(const ConvArgs a)
{
    const int tile = blockIdx.x;
    const int nsteps = a.kh * a.kw * (a.Ci / CB);
    const int first = (int)(((long)tile * nsteps) / a.sk_chunk);
    const int last = (int)(((long)(tile + 1) * nsteps - 1) / a.sk_chunk);
    if (last == first) return;                  // one run covered the whole tile and wrote it through the epilogue
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 31, half = lane >> 5;
    const int cg = tile % a.n_co_groups, pxb = tile / a.n_co_groups;
    const int HoWo = a.Ho * a.Wo, CoB = a.Co / CB;
    bool pvalid[PXT];
    size_t out_pix[PXT];
#pragma unroll
    for (int t = 0; t < PXT; ++t)
    {
        const int p = ((pxb * 4 + wave) * PXT + t) * 32 + col;
        pvalid[t] = p < a.P;
        const int pc = pvalid[t] ? p : 0;
        const int n = pc / HoWo, rem = pc - n * HoWo;
        out_pix[t] = ((size_t)n * CoB * HoWo + rem) * CB;
    }
    floatx16 acc[COT][PXT];
    const float4 *r4 = reinterpret_cast<const float4 *>(a.sk_scratch + (size_t)tile * a.sk_parts * sk_part_floats<COT, PXT>()) +
                       (size_t)wave * (COT * PXT * 4 * WAVE) + lane;
    for (int part = 0; part <= last - first; ++part)
    {
#pragma unroll
        for (int c = 0; c < COT; ++c)
#pragma unroll
            for (int t = 0; t < PXT; ++t)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                {
                    const float4 v = r4[((c * PXT + t) * 4 + q) * WAVE];
                    if (part == 0) { acc[c][t][4 * q] = v.x; acc[c][t][4 * q + 1] = v.y; acc[c][t][4 * q + 2] = v.z; acc[c][t][4 * q + 3] = v.w; }
                    else { acc[c][t][4 * q] += v.x; acc[c][t][4 * q + 1] += v.y; acc[c][t][4 * q + 2] += v.z; acc[c][t][4 * q + 3] += v.w; }
                }
        r4 += sk_part_floats<COT, PXT>() / 4;
    }
    conv_epilogue<COT, PXT>(a, acc, cg, half, HoWo, pvalid, out_pix);
}

// ---------------------------------------------------------------------------------------------
// first layers: Ci in {1,2,3}; input block is [H][W][Ci], filter [Co/16][kh][kw][Ci][16]
// grid.x over pixels, grid.y = output channel block (uniform per workgroup -> scalar weight loads)
template <int CI>
__global__ __launch_bounds__(256) void conv_smallci_f32_kernel(const ConvArgs a)
{
    // a lane computes all 16 channels of one output pixel; the wave's 64 x 16 results are turned round in a
    // wave-private LDS tile so that every store instruction writes 1 KiB of consecutive bytes (a lane
    // storing its own 64 bytes in four pieces touches a quarter of each line per instruction)
    constexpr int ROW = CB + 4;                              // padded pixel row in floats
    __shared__ __align__(16) float tile[4][WAVE * ROW];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int p0 = blockIdx.x * 256 + threadIdx.x;
    const bool live = p0 < a.P;
    const int p = live ? p0 : 0;
    const int cob = blockIdx.y;
    const int HoWo = a.Ho * a.Wo;
    const int n = p / HoWo;
    const int rem = p - n * HoWo;
    const int oh = rem / a.Wo;
    const int ow = rem - oh * a.Wo;
    const int ih0 = oh * a.stride_h - a.pt, iw0 = ow * a.stride - a.pl;
    const float *img = a.in + (size_t)n * a.H * a.W * CI;
    const float *w = a.filt + (size_t)cob * a.kh * a.kw * CI * CB;

    float acc[CB];
#pragma unroll
    for (int j = 0; j < CB; ++j) acc[j] = 0.f;
    // One window tap per iteration, straight-line inside (a padded tap reads the zero block): the tap's
    // CI x 16 weights are uniform, i.e. scalar loads feeding the FMAs directly.  The loop is kept rolled on
    // purpose: unrolled, the compiler hoists all kh*kw*CI*16 scalar weights and spills them.
    const int taps = a.kh * a.kw;
    int ta = 0, tb = 0;
#pragma unroll 1
    for (int tap = 0; tap < taps; ++tap)
    {
        const int ih = ih0 + ta, iw = iw0 + tb;
        const bool ok = live && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
        const float *ip = ok ? img + (ih * a.W + iw) * CI : g_zero_block;
        const float *wp = w + tap * (CI * CB);
        float x[CI];
#pragma unroll
        for (int ci = 0; ci < CI; ++ci) x[ci] = ip[ci];
#pragma unroll
        for (int ci = 0; ci < CI; ++ci)
#pragma unroll
            for (int j = 0; j < CB; ++j) acc[j] = fmaf(x[ci], wp[ci * CB + j], acc[j]);
        if (++tb == a.kw) { tb = 0; ++ta; }
    }
    float *mine = &tile[wave][lane * ROW];
#pragma unroll
    for (int q = 0; q < 4; ++q)
        reinterpret_cast<float4 *>(mine)[q] = make_float4(acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]);
    // the pixel's position in the output travels with its row (in the padding): consecutive pixels of the
    // wave's run are consecutive in the output except where the run crosses into the next image
    const unsigned long long opos = (((unsigned long long)n * (a.Co / CB) + cob) * HoWo + rem) * CB;
    *reinterpret_cast<uint2 *>(mine + CB) = make_uint2((unsigned)opos, (unsigned)(opos >> 32));
    __syncthreads();
    // vector v of the wave's 64-pixel run: pixel v / 4, channel quad v % 4
    const float nscale = act_scale(a.act, a.slope);
    const int wave_p0 = blockIdx.x * 256 + wave * WAVE;
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        const int v = j * WAVE + lane, px = v >> 2, q = v & 3;
        if (wave_p0 + px < a.P)
        {
            const uint2 op = *reinterpret_cast<const uint2 *>(&tile[wave][px * ROW + CB]);
            float4 *o = reinterpret_cast<float4 *>(a.out + (((unsigned long long)op.y << 32) | op.x)) + q;
            float4 r = *reinterpret_cast<const float4 *>(&tile[wave][px * ROW + q * 4]);
            if (a.accumulate)
            {
                const float4 old = *o;
                r.x += old.x; r.y += old.y; r.z += old.z; r.w += old.w;
            }
            if (a.bias)
            {
                const float4 b = *reinterpret_cast<const float4 *>(a.bias + cob * CB + q * 4);
                r.x += b.x; r.y += b.y; r.z += b.z; r.w += b.w;
            }
            r.x = act_bf(r.x, nscale); r.y = act_bf(r.y, nscale); r.z = act_bf(r.z, nscale); r.w = act_bf(r.w, nscale);
            *o = r;
        }
    }
}

// Ci in {1,2,3} on the matrix cores.  The reduction index (tap, ci) is only kh*kw*Ci long (27 for
// a 3x3 RGB stem) and the filter block [kh][kw][Ci][16] is already a [K][16] matrix, so a K-step
// of the 32x32x2 MFMA takes one reduction element in lanes 0..31 and another in lanes 32..63: one
// input dword and one filter dword per lane and step, no repacking.  The order of the reduction is
// free, and it is chosen so that every step's window positions are compile-time constants:
//   Ci == 2: step s = tap s, the wave halves take ci 0 / 1
//   Ci == 3: steps 0..taps-1 the same with ci 0 / 1, then ci 2 of taps 2j / 2j+1 in step taps+j
//   Ci == 1: step s = taps 2s / 2s+1
// Row and column validity of the window is computed once per pixel; every load is issued before the
// first MFMA, masked positions load from the zero block.  A wave multiplies PXT tiles of 32 pixels
// by one tile of 32 output channels.
template <int CI, int KH, int KW>
struct SmallCiSteps
{
    static constexpr int TAPS = KH * KW;
    static constexpr int NS = CI == 1 ? (TAPS + 1) / 2 : CI == 2 ? TAPS : TAPS + (TAPS + 1) / 2;
    // window tap and channel of (step, wave half); tap == TAPS means "nothing" (contributes zero)
    static constexpr int tap(int s, int h)
    {
        if (CI == 1) return 2 * s + h < TAPS ? 2 * s + h : TAPS;
        if (CI == 2) return s;
        if (s < TAPS) return s;
        return 2 * (s - TAPS) + h < TAPS ? 2 * (s - TAPS) + h : TAPS;
    }
    static constexpr int ci(int s, int h)
    {
        if (CI == 1) return 0;
        if (CI == 2) return h;
        return s < TAPS ? h : 2;
    }
};

template <int CI, int KH, int KW, int PXT>
__global__ __launch_bounds__(256) void conv_smallci_mfma_f32_kernel(const ConvArgs a)
{
    using St = SmallCiSteps<CI, KH, KW>;
    constexpr int NS = St::NS, TAPS = St::TAPS;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int cg = blockIdx.y;                       // tile of 32 output channels
    const int HoWo = a.Ho * a.Wo;
    const int CoB = a.Co / CB;

    const float *img[PXT];                           // window origin of the lane's pixel (may lie outside)
    bool rowok[PXT][KH], colok[PXT][KW];
    bool pvalid[PXT];
    size_t out_pix[PXT];
#pragma unroll
    for (int t = 0; t < PXT; ++t)
    {
        const int p = ((blockIdx.x * 4 + wave) * PXT + t) * 32 + col;
        pvalid[t] = p < a.P;
        const int pc = pvalid[t] ? p : 0;
        const int n = pc / HoWo;
        const int rem = pc - n * HoWo;
        const int oh = rem / a.Wo;
        const int ow = rem - oh * a.Wo;
        const int ih0 = oh * a.stride_h - a.pt, iw0 = ow * a.stride - a.pl;
#pragma unroll
        for (int r = 0; r < KH; ++r) rowok[t][r] = pvalid[t] && (unsigned)(ih0 + r) < (unsigned)a.H;
#pragma unroll
        for (int c = 0; c < KW; ++c) colok[t][c] = (unsigned)(iw0 + c) < (unsigned)a.W;
        // 32-bit element offsets inside one image (the launcher checks H*W*Ci < 2^31)
        img[t] = a.in + (size_t)n * a.H * a.W * CI + (ih0 * a.W + iw0) * CI;
        out_pix[t] = ((size_t)n * CoB * HoWo + rem) * CB;
    }
    // filter row of this lane: channel co = cg*32 + col, reduction element k at w_row[k * 16]
    const int co = cg * 32 + col;
    const bool co_ok = co < a.Co;
    const int cc = co_ok ? co : a.Co - 1;
    const float *w_row = a.filt + (size_t)(cc / CB) * (TAPS * CI) * CB + (cc % CB);

    float av[NS], bv[NS][PXT];
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        const int t0 = St::tap(s, 0), t1 = St::tap(s, 1);
        const int c0 = St::ci(s, 0), c1 = St::ci(s, 1);
        const bool e0 = t0 < TAPS, e1 = t1 < TAPS;       // compile-time after unrolling
        const int k0 = e0 ? t0 * CI + c0 : 0, k1 = e1 ? t1 * CI + c1 : 0;
        const bool exists = half ? e1 : e0;
        const float *wp = exists && co_ok ? w_row + (half ? k1 : k0) * CB : g_zero_block;
        av[s] = *wp;
        const int r0 = e0 ? t0 / KW : 0, q0 = e0 ? t0 % KW : 0;
        const int r1 = e1 ? t1 / KW : 0, q1 = e1 ? t1 % KW : 0;
        const int d0 = (r0 * a.W + q0) * CI + c0, d1 = (r1 * a.W + q1) * CI + c1;
#pragma unroll
        for (int t = 0; t < PXT; ++t)
        {
            const bool ok = half ? (e1 && rowok[t][r1] && colok[t][q1]) : (e0 && rowok[t][r0] && colok[t][q0]);
            const float *bp = ok ? img[t] + (half ? d1 : d0) : g_zero_block;
            bv[s][t] = *bp;
        }
    }

    floatx16 acc[1][PXT];
#pragma unroll
    for (int t = 0; t < PXT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[0][t][r] = 0.f;
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int t = 0; t < PXT; ++t)
            acc[0][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[s], bv[s][t], acc[0][t], 0, 0, 0);
    conv_epilogue<1, PXT>(a, acc, cg, half, HoWo, pvalid, out_pix);
}

// First layers with a 3x3 window (Ci in {1,2,3}), any multiple of 16 output channels: the input patch
// under a 16 x 16 tile of output pixels is staged ONCE per workgroup in LDS (coalesced row segments of the
// [H][W][Ci] image, zero where the window leaves the image), and the product runs on
// v_mfma_f32_16x16x4_f32: rows = the 16 channels of the block, columns = the 16 pixels of one tile row,
// K-step = four consecutive reduction elements k = tap * Ci + ci, one per 16-lane group.  In LDS the patch
// has a compile-time pitch, so the position of (tap, ci) relative to a lane's pixel is a compile-time
// constant: a B operand costs one LDS read with an immediate offset, where a gather from global memory
// costs about eight address instructions per element (what bounds the kernels above on these layers).
// A lane ends up with four consecutive channels of one pixel; a store instruction covers 16 pixels x 64
// bytes of consecutive memory.  Wave w owns tile rows 4w .. 4w+3; a workgroup runs NCOB channel blocks on
// the patch it staged.
// VEC: the patch rows are staged with 16-byte loads.  A row segment starts at float (16 S tx - l_pad) * CI of its image row,
// i.e. 0..3 floats (`lead`, the same for every tile of a launch) past a 16-byte boundary; the segment is fetched from that
// boundary on, 13 times fewer load instructions and index computations than float by float (the launcher asks for it when
// image rows are whole 16-byte pieces, so that a piece is either inside the image or outside it).
template <int CI, int S, int NCOB, bool POOL = false, bool VEC = false>
__global__ __launch_bounds__(256) void conv_stem3x3_lds_f32_kernel(const ConvArgs a, int tiles_x, int tiles_y)
{
    typedef float floatx4v __attribute__((ext_vector_type(4)));
    constexpr int T = 16;                                    // tile side in output pixels
    constexpr int PH = (T - 1) * S + 3, PW = PH;             // input patch in pixels
    // The patch is staged by the memory pipeline (global_load_lds: a wave's 64 lanes write consecutive LDS, each lane gives
    // its own global address, positions outside the image read a block of zeros): no registers, no LDS store instructions.
    // VEC: 16-byte pieces, J lanes per patch row, the row pitch is 4 J floats so that a wave's pieces are consecutive.
    constexpr int P4 = (PW * CI + 3 + 3) / 4;                // 16-byte pieces per staged row (VEC)
    constexpr int J = P4 <= 8 ? 8 : P4 <= 16 ? 16 : P4 <= 32 ? 32 : 64;   // lanes per row (power of two)
    static_assert(!VEC || P4 <= 64, "patch row too long");
    constexpr int PITCH = VEC ? 4 * J : PW * CI;             // floats per staged patch row
    constexpr int VROWS = 256 / J, VPASS = (PH + VROWS - 1) / VROWS;
    constexpr int SPASS = (PH * PITCH + 255) / 256;          // rounds of 256 floats (not VEC)
    constexpr int NEL = VEC ? VPASS * VROWS * PITCH : SPASS * 256;   // every lane writes in every round
    constexpr int K = 9 * CI, NS = (K + 3) / 4;
    __shared__ __align__(16) float patch[NEL];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 15, kq = lane >> 4;
    const int CoB = a.Co / CB;
    const int HoWo = a.Ho * a.Wo;
    int tile = blockIdx.x;
    const int n = tile / (tiles_x * tiles_y);
    tile -= n * (tiles_x * tiles_y);
    const int ty = tile / tiles_x, tx = tile - ty * tiles_x;
    const int oh0 = ty * T, ow0 = tx * T;
    const int iw_base = ow0 * S - a.pl;

    // the first channel block's filter and bias are requested before the patch, so that one memory latency covers both
    // filter: element k of channel co at w_blk[k * 16 + co % 16]; this lane's k in step s is 4s + kq
    float av[NS];
    float4 bb = make_float4(0.f, 0.f, 0.f, 0.f);
    auto load_filter = [&](const int cob) {
        const float *w_blk = a.filt + (size_t)cob * (K * CB) + col;
#pragma unroll
        for (int s = 0; s < NS; ++s)
        {
            const int k = 4 * s + kq;
            const float *wp = k < K ? w_blk + k * CB : g_zero_block;
            av[s] = *wp;
        }
        if (a.bias) bb = *reinterpret_cast<const float4 *>(a.bias + cob * CB + 4 * kq);
    };
    load_filter(blockIdx.y * NCOB);

    // ---- stage the patch --------------------------------------------------------------------------------
    // stage_patch(tile id, LDS base of round 0, LDS floats between rounds): requests the patch under tile `t` of the launch
    const int row_el = a.W * CI;                             // floats per image row
    const int lead = VEC ? ((iw_base * CI) & 3) : 0;         // two's complement: also right for -CI; the same for every tile
    auto stage_patch = [&](int t, float *dst, const int round_floats) {
        const int n_ = t / (tiles_x * tiles_y);
        t -= n_ * (tiles_x * tiles_y);
        const int ty_ = t / tiles_x, tx_ = t - ty_ * tiles_x;
        const int ih_base = ty_ * T * S - a.pt, iw_b = tx_ * T * S - a.pl;
        const float *img = a.in + (size_t)n_ * a.H * a.W * CI;
        if (VEC)
        {
            const int xa = iw_b * CI - lead;                 // multiple of 4
            const int j = tid & (J - 1), r0 = tid / J;
#pragma unroll
            for (int ps = 0; ps < VPASS; ++ps)
            {
                const int py = r0 + ps * VROWS, ih = ih_base + py, xe = xa + 4 * j;
                const bool ok = j < P4 && py < PH && (unsigned)ih < (unsigned)a.H && xe >= 0 && xe < row_el;
                const float *gp = ok ? img + ih * row_el + xe : g_zero_block;
                // lane (row r0, piece j) of round ps writes patch[(ps * VROWS + r0) * PITCH + 4 j] = 16 bytes at 16 (ps * 256 + tid)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                                 (__attribute__((address_space(3))) void *)&dst[ps * round_floats + wave * 64 * 4], 16, 0, 0);
            }
        }
        else
        {
            // element e = (patch row, position inside the row segment)
#pragma unroll
            for (int j = 0; j < SPASS; ++j)
            {
                const int e = tid + j * 256;
                const int py = e / PITCH, x = e - py * PITCH;
                const int ih = ih_base + py, xe = iw_b * CI + x;
                const bool ok = py < PH && (unsigned)ih < (unsigned)a.H && (unsigned)xe < (unsigned)row_el;
                const float *gp = ok ? img + ih * row_el + xe : g_zero_block;
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                                 (__attribute__((address_space(3))) void *)&dst[j * round_floats + wave * 64], 4, 0, 0);
            }
        }
    };
    stage_patch(blockIdx.x, patch, VEC ? 256 * 4 : 256);
    __builtin_amdgcn_s_waitcnt(0x0F70);                      // vmcnt(0): this lane's pieces have landed
    __syncthreads();

    // patch position of reduction element k = tap * CI + ci = 4 s + kq, relative to the lane's pixel: window row k / (3 CI),
    // then k % (3 CI) floats along the row (the three columns of a window row are contiguous)
    const int lane_base = 4 * wave * S * PITCH + col * S * CI + lead;   // pixel (row 4w, column col); tile row t adds t*S*PITCH
    int off[NS];
    bool kvalid[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        const int k = 4 * s + kq;
        kvalid[s] = 4 * s + 3 < K || k < K;                  // compile-time true but for the last step
        const int kc = kvalid[s] ? k : 0;
        const int wr = (kc >= 3 * CI ? 1 : 0) + (kc >= 6 * CI ? 1 : 0);
        off[s] = lane_base + wr * PITCH + (kc - wr * 3 * CI);
    }
    const float nscale = act_scale(a.act, a.slope);
    const int ow = ow0 + col;

    // ---- the workgroup's channel blocks, one after the other on the same patch ------------------------
#pragma unroll
    for (int cb_i = 0; cb_i < NCOB; ++cb_i)
    {
        const int cob = blockIdx.y * NCOB + cb_i;            // the launcher makes Co / 16 a multiple of NCOB
        if (cb_i > 0) load_filter(cob);
        floatx4v acc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t] = floatx4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int t = 0; t < 4; ++t)
            {
                const float b = patch[off[s] + t * (S * PITCH)];
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[s], kvalid[s] ? b : 0.f, acc[t], 0, 0, 0);
            }
        // lane: channels cob*16 + 4*kq .. +3 of pixel (oh0 + 4w + t, ow0 + col)
        if (POOL)
        {
            // MaxPool2D 2x2 stride 2 (no padding) of the activated result, in registers: tile rows t and
            // t+1 are this lane's own accumulators, the neighbouring column is lane ^ 1.  Even columns
            // store; the output tensor is [N][Co/16][Ho/2][Wo/2][16].
            const int Hp = a.Ho >> 1, Wp = a.Wo >> 1;
#pragma unroll
            for (int t = 0; t < 4; t += 2)
            {
                float m[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    // the maximum first, bias and activation once: x -> act(x + b) is non-decreasing (rounding included;
                    // negative LeakyReLU slopes are refused for this call), so it commutes with max bit for bit
                    const float be = e == 0 ? bb.x : e == 1 ? bb.y : e == 2 ? bb.z : bb.w;
                    const float v = acc[t][e] > acc[t + 1][e] ? acc[t][e] : acc[t + 1][e];
                    const float u = __shfl_xor(v, 1, WAVE);
                    m[e] = act_bf((v > u ? v : u) + be, nscale);
                }
                const int ohp = (oh0 + 4 * wave + t) >> 1, owp = ow >> 1;
                if ((col & 1) == 0 && ohp < Hp && owp < Wp)
                    *reinterpret_cast<float4 *>(a.out + (((size_t)n * CoB + cob) * (Hp * Wp) + ohp * Wp + owp) * CB + 4 * kq) =
                        make_float4(m[0], m[1], m[2], m[3]);
            }
            continue;
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
        {
            const int oh = oh0 + 4 * wave + t;
            const bool ok = oh < a.Ho && ow < a.Wo;
            float4 *o = reinterpret_cast<float4 *>(a.out + (((size_t)n * CoB + cob) * HoWo + (ok ? oh * a.Wo + ow : 0)) * CB + 4 * kq);
            float4 v = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
            if (a.accumulate)
            {
                float4 old = make_float4(0.f, 0.f, 0.f, 0.f);
                if (ok) old = *o;
                v.x += old.x; v.y += old.y; v.z += old.z; v.w += old.w;
            }
            v.x += bb.x; v.y += bb.y; v.z += bb.z; v.w += bb.w;
            v.x = act_bf(v.x, nscale); v.y = act_bf(v.y, nscale); v.z = act_bf(v.z, nscale); v.w = act_bf(v.w, nscale);
            if (ok) *o = v;
        }
    }
}

// First layer (3x3 window, 1-3 input channels) + bias + activation followed by a 3x3 stride-1 depthwise convolution with
// one pixel of padding all round + bias + activation, in one launch (the reference's Conv2D_ReLU_DepthwiseConv2D_ReLU
// pairing, fused_interface_abstract.hpp:1840; MobileNetV1's first two layers).  A workgroup produces a 14 x 14 tile of
// the depthwise output: it stages the input patch and multiplies exactly like conv_stem3x3_lds_f32_kernel, but on the
// 16 x 16 tile of first-layer pixels that the 14 x 14 depthwise outputs need (one pixel of halo all round; positions
// outside the first layer's output are the depthwise layer's zero padding), parks the activated result of one channel
// block in LDS as [pixel][16 channels] and runs the depthwise window on it like dw3x3_f32_tile_kernel (a lane = one
// column, four channels, four rows, a three-row register window; the same order of operations, so the result equals
// the two launches bit for bit).  The first layer's output (the largest tensor of the model) is never written or read.
struct StemDwArgs
{
    const float *dw_filt;   // [Co/16][3][3][16]
    const float *dw_bias;   // [Co] or nullptr
};

template <int CI, int S, int NCOB, bool RELU = false>
__global__ __launch_bounds__(256, 4) void conv_stem3x3_dw3x3_f32_kernel(const ConvArgs a, const StemDwArgs d, int tiles_x, int tiles_y)
{
    typedef float floatx4v __attribute__((ext_vector_type(4)));
    constexpr int T = 16, TO = 14;                           // first-layer tile side, depthwise tile side
    constexpr int PH = (T - 1) * S + 3, PW = PH;             // input patch in pixels
    constexpr int PITCH = PW * CI;
    constexpr int SPASS = (PH * PITCH + 255) / 256;
    constexpr int NEL = SPASS * 256;
    constexpr int K = 9 * CI, NS = (K + 3) / 4;
    __shared__ __align__(16) float patch[NEL];
    __shared__ float4 mid[T * T * 4];                        // [row][column][channel quad] of one channel block
    // Both layers' filters and biases of the workgroup's channel blocks, staged with the patch: the passes below then read
    // them from LDS instead of waiting for memory twice per pass.  Per block: F4 pieces of first-layer filter, 36 of
    // depthwise filter, 4 + 4 of the two biases (zeros where there is none); a piece is 16 bytes.
    constexpr int F4 = K * CB / 4, PB = F4 + 44, NP = NCOB * PB, PRND = (NP + 255) / 256;
    __shared__ float4 par[PRND * 256];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 15, kq = lane >> 4;
    const int CoB = a.Co / CB;
    const int HoWo = a.Ho * a.Wo;
    int tile = blockIdx.x;
    const int n = tile / (tiles_x * tiles_y);
    tile -= n * (tiles_x * tiles_y);
    const int ty = tile / tiles_x, tx = tile - ty * tiles_x;
    const int oh0 = ty * TO - 1, ow0 = tx * TO - 1;          // first-layer pixel of tile position (0, 0)
    const int ih_base = oh0 * S - a.pt, iw_base = ow0 * S - a.pl;

    // ---- stage the input patch (memory pipeline straight to LDS, zeros outside the image) -----------------
    const float *img = a.in + (size_t)n * a.H * a.W * CI;
    const int row_el = a.W * CI;
#pragma unroll
    for (int j = 0; j < SPASS; ++j)
    {
        const int e = tid + j * 256;
        const int py = e / PITCH, x = e - py * PITCH;
        const int ih = ih_base + py, xe = iw_base * CI + x;
        const bool ok = py < PH && (unsigned)ih < (unsigned)a.H && (unsigned)xe < (unsigned)row_el;
        const float *gp = ok ? img + ih * row_el + xe : g_zero_block;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                         (__attribute__((address_space(3))) void *)&patch[j * 256 + wave * 64], 4, 0, 0);
    }
    {
        const int cob0 = blockIdx.y * NCOB;
        const float4 *zero4 = reinterpret_cast<const float4 *>(g_zero_block);
#pragma unroll
        for (int r = 0; r < PRND; ++r)
        {
            const int piece = tid + r * 256;
            const int b = piece / PB, i = piece - b * PB, cob = cob0 + b;
            const float4 *gp = zero4;
            if (piece < NP)
            {
                if (i < F4) gp = reinterpret_cast<const float4 *>(a.filt + (size_t)cob * (K * CB)) + i;
                else if (i < F4 + 36) gp = reinterpret_cast<const float4 *>(d.dw_filt) + (size_t)cob * 36 + (i - F4);
                else if (i < F4 + 40) { if (a.bias) gp = reinterpret_cast<const float4 *>(a.bias + cob * CB) + (i - F4 - 36); }
                else if (d.dw_bias) gp = reinterpret_cast<const float4 *>(d.dw_bias + cob * CB) + (i - F4 - 40);
            }
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gp,
                                             (__attribute__((address_space(3))) void *)&par[r * 256 + wave * 64], 16, 0, 0);
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();

    const int lane_base = 4 * wave * S * PITCH + col * S * CI;
    int off[NS];
    bool kvalid[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
    {
        const int k = 4 * s + kq;
        kvalid[s] = 4 * s + 3 < K || k < K;
        const int kc = kvalid[s] ? k : 0;
        const int wr = (kc >= 3 * CI ? 1 : 0) + (kc >= 6 * CI ? 1 : 0);
        off[s] = lane_base + wr * PITCH + (kc - wr * 3 * CI);
    }
    const float nscale = act_scale(a.act, a.slope);
    const int ow1 = ow0 + col;                               // first-layer column of this lane
    const bool col_in = (unsigned)ow1 < (unsigned)a.Wo;

    // depthwise phase: lane = (channel quad q, column dx, row group sy), rows sy*4 .. sy*4+3 of the 14 x 14 tile
    const int q = tid & 3, slot = tid >> 2;
    const int dx = slot & 15, sy = slot >> 4;
    const int dwo = tx * TO + dx;                            // depthwise output column
    const bool dcol_ok = dx < TO && dwo < a.Wo;

#pragma unroll 1
    for (int cb_i = 0; cb_i < NCOB; ++cb_i)
    {
        const int cob = blockIdx.y * NCOB + cb_i;
        // ---- first layer on the 16 x 16 tile ---------------------------------------------------------------
        const float4 *pb = par + cb_i * PB;                  // this block's staged parameters
        const float *w_blk = reinterpret_cast<const float *>(pb) + col;
        float av[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s)
        {
            const int k = 4 * s + kq;
            av[s] = k < K ? w_blk[(k < K ? k : 0) * CB] : 0.f;
        }
        floatx4v acc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t] = floatx4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int t = 0; t < 4; ++t)
            {
                const float b = patch[off[s] + t * (S * PITCH)];
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[s], kvalid[s] ? b : 0.f, acc[t], 0, 0, 0);
            }
        const float4 bb = pb[F4 + 36 + kq];
        if (cb_i > 0) __syncthreads();                       // the previous block's depthwise reads are done
#pragma unroll
        for (int t = 0; t < 4; ++t)
        {
            const int row = 4 * wave + t, oh1 = oh0 + row;
            float4 v = make_float4(acc[t][0] + bb.x, acc[t][1] + bb.y, acc[t][2] + bb.z, acc[t][3] + bb.w);
            v.x = act_k<RELU>(v.x, nscale); v.y = act_k<RELU>(v.y, nscale); v.z = act_k<RELU>(v.z, nscale); v.w = act_k<RELU>(v.w, nscale);
            // outside the first layer's output: the depthwise layer's padding
            if (!(col_in && (unsigned)oh1 < (unsigned)a.Ho)) v = make_float4(0.f, 0.f, 0.f, 0.f);
            mid[(row * T + col) * 4 + kq] = v;
        }
        __syncthreads();

        // ---- depthwise 3x3 on the parked tile ----------------------------------------------------------------
        float4 w[9];
#pragma unroll
        for (int t = 0; t < 9; ++t) w[t] = pb[F4 + t * 4 + q];
        const float4 dbias = pb[F4 + 40 + q];
        const float4 *xs = mid + ((sy * 4) * T + (dx < TO ? dx : 0)) * 4 + q;     // idle columns read in bounds
        float4 *dst = reinterpret_cast<float4 *>(a.out) + ((size_t)(n * CoB + cob) * HoWo + dwo) * 4 + q;
        float4 win[3][3];
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int c = 0; c < 3; ++c) win[r][c] = xs[(r * T + c) * 4];
#pragma unroll
        for (int o = 0; o < 4; ++o)
        {
            const int lr = sy * 4 + o;                       // row inside the 14 x 14 tile
            const int rr = lr + 2 < T ? o + 2 : o;           // rows 14, 15 of the tile have no third window row: not stored
#pragma unroll
            for (int c = 0; c < 3; ++c) win[(o + 2) % 3][c] = xs[(rr * T + c) * 4];
            const int oh = ty * TO + lr;
            const bool ok = dcol_ok && lr < TO && oh < a.Ho;
            float4 acc2 = dbias;
#pragma unroll
            for (int r = 0; r < 3; ++r)
#pragma unroll
                for (int c = 0; c < 3; ++c)
                {
                    const float4 x = win[(o + r) % 3][c];
                    const float4 k = w[r * 3 + c];
                    acc2.x = fmaf(x.x, k.x, acc2.x); acc2.y = fmaf(x.y, k.y, acc2.y);
                    acc2.z = fmaf(x.z, k.z, acc2.z); acc2.w = fmaf(x.w, k.w, acc2.w);
                }
            acc2.x = act_k<RELU>(acc2.x, nscale); acc2.y = act_k<RELU>(acc2.y, nscale);
            acc2.z = act_k<RELU>(acc2.z, nscale); acc2.w = act_k<RELU>(acc2.w, nscale);
            if (ok) dst[(size_t)oh * a.Wo * 4] = acc2;
        }
    }
}

// Pointwise convolution (1x1 window, stride 1, no padding; 16 * CIB input channels, CIB <= 8) + bias + activation followed by a 3x3
// depthwise convolution of stride S + bias + activation, in one launch: the reference's Conv2D_ReLU_DepthwiseConv2D_ReLU
// pairing (fused_interface_abstract.hpp:1840) for the blocked layers, MobileNetV1's 1x1 -> 3x3 depthwise sequence.  The
// pointwise layer's output, the largest tensor of such a pair, is neither written nor read.
// A workgroup owns 32 * COT channels and a tile of TOH x TOW depthwise outputs of one image (14 x 14 at stride 1, 7 x 8 at
// stride 2).  The PH x PW pointwise pixels under that tile (16 x 16 / 15 x 17, at most 256) are eight 32-pixel MFMA tiles,
// two per wave; the filter slice of the workgroup is staged in LDS once (memory pipeline, padded 16 x 16 tiles), the
// activation operand goes from memory to the MFMA register as in conv_lds_tile, and the K loop is unrolled: no barrier
// and no staging inside it.  The products are added in conv_lds_tile's order.  The activated result is parked in LDS as
// [pixel][channel] (zeros outside the pointwise layer's map: the depthwise layer's padding) and the depthwise window
// runs on it like dw3x3_f32_tile_kernel (a lane = four channels of one column, a run of rows, the same order of operations).
// The halo is computed again by the neighbouring workgroups: 256 / 196 = 1.31 x the pointwise work at stride 1,
// 255 / 224 = 1.14 x at stride 2.
template <int S>
struct PwDwTile
{
    static constexpr int TOH = S == 1 ? 14 : 7, TOW = S == 1 ? 14 : 8;
    static constexpr int PH = (TOH - 1) * S + 3, PW = (TOW - 1) * S + 3;
    static constexpr int NPX = PH * PW;
    static_assert(NPX <= 256, "pointwise pixels of a tile vs eight MFMA tiles");
};

struct PwDwGeom
{
    int Hd, Wd;          // depthwise output map
    int dpt, dpl;        // depthwise padding, top and left
    int tiles_x, tiles_y;
    int n_cg;            // channel groups (32 COT channels each)
    int n_wgs, per_xcd;  // workgroups = tiles x channel groups, and their share per XCD
};

template <int S, int COT, int CIB, bool RELU = false>
__global__ __launch_bounds__(256, 2) void conv_pw_dw3x3_f32_kernel(const ConvArgs a, const StemDwArgs d, const PwDwGeom g)
{
    using TL = PwDwTile<S>;
    constexpr int TOH = TL::TOH, TOW = TL::TOW, PW = TL::PW, NPX = TL::NPX;
    constexpr int CG = 32 * COT;                             // channels of the workgroup
    constexpr int MIDP = CG + 4;                             // floats per parked pixel: 16 bytes of padding spread the banks
    constexpr int NFT = 2 * COT * CIB;                       // 16 x 16 filter tiles of the workgroup
    // the filter slice is dead when the K loop ends and the parked tile is born after it: they share their LDS
    constexpr int MID_FLOATS = 256 * MIDP, FILT_FLOATS = NFT * A_TILE_FLOATS;
    __shared__ __align__(16) float lds[MID_FLOATS > FILT_FLOATS ? MID_FLOATS : FILT_FLOATS];
    __shared__ __align__(16) float s_bias[CG];
    float *const filt = lds, *const mid = lds;

    // logical id = (tile, channel group), the channel group fastest; consecutive logical ids run on one XCD: the channel
    // groups of a tile find its input pixels in that XCD's L2, and so do neighbouring tiles their shared halo
    const int bid = blockIdx.x;
    const int lid = (bid % NUM_XCD) * g.per_xcd + bid / NUM_XCD;
    if (lid >= g.n_wgs) return;                              // the whole workgroup leaves, before any barrier
    const int cg = lid % g.n_cg, tile_id = lid / g.n_cg;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, half = lane >> 5;
    const int tiles = g.tiles_x * g.tiles_y;
    const int n = tile_id / tiles, trem = tile_id - n * tiles;
    const int ty = trem / g.tiles_x, tx = trem - ty * g.tiles_x;
    const int py0 = ty * TOH * S - g.dpt, px0 = tx * TOW * S - g.dpl;   // pointwise pixel of patch position (0, 0)
    const int HW = a.H * a.W, CoB = a.Co / CB;
    const float nscale = act_scale(a.act, a.slope);

    // ---- requests first: filter slice to LDS, biases, depthwise taps ------------------------------------------------
    {
        // the slice is 2 COT consecutive channel blocks of CIB tiles each: contiguous in memory, tile after tile
        const float *fsrc = a.filt + (size_t)cg * NFT * (CB * CB) + lane * 4;
#pragma unroll
        for (int t = wave; t < NFT; t += 4)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(fsrc + t * (CB * CB)),
                                             (__attribute__((address_space(3))) void *)&filt[t * A_TILE_FLOATS], 16, 0, 0);
    }
    float my_bias = 0.f;
    if (tid < CG && a.bias) my_bias = a.bias[cg * CG + tid];
    // depthwise phase: lane = (channel quad q, column dx, row group rg)
    constexpr int NQ = CG / 4, TCOLS = S == 1 ? 16 : 8, NRG = 256 / (NQ * TCOLS), RPG = (TOH + NRG - 1) / NRG;
    const int q = tid % NQ, dslot = tid / NQ, dx = dslot % TCOLS, rg = dslot / TCOLS;
    const int dcob = cg * (CG / CB) + q / 4, dq4 = (q & 3) * 4;   // channel block and first channel inside it
    float4 w[9];
    {
        const float4 *wq = reinterpret_cast<const float4 *>(d.dw_filt + (size_t)dcob * (9 * CB) + dq4);
#pragma unroll
        for (int t = 0; t < 9; ++t) w[t] = wq[t * 4];
    }
    float4 dbias = make_float4(0.f, 0.f, 0.f, 0.f);
    if (d.dw_bias) dbias = *reinterpret_cast<const float4 *>(d.dw_bias + dcob * CB + dq4);

    // ---- pointwise layer on the patch --------------------------------------------------------------------------------
    // this lane's two pixels: patch index p = (2 wave + t) * 32 + col -> position (p / PW, p % PW)
    const float *in_px[2];
    bool pin[2];                                             // inside the pointwise layer's map
    int pidx[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
    {
        const int pp = (2 * wave + t) * 32 + col;
        const int py = pp / PW, pxx = pp - py * PW;
        const int oh = py0 + py, ow = px0 + pxx;
        pin[t] = pp < NPX && (unsigned)oh < (unsigned)a.H && (unsigned)ow < (unsigned)a.W;
        pidx[t] = pp;
        in_px[t] = pin[t] ? a.in + ((size_t)n * CIB * HW + oh * a.W + ow) * CB + half * 8 : g_zero_block + half * 8;
    }
    const int in_blk32 = HW * CB;
    float4 B[2][2][2];                                       // [buffer][pixel tile][half of the eight channels]
    auto fetch = [&](const int buf, const int cib) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
        {
            const float4 *p4 = reinterpret_cast<const float4 *>(in_px[t] + (pin[t] ? cib * in_blk32 : 0));
            B[buf][t][0] = p4[0];
            B[buf][t][1] = p4[1];
        }
    };
    fetch(0, 0);
    if (CIB > 1) fetch(1, 1);
    if (tid < CG) s_bias[tid] = my_bias;
    __builtin_amdgcn_s_waitcnt(0x0F70);                      // vmcnt(0): the filter tiles have landed
    __syncthreads();

    int a_rd[COT];
#pragma unroll
    for (int c = 0; c < COT; ++c) a_rd[c] = (c * 2 + (col >> 4)) * CIB * A_TILE_FLOATS + half * 8 * CB + (col & 15);
    floatx16 acc[COT][2];
#pragma unroll
    for (int c = 0; c < COT; ++c)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[c][t][r] = 0.f;
#pragma unroll
    for (int s = 0; s < CIB; ++s)
    {
        float A[COT][8];
#pragma unroll
        for (int c = 0; c < COT; ++c)
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) A[c][kk] = filt[a_rd[c] + s * A_TILE_FLOATS + kk * CB];
#pragma unroll
        for (int kk = 0; kk < 8; ++kk)
#pragma unroll
            for (int t = 0; t < 2; ++t)
            {
                const float4 bv = B[s & 1][t][kk >> 2];
                const float b = (kk & 3) == 0 ? bv.x : (kk & 3) == 1 ? bv.y : (kk & 3) == 2 ? bv.z : bv.w;
#pragma unroll
                for (int c = 0; c < COT; ++c)
                    acc[c][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(A[c][kk], b, acc[c][t], 0, 0, 0);
            }
        if (s + 2 < CIB) fetch(s & 1, s + 2);
    }

    __syncthreads();                                         // every wave has read its last filter operand
    // ---- bias, activation, park in LDS: a lane holds channels c*32 + 8 qq + 4 half + 0..3 of its pixel -------------
    // pixels outside the pointwise layer's map are the depthwise layer's padding: those lanes store zeros (a branch on
    // the lane mask: no select per value)
#pragma unroll
    for (int t = 0; t < 2; ++t)
    {
        if (pin[t])
        {
#pragma unroll
            for (int c = 0; c < COT; ++c)
#pragma unroll
                for (int qq = 0; qq < 4; ++qq)
                {
                    const int ch = c * 32 + 8 * qq + 4 * half;
                    const float4 bb = *reinterpret_cast<const float4 *>(&s_bias[ch]);
                    const float4 v = make_float4(act_k<RELU>(acc[c][t][4 * qq + 0] + bb.x, nscale), act_k<RELU>(acc[c][t][4 * qq + 1] + bb.y, nscale),
                                                 act_k<RELU>(acc[c][t][4 * qq + 2] + bb.z, nscale), act_k<RELU>(acc[c][t][4 * qq + 3] + bb.w, nscale));
                    *reinterpret_cast<float4 *>(&mid[pidx[t] * MIDP + ch]) = v;
                }
        }
        else
        {
#pragma unroll
            for (int c = 0; c < COT; ++c)
#pragma unroll
                for (int qq = 0; qq < 4; ++qq)
                    *reinterpret_cast<float4 *>(&mid[pidx[t] * MIDP + c * 32 + 8 * qq + 4 * half]) = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    __syncthreads();

    // ---- depthwise 3x3 on the parked patch ---------------------------------------------------------------------------
    const int dwo = tx * TOW + dx;                           // depthwise output column
    const bool dcol_ok = dx < TOW && dwo < g.Wd;
    const int dxc = dx < TOW ? dx : 0;                       // idle columns read in bounds
    const float *xs = mid + (dxc * S) * MIDP + q * 4;        // window column 0 of this lane, patch row 0
    float4 *dst = reinterpret_cast<float4 *>(a.out + (((size_t)n * CoB + dcob) * g.Hd * g.Wd + dwo) * CB + dq4);
    auto at = [&](const int row, const int c) { return *reinterpret_cast<const float4 *>(xs + (row * PW + c) * MIDP); };
    const int r0 = rg * RPG;                                 // first output row of this lane inside the tile
    float4 win[3][3];
    if (S == 1)
    {
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int c = 0; c < 3; ++c) win[r][c] = at(r0 + r, c);
    }
#pragma unroll
    for (int o = 0; o < RPG; ++o)
    {
        const int lr = r0 + o;                               // output row inside the tile
        const bool row_in = lr < TOH;
        const int lrc = row_in ? lr : TOH - 1;               // rows past the tile read in bounds, nothing is stored
        if (S == 1)
        {
#pragma unroll
            for (int c = 0; c < 3; ++c) win[(o + 2) % 3][c] = at(lrc + 2, c);
        }
        else
        {
#pragma unroll
            for (int r = 0; r < 3; ++r)
#pragma unroll
                for (int c = 0; c < 3; ++c) win[(o + r) % 3][c] = at(lrc * S + r, c);
        }
        const int oh = ty * TOH + lr;
        const bool ok = dcol_ok && row_in && oh < g.Hd;
        float4 acc2 = dbias;
#pragma unroll
        for (int r = 0; r < 3; ++r)
#pragma unroll
            for (int c = 0; c < 3; ++c)
            {
                const float4 x = win[(o + r) % 3][c];
                const float4 k = w[r * 3 + c];
                acc2.x = fmaf(x.x, k.x, acc2.x); acc2.y = fmaf(x.y, k.y, acc2.y);
                acc2.z = fmaf(x.z, k.z, acc2.z); acc2.w = fmaf(x.w, k.w, acc2.w);
            }
        acc2.x = act_k<RELU>(acc2.x, nscale); acc2.y = act_k<RELU>(acc2.y, nscale);
        acc2.z = act_k<RELU>(acc2.z, nscale); acc2.w = act_k<RELU>(acc2.w, nscale);
        if (ok) dst[(size_t)oh * g.Wd * 4] = acc2;
    }
}

// Operand streams through buffer loads (conv_lds_tile's BUF form)?  An ordinary convolution (no slabs) whose input and
// filter are at most BUF_MAX_BYTES each; SMALL_HIP_TUNE key conv_buf=0 keeps the flat-address form.
bool buffer_form(const ConvArgs &a)
{
    static const bool off = tune_int("conv_buf", 1) == 0;
    const long long in_bytes = (long long)a.batch * a.Ci * a.H * a.W * (long long)sizeof(float);
    const long long f_bytes = (long long)((a.Co + CB - 1) / CB * CB) * a.Ci * a.kh * a.kw * (long long)sizeof(float);
    const long long out_bytes = (long long)a.batch * a.Co * a.Ho * a.Wo * (long long)sizeof(float);   // the pooled tensor is smaller
    return !off && a.slabs == 0 && in_bytes <= BUF_MAX_BYTES && f_bytes <= BUF_MAX_BYTES && out_bytes <= BUF_MAX_BYTES;
}

template <int COT, int PXT>
void launch_splitk(ConvArgs &a, hipStream_t s)
{
    set_pixel_divisors(a, false);
    a.n_co_groups = (a.Co + 32 * COT - 1) / (32 * COT);
    a.n_px_blocks = (a.P + 32 * PXT - 1) / (32 * PXT);
    a.n_blocks = a.n_co_groups * a.n_px_blocks;
    a.per_xcd = (a.n_blocks + NUM_XCD - 1) / NUM_XCD;
    const dim3 grid(a.per_xcd * NUM_XCD, a.slabs > 0 ? a.slabs : 1);
    if (buffer_form(a)) hipLaunchKernelGGL((conv_mfma_f32_splitk_kernel<COT, PXT, true>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((conv_mfma_f32_splitk_kernel<COT, PXT>), grid, dim3(256), 0, s, a);
}

// Whole rounds + cut tail (conv_mfma_f32_hybrid_kernel) or whole tiles only?  A split-K piece multiplies about half as
// fast as a whole tile (operands straight from global memory, one MFMA chain per wave), so the cut tail wins while the
// left-over tiles fill at most two thirds of a round and loses beyond, whatever the wave tile and the number of whole rounds.
// Batch sweeps, left-over tiles of 256 -> gain (+) or loss (-) in us: 1x1 256->256 @28x28 (16 K-steps) 32: +3, 128: +1,
// 224: -3; 512->512 @14x14 (32) 80: +2..6, 176: -2, 224: -6; 3x3 64->128 @52x52 (36) 84: +1, 168: -3, 252: -7;
// 3x3 128->256 @26x26 (72) 20: +25, 84: +10, 128: +4, 168: -3, 216: -10; 3x3 256->512 @13x13 (144) 40: +42, 128: +13,
// 168: -12, 216: -27.
template <int COT, int PXT>
bool tail_pays(int n_main, int rest, int nsteps)
{
    // SMALL_HIP_TUNE key conv_tail: 0 = never, 2 = whenever tiles are left over
    static const int knob = tune_int("conv_tail", 1);
    (void)n_main;
    if (knob == 0 || rest == 0 || nsteps < 8) return false;
    // with the split-K pieces on buffer loads the break-even moved up: left-over tiles 160..168 now gain 3..8 us (3x3
    // 128->256 @26x26, 64->128 @52x52 with pooling), 212..252 still lose 1..4 us
    return knob == 2 || rest <= 11 * NUM_CU / 16;
}

template <int COT, int PXT>
void launch_mfma(ConvArgs &a, hipStream_t s)
{
    set_pixel_divisors(a, false);
    a.n_co_groups = (a.Co + 32 * COT - 1) / (32 * COT);
    a.n_px_blocks = (a.P + 32 * PXT * 4 - 1) / (32 * PXT * 4);
    a.n_blocks = a.n_co_groups * a.n_px_blocks;
    a.per_xcd = (a.n_blocks + NUM_XCD - 1) / NUM_XCD;
    const int n_main = a.n_blocks / NUM_CU * NUM_CU, rest = a.n_blocks - n_main;
    // flat addresses: pointwise form of the main loop for 1x1 windows (SMALL_HIP_TUNE key conv_pw=0 switches it off)
    static const bool pw_off = tune_int("conv_pw", 1) == 0;
    // (only where the buffer-load form is not allowed: that one needs no special case for 1x1 windows and is faster,
    // MobileNetV1 batch 64: 512 -> 512 @14x14 55.8 -> 52.5 us, 1024 -> 1024 @7x7 64.4 -> 54.9 us)
    const bool buf = buffer_form(a);
    const bool pw = !buf && !pw_off && a.kh == 1 && a.kw == 1 && a.stride == 1 && a.stride_h == 1 && a.pt == 0 && a.pl == 0 &&
                    a.Ho == a.H && a.Wo == a.W;
    const unsigned slabs_y = a.slabs > 0 ? a.slabs : 1;
    if (tail_pays<COT, PXT>(n_main, rest, a.kh * a.kw * (a.Ci / CB)))
    {
        a.n_main = n_main;
        const dim3 grid(n_main + rest * 4 * COT * PXT, slabs_y);
        if (pw) hipLaunchKernelGGL((conv_mfma_f32_hybrid_kernel<COT, PXT, false, true>), grid, dim3(256), 0, s, a);
        else if (buf) hipLaunchKernelGGL((conv_mfma_f32_hybrid_kernel<COT, PXT, false, false, true>), grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL((conv_mfma_f32_hybrid_kernel<COT, PXT>), grid, dim3(256), 0, s, a);
    }
    else
    {
        const dim3 grid(a.per_xcd * NUM_XCD, slabs_y);
        if (pw) hipLaunchKernelGGL((conv_mfma_f32_lds_kernel<COT, PXT, false, true>), grid, dim3(256), 0, s, a);
        else if (buf) hipLaunchKernelGGL((conv_mfma_f32_lds_kernel<COT, PXT, false, false, true>), grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL((conv_mfma_f32_lds_kernel<COT, PXT>), grid, dim3(256), 0, s, a);
    }
}

// slabs > 0: a grouped convolution, `slabs` (image, group) slabs of one launch (batch must be 1: a slab is one image
// of Ci channels); slab y takes filter block (slab0 + y) % groups
struct GroupSlabs
{
    int slabs = 0, groups = 1, slab0 = 0;
    int stride_h = 0;        // > 0: another vertical stride (1 for the 1-D layers)
};

// The equal-share split of a launch: fills the sk_* fields and the tile counts; returns the scratch bytes it needs, 0 when
// the shape does not qualify.  Few tiles that do not fill whole rounds and a long reduction (measured, batch 16 on 13x13
// maps: 512 -> 1024 3x3 287 -> 264 us, 1024 -> 1024 519 -> 467 us, 256 -> 512 (144 steps) 81 -> 69 us; with 72 steps or
// fewer the fix-up pass costs more than the balance gains).  SMALL_HIP_TUNE keys conv_streamk=<workgroups per compute
// unit> (default 3: 512 -> 1024 @13x13 b16 200.8 -> 198.2 us, 1024 -> 1024 420 -> 416 against 2; 0 = never), conv_streamk_min=<steps> (default 128)
template <int COT, int PXT>
size_t streamk_plan(ConvArgs &a)
{
    static const int min_steps = tune_int("conv_streamk_min", 128);
    static const int per_cu = tune_int("conv_streamk", 3);
    if (per_cu <= 0 || a.slabs != 0 || a.Co % (32 * COT) != 0) return 0;
    a.n_co_groups = (a.Co + 32 * COT - 1) / (32 * COT);
    a.n_px_blocks = (a.P + 32 * PXT * 4 - 1) / (32 * PXT * 4);
    a.n_blocks = a.n_co_groups * a.n_px_blocks;
    const int nsteps = a.kh * a.kw * (a.Ci / CB);
    const long total = (long)a.n_blocks * nsteps;
    if (a.n_blocks <= NUM_CU / 2 || a.n_blocks >= 3 * NUM_CU || a.n_blocks % NUM_CU == 0 || nsteps < min_steps) return 0;
    const int chunks = per_cu * NUM_CU;
    a.sk_chunk = (int)((total + chunks - 1) / chunks);
    a.sk_chunks = (int)((total + a.sk_chunk - 1) / a.sk_chunk);
    a.sk_parts = (nsteps + a.sk_chunk - 1) / a.sk_chunk + 1;
    a.per_xcd = (a.sk_chunks + NUM_XCD - 1) / NUM_XCD;
    return (size_t)a.n_blocks * a.sk_parts * sk_part_floats<COT, PXT>() * sizeof(float);
}

// the equal-share launch pair; *done = false: the shape does not qualify.  The first call on a stream allocates the
// scratch block (small_hip_workspace_reserve does it ahead of time), like the uint8 convolution's filter pre-pass.
template <int COT, int PXT>
int launch_streamk(const char *op, ConvArgs &a, hipStream_t s, bool *done)
{
    *done = false;
    set_pixel_divisors(a, false);
    const size_t bytes = streamk_plan<COT, PXT>(a);
    if (bytes == 0) return SMALL_HIP_OK;
    WorkspaceLease lease;            // held until both launches are enqueued
    if (int rc = lease_workspace(bytes, s, &lease)) return rc;
    a.sk_scratch = static_cast<float *>(lease.ptr);
    if (buffer_form(a)) hipLaunchKernelGGL((conv_mfma_f32_streamk_kernel<COT, PXT, true>), dim3(a.per_xcd * NUM_XCD), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((conv_mfma_f32_streamk_kernel<COT, PXT>), dim3(a.per_xcd * NUM_XCD), dim3(256), 0, s, a);
    SHP_LAUNCH_CHECK(op);
    hipLaunchKernelGGL((conv_streamk_fixup_kernel<COT, PXT>), dim3(a.n_blocks), dim3(256), 0, s, a);
    SHP_LAUNCH_CHECK(op);
    *done = true;
    return SMALL_HIP_OK;
}

// few tiles and a long reduction: K split over the four waves of a workgroup (measured: from one tile per SIMD the
// whole-rounds + tail kernel with 1x1 wave tiles is ahead, e.g. 256->512 3x3 @13x13 batch 16, 1360 tiles: 81 us against 91 us)
inline bool wants_splitk(long tiles32, int nsteps)
{
    static const int force = tune_int("conv_splitk", -1);
    return force >= 0 ? force == 1 : (tiles32 < 4L * NUM_CU && nsteps >= 16);
}

int conv_f32(const char *op, int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int Co,
             int Ci, int H, int W, const float *in, const float *filt, const float *bias, int act, float slope,
             int accumulate, float *out, small_hip_stream_t stream, const GroupSlabs grp = GroupSlabs{})
{
    // interface_abstract.hpp:70-220: pick the channel branch first, the stride inside it
    const bool blocked = Ci > 0 && Ci % CB == 0;
    const bool small_ci = Ci == 1 || Ci == 2 || Ci == 3;
    if (!blocked && !small_ci) return SMALL_HIP_ECHANNELS;
    if (stride != 1 && stride != 2) return SMALL_HIP_ESTRIDE;
    if (batch <= 0 || kh <= 0 || kw <= 0 || H <= 0 || W <= 0 || Co <= 0 || !pads_ok(pt, pb, pl, pr))
    { set_error("%s: bad size", op); return SMALL_HIP_EINVAL; }
    if (Co % CB != 0) { set_error("%s: output_channels must be a multiple of 16 (pad the filter)", op); return SMALL_HIP_EINVAL; }
    if (!in || !filt || !out || !aligned16(filt) || !aligned16(out) || (blocked && !aligned16(in)) ||
        (bias && !aligned16(bias)))
    { set_error("%s: null or misaligned pointer", op); return SMALL_HIP_EINVAL; }
    if (in == out) { set_error("%s: in-place convolution is not supported", op); return SMALL_HIP_EINVAL; }
    if (act < SMALL_HIP_ACT_NONE || act > SMALL_HIP_ACT_LEAKY) { set_error("%s: bad activation", op); return SMALL_HIP_EINVAL; }

    ConvArgs a{};
    a.in = in; a.filt = filt; a.bias = bias; a.out = out;
    a.batch = batch; a.Co = Co; a.Ci = Ci; a.H = H; a.W = W;
    a.kh = kh; a.kw = kw; a.stride = stride; a.pt = pt; a.pl = pl;
    a.stride_h = grp.stride_h > 0 ? grp.stride_h : stride;
    a.Ho = out_dim(H, pt, pb, kh, a.stride_h);
    a.Wo = out_dim(W, pl, pr, kw, stride);
    a.act = act; a.slope = slope; a.accumulate = accumulate;
    if (grp.slabs > 0)
    {
        if (batch != 1 || !blocked || grp.slabs > 65535) { set_error("%s: bad slab launch", op); return SMALL_HIP_EINVAL; }
        a.slabs = grp.slabs; a.groups = grp.groups; a.slab0 = grp.slab0;
        a.in_slab = (long long)Ci * H * W;
        a.out_slab = (long long)Co * a.Ho * a.Wo;
        a.filt_slab = (long long)Co * Ci * kh * kw;
    }
    const long P = (long)batch * a.Ho * a.Wo;
    if (P == 0) return SMALL_HIP_OK;
    if (P > 0x7fffffffL / 64) { set_error("%s: batch*Ho*Wo too large for one launch", op); return SMALL_HIP_EINVAL; }
    if ((long)Ci * H * W > 0x7fffffffL / 2 || (long)Ci * kh * kw * CB > 0x7fffffffL / 2)
    { set_error("%s: one image or one filter block too large for 32-bit offsets", op); return SMALL_HIP_EINVAL; }
    a.P = (int)P;
    hipStream_t s = as_stream(stream);

    if (small_ci)
    {
        // 3x3 windows: the LDS-staged 16x16x4 MFMA kernel (SMALL_HIP_TUNE key stem_lds=0 switches it off)
        static const bool stem_lds_off = tune_int("stem_lds", 1) == 0;
        if (!stem_lds_off && kh == 3 && kw == 3 && (long)H * W * Ci < 0x7fffffffL)
        {
            const int tiles_x = (a.Wo + 15) / 16, tiles_y = (a.Ho + 15) / 16;
            const long nt = (long)batch * tiles_x * tiles_y;
            if (nt <= 0x7fffffffL)
            {
                const int CoB = Co / CB;
                const int ncob = CoB % 4 == 0 ? 4 : CoB % 2 == 0 ? 2 : 1;
                const dim3 gs((unsigned)nt, (unsigned)(CoB / ncob));
                void (*ks)(const ConvArgs, int, int) = nullptr;
                // 16-byte staging (possible when every image row is whole 16-byte pieces) is measured level or slightly behind
                // here (224x224x3 -> 32 stride 2: 33.6 against 34.6 us) and ahead in the pooling form below; on request only
                static const bool vec_on = tune_int("stem_vec", 0) == 1;
                const bool vec = vec_on && (W * Ci) % 4 == 0 && aligned16(in);
#define SHP_STEM_V(CI_, S_, V_) (ncob == 4 ? conv_stem3x3_lds_f32_kernel<CI_, S_, 4, false, V_> : ncob == 2 ? conv_stem3x3_lds_f32_kernel<CI_, S_, 2, false, V_> : conv_stem3x3_lds_f32_kernel<CI_, S_, 1, false, V_>)
#define SHP_STEM(CI_, S_) (vec ? SHP_STEM_V(CI_, S_, true) : SHP_STEM_V(CI_, S_, false))
                if (stride == 1) ks = Ci == 1 ? SHP_STEM(1, 1) : Ci == 2 ? SHP_STEM(2, 1) : SHP_STEM(3, 1);
                else ks = Ci == 1 ? SHP_STEM(1, 2) : Ci == 2 ? SHP_STEM(2, 2) : SHP_STEM(3, 2);
#undef SHP_STEM
#undef SHP_STEM_V
                hipLaunchKernelGGL(ks, gs, dim3(256), 0, s, a, tiles_x, tiles_y);
                SHP_LAUNCH_CHECK(op);
                return SMALL_HIP_OK;
            }
        }
        const dim3 grid((unsigned)((a.P + 255) / 256), (unsigned)(Co / CB));
        static const bool smallci_valu = tune_int("smallci_valu", 0) == 1;
        // measured: with 16 output channels half of every 32-row MFMA tile is idle and the vector-ALU
        // kernel is faster
        if (!smallci_valu && Co >= 32 && (long)H * W * Ci < 0x7fffffffL)
        {
            constexpr int PXT = 2;
            const dim3 gm((unsigned)((a.P + 32 * PXT * 4 - 1) / (32 * PXT * 4)), (unsigned)((Co + 31) / 32));
            void (*km)(const ConvArgs) = nullptr;
            if (kh == 3 && kw == 3)
                km = Ci == 1 ? conv_smallci_mfma_f32_kernel<1, 3, 3, PXT> : Ci == 2 ? conv_smallci_mfma_f32_kernel<2, 3, 3, PXT>
                                                                           : conv_smallci_mfma_f32_kernel<3, 3, 3, PXT>;
            else if (kh == 10 && kw == 4 && Ci == 1)          // the keyword-spotting stem
                km = conv_smallci_mfma_f32_kernel<1, 10, 4, PXT>;
            if (km)
            {
                hipLaunchKernelGGL(km, gm, dim3(256), 0, s, a);
                SHP_LAUNCH_CHECK(op);
                return SMALL_HIP_OK;
            }
        }
        if (Ci == 1) hipLaunchKernelGGL(conv_smallci_f32_kernel<1>, grid, dim3(256), 0, s, a);
        else if (Ci == 2) hipLaunchKernelGGL(conv_smallci_f32_kernel<2>, grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL(conv_smallci_f32_kernel<3>, grid, dim3(256), 0, s, a);
        SHP_LAUNCH_CHECK(op);
        return SMALL_HIP_OK;
    }

    // Wave tile (in 32-channel x 32-pixel MFMA tiles).  Measured on MI355X inside whole-model runs with
    // the balanced tail in place: 2x2 only pays with many tiles per SIMD and a long reduction (big
    // 3x3 layers), 2x1 from 4 tiles per SIMD (from 2 when the reduction has at least 72 steps: 128->256 3x3 @26x26 b16, 2.6 tiles per SIMD, 74 -> 69 us; 1024->1024 1x1 @7x7 b64 with 64 steps stays 1x1: 69 against 73 us), 1x1 below (few tiles: balance matters more than
    // operand re-use).
    const long tiles32 = (long)((Co + 31) / 32) * ((P + 31) / 32) * (grp.slabs > 0 ? grp.slabs : 1);
    const long simds = 4L * NUM_CU;
    const int nsteps = kh * kw * (Ci / CB);
    int cot = 1, pxt = 1;
    if (Co % 64 == 0 && tiles32 >= 16 * simds && nsteps >= 32) { cot = 2; pxt = 2; }
    else if (Co % 64 == 0 && (tiles32 >= 4 * simds || (tiles32 >= 2 * simds && nsteps >= 72))) { cot = 2; pxt = 1; }
    if (wants_splitk(tiles32, nsteps))
    {
        launch_splitk<1, 1>(a, s);
        SHP_LAUNCH_CHECK(op);
        return SMALL_HIP_OK;
    }
    // SMALL_HIP_TUNE key conv_tile=<cot>x<pxt> forces a wave tile (32-channel x 32-pixel units; 1x1 1x2 2x1 2x2)
    {
        int c2 = 0, p2 = 0;
        if (tune_pair("conv_tile", &c2, &p2)) { cot = c2; pxt = p2; }
    }
    // few tiles, long reduction: equal shares of the K-steps
    {
        bool done = false;
        if (int rc = launch_streamk<2, 1>(op, a, s, &done)) return rc;
        if (done) return SMALL_HIP_OK;
    }
    if (cot == 2 && pxt == 2) launch_mfma<2, 2>(a, s);
    else if (cot == 1 && pxt == 2) launch_mfma<1, 2>(a, s);
    else if (cot == 2 && pxt == 1) launch_mfma<2, 1>(a, s);
    else launch_mfma<1, 1>(a, s);
    SHP_LAUNCH_CHECK(op);
    return SMALL_HIP_OK;
}

template <int COT, int PXT>
void launch_mfma_pool(ConvArgs &a, hipStream_t s)
{
    set_pixel_divisors(a, true);
    a.n_co_groups = (a.Co + 32 * COT - 1) / (32 * COT);
    a.n_px_blocks = (a.P + 32 * PXT * 4 - 1) / (32 * PXT * 4);
    a.n_blocks = a.n_co_groups * a.n_px_blocks;
    a.per_xcd = (a.n_blocks + NUM_XCD - 1) / NUM_XCD;
    const int n_main = a.n_blocks / NUM_CU * NUM_CU, rest = a.n_blocks - n_main;
    if (tail_pays<COT, PXT>(n_main, rest, a.kh * a.kw * (a.Ci / CB)))
    {
        a.n_main = n_main;
        if (buffer_form(a)) hipLaunchKernelGGL((conv_mfma_f32_hybrid_kernel<COT, PXT, true, false, true>), dim3(n_main + rest * 4 * COT * PXT), dim3(256), 0, s, a);
        else hipLaunchKernelGGL((conv_mfma_f32_hybrid_kernel<COT, PXT, true>), dim3(n_main + rest * 4 * COT * PXT), dim3(256), 0, s, a);
    }
    else if (buffer_form(a)) hipLaunchKernelGGL((conv_mfma_f32_lds_kernel<COT, PXT, true, false, true>), dim3(a.per_xcd * NUM_XCD), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((conv_mfma_f32_lds_kernel<COT, PXT, true>), dim3(a.per_xcd * NUM_XCD), dim3(256), 0, s, a);
}

// Conv2D + bias + activation + MaxPool2D 2x2 stride 2 (no pool padding) in one launch
int conv_pool_f32(const char *op, int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int pool_kh,
                  int pool_kw, int pool_stride, int ppt, int ppb, int ppl, int ppr, int Co, int Ci, int H, int W,
                  const float *in, const float *filt, const float *bias, int act, float slope, float *out,
                  small_hip_stream_t stream)
{
    const bool blocked = Ci > 0 && Ci % CB == 0;
    const bool small_ci = Ci == 1 || Ci == 2 || Ci == 3;
    if (!blocked && !small_ci) return SMALL_HIP_ECHANNELS;
    if (stride != 1 && stride != 2) return SMALL_HIP_ESTRIDE;
    if (pool_kh != 2 || pool_kw != 2 || pool_stride != 2 || ppt || ppb || ppl || ppr)
    { set_error("%s: only a 2x2 stride-2 pooling window without padding is fused", op); return SMALL_HIP_EINVAL; }
    if (small_ci && (kh != 3 || kw != 3))
    { set_error("%s: first layers (1-3 input channels) are fused for 3x3 windows only", op); return SMALL_HIP_EINVAL; }
    if (batch <= 0 || kh <= 0 || kw <= 0 || H <= 0 || W <= 0 || Co <= 0 || !pads_ok(pt, pb, pl, pr))
    { set_error("%s: bad size", op); return SMALL_HIP_EINVAL; }
    if (Co % CB != 0) { set_error("%s: output_channels must be a multiple of 16 (pad the filter)", op); return SMALL_HIP_EINVAL; }
    if (!in || !filt || !out || !aligned16(filt) || !aligned16(out) || (blocked && !aligned16(in)) ||
        (bias && !aligned16(bias)))
    { set_error("%s: null or misaligned pointer", op); return SMALL_HIP_EINVAL; }
    if (in == out) { set_error("%s: in-place operation is not supported", op); return SMALL_HIP_EINVAL; }
    if (act < SMALL_HIP_ACT_NONE || act > SMALL_HIP_ACT_LEAKY) { set_error("%s: bad activation", op); return SMALL_HIP_EINVAL; }
    if (act == SMALL_HIP_ACT_LEAKY && slope < 0.f)
    { set_error("%s: a negative slope is not monotone; issue the layers separately", op); return SMALL_HIP_EINVAL; }

    ConvArgs a{};
    a.in = in; a.filt = filt; a.bias = bias; a.out = out;
    a.batch = batch; a.Co = Co; a.Ci = Ci; a.H = H; a.W = W;
    a.kh = kh; a.kw = kw; a.stride = stride; a.pt = pt; a.pl = pl;
    a.stride_h = stride;
    a.Ho = out_dim(H, pt, pb, kh, stride);
    a.Wo = out_dim(W, pl, pr, kw, stride);
    a.act = act; a.slope = slope; a.accumulate = 0;
    if (a.Ho < 2 || a.Wo < 2) return SMALL_HIP_OK;        // no pooling window fits: empty output
    if ((long)Ci * H * W > 0x7fffffffL / 2 || (long)Ci * kh * kw * CB > 0x7fffffffL / 2)
    { set_error("%s: one image or one filter block too large for 32-bit offsets", op); return SMALL_HIP_EINVAL; }
    hipStream_t s = as_stream(stream);
    if (small_ci)
    {
        const int tiles_x = (a.Wo + 15) / 16, tiles_y = (a.Ho + 15) / 16;
        const long nt = (long)batch * tiles_x * tiles_y;
        if (nt > 0x7fffffffL) { set_error("%s: too many tiles for one launch", op); return SMALL_HIP_EINVAL; }
        a.P = batch * a.Ho * a.Wo;
        const int CoB = Co / CB;
        const int ncob = CoB % 4 == 0 ? 4 : CoB % 2 == 0 ? 2 : 1;
        const dim3 gs((unsigned)nt, (unsigned)(CoB / ncob));
        void (*ks)(const ConvArgs, int, int) = nullptr;
        // 16-byte staging when every image row is whole 16-byte pieces (416x416x3 -> 16 + pool, batch 16: 47.8 -> 43.8 us)
        static const bool vec_off = tune_int("stem_vec", 1) == 0;
        const bool vec = !vec_off && (W * Ci) % 4 == 0 && aligned16(in);
#define SHP_STEM_V(CI_, S_, V_) (ncob == 4 ? conv_stem3x3_lds_f32_kernel<CI_, S_, 4, true, V_> : ncob == 2 ? conv_stem3x3_lds_f32_kernel<CI_, S_, 2, true, V_> : conv_stem3x3_lds_f32_kernel<CI_, S_, 1, true, V_>)
#define SHP_STEM(CI_, S_) (vec ? SHP_STEM_V(CI_, S_, true) : SHP_STEM_V(CI_, S_, false))
        if (stride == 1) ks = Ci == 1 ? SHP_STEM(1, 1) : Ci == 2 ? SHP_STEM(2, 1) : SHP_STEM(3, 1);
        else ks = Ci == 1 ? SHP_STEM(1, 2) : Ci == 2 ? SHP_STEM(2, 2) : SHP_STEM(3, 2);
#undef SHP_STEM
#undef SHP_STEM_V
        hipLaunchKernelGGL(ks, gs, dim3(256), 0, s, a, tiles_x, tiles_y);
        SHP_LAUNCH_CHECK(op);
        return SMALL_HIP_OK;
    }
    // pixel tiles of 8 pooling windows; P = 4 x the number of windows
    const long nwin = (long)batch * (a.Ho / 2) * (a.Wo / 2);
    if (nwin > 0x7fffffffL / 16) { set_error("%s: too many pixels for one launch", op); return SMALL_HIP_EINVAL; }
    a.P = (int)(nwin * 4);
    const long ntiles = (nwin + 7) / 8;
    const long tiles32 = (long)((Co + 31) / 32) * ntiles;
    const long simds = 4L * NUM_CU;
    const int nsteps = kh * kw * (Ci / CB);
    if (Co % 64 == 0 && tiles32 >= 16 * simds && nsteps >= 32) launch_mfma_pool<2, 2>(a, s);
    else if (Co % 64 == 0 && tiles32 >= 4 * simds) launch_mfma_pool<2, 1>(a, s);
    else launch_mfma_pool<1, 1>(a, s);
    SHP_LAUNCH_CHECK(op);
    return SMALL_HIP_OK;
}

// First layer + bias + activation + DepthwiseConv2D 3x3 stride 1 (one pixel of padding) + bias + activation in one launch
int stem_dw_f32(const char *op, int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int dw_kh, int dw_kw,
                int dw_stride, int dpt, int dpb, int dpl, int dpr, int Co, int Ci, int H, int W, const float *in,
                const float *filt, const float *bias, const float *dw_filt, const float *dw_bias, int act, float slope,
                float *out, small_hip_stream_t stream)
{
    if (Ci != 1 && Ci != 2 && Ci != 3)
    { set_error("%s: only first layers (1-3 input channels) are fused with the depthwise layer", op); return SMALL_HIP_EINVAL; }
    if (stride != 1 && stride != 2) return SMALL_HIP_ESTRIDE;
    if (kh != 3 || kw != 3 || dw_kh != 3 || dw_kw != 3 || dw_stride != 1 || dpt != 1 || dpb != 1 || dpl != 1 || dpr != 1)
    { set_error("%s: fused for a 3x3 convolution followed by a 3x3 stride-1 depthwise convolution with padding 1", op); return SMALL_HIP_EINVAL; }
    if (batch <= 0 || H <= 0 || W <= 0 || Co <= 0 || !pads_ok(pt, pb, pl, pr)) { set_error("%s: bad size", op); return SMALL_HIP_EINVAL; }
    if (Co % CB != 0) { set_error("%s: output_channels must be a multiple of 16 (pad the filter)", op); return SMALL_HIP_EINVAL; }
    if (!in || !filt || !dw_filt || !out || !aligned16(filt) || !aligned16(dw_filt) || !aligned16(out) ||
        (bias && !aligned16(bias)) || (dw_bias && !aligned16(dw_bias)))
    { set_error("%s: null or misaligned pointer", op); return SMALL_HIP_EINVAL; }
    if (in == out) { set_error("%s: in-place operation is not supported", op); return SMALL_HIP_EINVAL; }
    if (act < SMALL_HIP_ACT_NONE || act > SMALL_HIP_ACT_LEAKY) { set_error("%s: bad activation", op); return SMALL_HIP_EINVAL; }

    ConvArgs a{};
    a.in = in; a.filt = filt; a.bias = bias; a.out = out;
    a.batch = batch; a.Co = Co; a.Ci = Ci; a.H = H; a.W = W;
    a.kh = 3; a.kw = 3; a.stride = stride; a.stride_h = stride; a.pt = pt; a.pl = pl;
    a.Ho = out_dim(H, pt, pb, 3, stride);
    a.Wo = out_dim(W, pl, pr, 3, stride);
    a.act = act; a.slope = slope; a.accumulate = 0;
    if (a.Ho <= 0 || a.Wo <= 0) return SMALL_HIP_OK;
    if ((long)Ci * H * W > 0x7fffffffL / 2) { set_error("%s: one image too large for 32-bit offsets", op); return SMALL_HIP_EINVAL; }
    const int tiles_x = (a.Wo + 13) / 14, tiles_y = (a.Ho + 13) / 14;
    const long nt = (long)batch * tiles_x * tiles_y;
    if (nt > 0x7fffffffL || (long)batch * Co * a.Ho * a.Wo > 0x7fffffffL * 4L)
    { set_error("%s: too many tiles for one launch", op); return SMALL_HIP_EINVAL; }
    a.P = batch * a.Ho * a.Wo;
    const int CoB = Co / CB;
    const int ncob = CoB % 2 == 0 ? 2 : 1;
    const StemDwArgs d{dw_filt, dw_bias};
    const dim3 gs((unsigned)nt, (unsigned)(CoB / ncob));
    void (*ks)(const ConvArgs, const StemDwArgs, int, int) = nullptr;
    const bool relu = act == SMALL_HIP_ACT_RELU;           // ReLU has its own instantiation: one instruction per value
#define SHP_SD_(CI_, S_, R_) (ncob == 2 ? conv_stem3x3_dw3x3_f32_kernel<CI_, S_, 2, R_> : conv_stem3x3_dw3x3_f32_kernel<CI_, S_, 1, R_>)
#define SHP_SD(CI_, S_) (relu ? SHP_SD_(CI_, S_, true) : SHP_SD_(CI_, S_, false))
    if (stride == 1) ks = Ci == 1 ? SHP_SD(1, 1) : Ci == 2 ? SHP_SD(2, 1) : SHP_SD(3, 1);
    else ks = Ci == 1 ? SHP_SD(1, 2) : Ci == 2 ? SHP_SD(2, 2) : SHP_SD(3, 2);
#undef SHP_SD
#undef SHP_SD_
    hipLaunchKernelGGL(ks, gs, dim3(256), 0, as_stream(stream), a, d, tiles_x, tiles_y);
    SHP_LAUNCH_CHECK(op);
    return SMALL_HIP_OK;
}

// Pointwise convolution + depthwise 3x3 in one launch (conv_pw_dw3x3_f32_kernel).
int pw_dw_f32(const char *op, int batch, int dw_stride, int dpt, int dpb, int dpl, int dpr, int Co, int Ci, int H, int W,
              const float *in, const float *filt, const float *bias, const float *dw_filt, const float *dw_bias, int act,
              float slope, float *out, small_hip_stream_t stream)
{
    if (dw_stride != 1 && dw_stride != 2) return SMALL_HIP_ESTRIDE;
    const int cib = Ci / CB;
    if (Ci % CB != 0 || !(cib == 1 || cib == 2 || cib == 3 || cib == 4 || cib == 6 || cib == 8) || Co % 32 != 0)
    { set_error("%s: the pointwise form is built for 16, 32, 48, 64, 96 or 128 input channels and output channels in whole groups of 32", op); return SMALL_HIP_EINVAL; }
    if (batch <= 0 || H <= 0 || W <= 0 || Co <= 0 || !pads_ok(dpt, dpb, dpl, dpr)) { set_error("%s: bad size", op); return SMALL_HIP_EINVAL; }
    if (!in || !filt || !dw_filt || !out || !aligned16(in) || !aligned16(filt) || !aligned16(dw_filt) || !aligned16(out) ||
        (bias && !aligned16(bias)) || (dw_bias && !aligned16(dw_bias)))
    { set_error("%s: null or misaligned pointer", op); return SMALL_HIP_EINVAL; }
    if (in == out) { set_error("%s: in-place operation is not supported", op); return SMALL_HIP_EINVAL; }
    if (act < SMALL_HIP_ACT_NONE || act > SMALL_HIP_ACT_LEAKY) { set_error("%s: bad activation", op); return SMALL_HIP_EINVAL; }
    ConvArgs a{};
    a.in = in; a.filt = filt; a.bias = bias; a.out = out;
    a.batch = batch; a.Co = Co; a.Ci = Ci; a.H = H; a.W = W; a.Ho = H; a.Wo = W;
    a.kh = 1; a.kw = 1; a.stride = 1; a.stride_h = 1;
    a.act = act; a.slope = slope;
    PwDwGeom g{};
    g.Hd = out_dim(H, dpt, dpb, 3, dw_stride);
    g.Wd = out_dim(W, dpl, dpr, 3, dw_stride);
    g.dpt = dpt; g.dpl = dpl;
    if (g.Hd <= 0 || g.Wd <= 0) return SMALL_HIP_OK;
    if ((long)Ci * H * W > 0x7fffffffL / 2) { set_error("%s: one image too large for 32-bit offsets", op); return SMALL_HIP_EINVAL; }
    const int toh = dw_stride == 1 ? PwDwTile<1>::TOH : PwDwTile<2>::TOH, tow = dw_stride == 1 ? PwDwTile<1>::TOW : PwDwTile<2>::TOW;
    g.tiles_x = (g.Wd + tow - 1) / tow; g.tiles_y = (g.Hd + toh - 1) / toh;
    const long nt = (long)batch * g.tiles_x * g.tiles_y;
    const StemDwArgs d{dw_filt, dw_bias};
    // channels per workgroup: 32 (four workgroups per compute unit) is measured ahead of 64 (two; the activation operand is
    // loaded once per 64 output channels) on every MobileNetV1 pair at batch 64, by 1-3 us.  SMALL_HIP_TUNE key pwdw_cot=1|2.
    int cot = 1;
    { static const int v = tune_int("pwdw_cot", 1); if (v == 1 || (v == 2 && Co % 64 == 0 && (cib == 2 || cib == 4 || cib == 8))) cot = v; }
    g.n_cg = Co / (32 * cot);
    if (nt * g.n_cg > 0x7fffffffL / 2) { set_error("%s: too many tiles for one launch", op); return SMALL_HIP_EINVAL; }
    g.n_wgs = (int)(nt * g.n_cg); g.per_xcd = (g.n_wgs + NUM_XCD - 1) / NUM_XCD;
    const dim3 grid(g.per_xcd * NUM_XCD);
    void (*k)(const ConvArgs, const StemDwArgs, const PwDwGeom) = nullptr;
#define SHP_PD_(S_, R_) (cot == 2 ? (cib == 2 ? conv_pw_dw3x3_f32_kernel<S_, 2, 2, R_> : cib == 4 ? conv_pw_dw3x3_f32_kernel<S_, 2, 4, R_> : conv_pw_dw3x3_f32_kernel<S_, 2, 8, R_>) \
                             : (cib == 1 ? conv_pw_dw3x3_f32_kernel<S_, 1, 1, R_> : cib == 2 ? conv_pw_dw3x3_f32_kernel<S_, 1, 2, R_> : cib == 3 ? conv_pw_dw3x3_f32_kernel<S_, 1, 3, R_> \
                                : cib == 4 ? conv_pw_dw3x3_f32_kernel<S_, 1, 4, R_> : cib == 6 ? conv_pw_dw3x3_f32_kernel<S_, 1, 6, R_> : conv_pw_dw3x3_f32_kernel<S_, 1, 8, R_>))
#define SHP_PD(S_) (relu ? SHP_PD_(S_, true) : SHP_PD_(S_, false))
    const bool relu = act == SMALL_HIP_ACT_RELU;           // ReLU has its own instantiation: one instruction per value
    k = dw_stride == 1 ? SHP_PD(1) : SHP_PD(2);
#undef SHP_PD_
#undef SHP_PD
    hipLaunchKernelGGL(k, grid, dim3(256), 0, as_stream(stream), a, d, g);
    SHP_LAUNCH_CHECK(op);
    return SMALL_HIP_OK;
}


} // namespace

extern "C" {

int small_hip_conv2d_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int Co, int Ci,
                         int H, int W, const float *in, const float *filt, float *out,
                         small_hip_stream_t stream)
{
    return conv_f32("small_hip_conv2d_f32", batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, filt,
                    nullptr, SMALL_HIP_ACT_NONE, 0.f, 0, out, stream);
}

int small_hip_partial_conv2d_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int Co,
                                 int Ci, int H, int W, const float *in, const float *filt, float *out,
                                 small_hip_stream_t stream)
{
    return conv_f32("small_hip_partial_conv2d_f32", batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in,
                    filt, nullptr, SMALL_HIP_ACT_NONE, 0.f, 1, out, stream);
}

int small_hip_conv2d_bias_act_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                                  int Co, int Ci, int H, int W, const float *in, const float *filt,
                                  const float *bias, int act, float slope, float *out,
                                  small_hip_stream_t stream)
{
    return conv_f32("small_hip_conv2d_bias_act_f32", batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in,
                    filt, bias, act, slope, 0, out, stream);
}

int small_hip_partial_conv2d_bias_act_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                                          int Co, int Ci, int H, int W, const float *in, const float *filt,
                                          const float *bias, int act, float slope, float *out,
                                          small_hip_stream_t stream)
{
    return conv_f32("small_hip_partial_conv2d_bias_act_f32", batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W,
                    in, filt, bias, act, slope, 1, out, stream);
}

int small_hip_conv2d_bias_act_maxpool2d_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                                            int pool_kh, int pool_kw, int pool_stride, int ppt, int ppb, int ppl,
                                            int ppr, int Co, int Ci, int H, int W, const float *in, const float *filt,
                                            const float *bias, int act, float slope, float *out,
                                            small_hip_stream_t stream)
{
    return conv_pool_f32("small_hip_conv2d_bias_act_maxpool2d_f32", batch, kh, kw, stride, pt, pb, pl, pr, pool_kh,
                         pool_kw, pool_stride, ppt, ppb, ppl, ppr, Co, Ci, H, W, in, filt, bias, act, slope, out, stream);
}

int small_hip_conv2d_bias_act_dwconv2d_bias_act_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                                                    int dw_kh, int dw_kw, int dw_stride, int dpt, int dpb, int dpl, int dpr,
                                                    int Co, int Ci, int H, int W, const float *in, const float *filt,
                                                    const float *bias, const float *dw_filt, const float *dw_bias, int act,
                                                    float slope, float *out, small_hip_stream_t stream)
{
    const char *op = "small_hip_conv2d_bias_act_dwconv2d_bias_act_f32";
    // a pointwise convolution of whole channel blocks in front of a 3x3 depthwise layer
    if (Ci > 3 && kh == 1 && kw == 1 && stride == 1 && pt == 0 && pb == 0 && pl == 0 && pr == 0 && dw_kh == 3 && dw_kw == 3)
        return pw_dw_f32(op, batch, dw_stride, dpt, dpb, dpl, dpr, Co, Ci, H, W, in, filt, bias, dw_filt, dw_bias, act, slope, out, stream);
    return stem_dw_f32(op, batch, kh, kw, stride, pt, pb, pl, pr, dw_kh, dw_kw,
                       dw_stride, dpt, dpb, dpl, dpr, Co, Ci, H, W, in, filt, bias, dw_filt, dw_bias, act, slope, out, stream);
}

size_t small_hip_conv2d_f32_workspace_bytes(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int Co, int Ci,
                                            int H, int W)
{
    if (batch <= 0 || kh <= 0 || kw <= 0 || Co <= 0 || Ci <= 0 || Ci % CB != 0 || Co % CB != 0 || (stride != 1 && stride != 2) ||
        !pads_ok(pt, pb, pl, pr))
        return 0;
    ConvArgs a{};
    a.Co = Co; a.Ci = Ci; a.kh = kh; a.kw = kw;
    const long P = (long)batch * out_dim(H, pt, pb, kh, stride) * out_dim(W, pl, pr, kw, stride);
    if (P <= 0 || P > 0x7fffffffL / 64) return 0;
    a.P = (int)P;
    if (wants_splitk((long)((Co + 31) / 32) * ((P + 31) / 32), kh * kw * (Ci / CB))) return 0;
    return streamk_plan<2, 1>(a);
}

int small_hip_conv2d_dwconv2d_one_launch_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int dw_kh,
                                             int dw_kw, int dw_stride, int dpt, int dpb, int dpl, int dpr, int Co, int Ci, int H,
                                             int W)
{
    if (batch <= 0 || H <= 0 || W <= 0 || Co <= 0 || Ci <= 0 || dw_kh != 3 || dw_kw != 3 || !pads_ok(pt, pb, pl, pr) ||
        !pads_ok(dpt, dpb, dpl, dpr) || (long)Ci * H * W > 0x7fffffffL / 2)
        return 0;
    if (Ci <= 3)
    {
        // a first layer on 16 x 16 tiles in front of a stride-1 depthwise layer with one pixel of padding (stem_dw_f32)
        if (kh != 3 || kw != 3 || (stride != 1 && stride != 2) || dw_stride != 1 || dpt != 1 || dpb != 1 || dpl != 1 || dpr != 1 ||
            Co % CB != 0)
            return 0;
        const long Ho = out_dim(H, pt, pb, 3, stride), Wo = out_dim(W, pl, pr, 3, stride);
        if (Ho <= 0 || Wo <= 0) return 0;
        const long nt = (long)batch * ((Wo + 13) / 14) * ((Ho + 13) / 14);
        return nt <= 0x7fffffffL && (long)batch * Co * Ho * Wo <= 0x7fffffffL * 4L ? 1 : 0;
    }
    // a pointwise convolution parked in LDS under 14 x 14 (stride 2: 7 x 8) depthwise tiles (pw_dw_f32): short reductions
    // on maps that fill those tiles to 70%, where the recomputed halo costs less than the second launch.  Measured on
    // MobileNetV1's pairs at batch 64: 32 -> 64 @112x112 stride 2 104 -> 54 us, 64 -> 128 @56x56 70 -> 54 us, 128 -> 256
    // @28x28 53 -> 46 us; 128 -> 128 @56x56 stride 2 81 -> 85 us (two launches stay)
    if (kh != 1 || kw != 1 || stride != 1 || pt || pb || pl || pr || Ci % CB != 0 || Co % 32 != 0 || (dw_stride != 1 && dw_stride != 2))
        return 0;
    const int cib = Ci / CB;
    if (!(cib <= 4 || ((cib == 6 || cib == 8) && dw_stride == 1))) return 0;
    const int Hd = out_dim(H, dpt, dpb, 3, dw_stride), Wd = out_dim(W, dpl, dpr, 3, dw_stride);
    if (Hd <= 0 || Wd <= 0) return 0;
    const int toh = dw_stride == 1 ? 14 : 7, tow = dw_stride == 1 ? 14 : 8;
    const long tx = (Wd + tow - 1) / tow, ty = (Hd + toh - 1) / toh;
    if (10L * Hd * Wd < 7 * (tx * tow) * (ty * toh)) return 0;
    if ((long)batch * tx * ty * (Co / 32) > 0x7fffffffL / 2) return 0;
    // the stand-alone convolution adds its products in one pass below eight K-steps; from eight on it may cut left-over
    // tiles along the input channels
    return cib < 8 ? 1 : 2;
}

int small_hip_conv2d_bias_act_dwconv2d_bias_act_via_f32(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                                                        int dw_kh, int dw_kw, int dw_stride, int dpt, int dpb, int dpl, int dpr,
                                                        int Co, int Ci, int H, int W, const float *in, const float *filt,
                                                        const float *bias, const float *dw_filt, const float *dw_bias, int act,
                                                        float slope, float *intermediate, float *out, small_hip_stream_t stream)
{
    const char *op = "small_hip_conv2d_bias_act_dwconv2d_bias_act_via_f32";
    if (!intermediate || !in || !out) { set_error("%s: null tensor", op); return SMALL_HIP_EINVAL; }
    {
        // whichever form runs, no tensor may be written while another launch or workgroup still reads it
        const long Ho = out_dim(H, pt, pb, kh, stride > 0 ? stride : 1), Wo = out_dim(W, pl, pr, kw, stride > 0 ? stride : 1);
        const long Hd = out_dim((int)Ho, dpt, dpb, dw_kh, dw_stride > 0 ? dw_stride : 1), Wd = out_dim((int)Wo, dpl, dpr, dw_kw, dw_stride > 0 ? dw_stride : 1);
        if (batch > 0 && Ci > 0 && Co > 0 && H > 0 && W > 0 && Ho > 0 && Wo > 0 && Hd > 0 && Wd > 0)
        {
            const size_t n_in = (size_t)batch * Ci * H * W, n_mid = (size_t)batch * Co * Ho * Wo, n_out = (size_t)batch * Co * Hd * Wd;
            auto overlap = [](const float *p, size_t n, const float *q, size_t m) { return p < q + m && q < p + n; };
            if (overlap(in, n_in, intermediate, n_mid) || overlap(in, n_in, out, n_out) || overlap(intermediate, n_mid, out, n_out))
            { set_error("%s: input, intermediate and output tensors must not overlap", op); return SMALL_HIP_EINVAL; }
        }
    }
    // SMALL_HIP_TUNE key fuse_form=3: always the two layers (read per call: tests switch it)
    if (tune_int("fuse_form", 0) != 3 &&
        small_hip_conv2d_dwconv2d_one_launch_f32(batch, kh, kw, stride, pt, pb, pl, pr, dw_kh, dw_kw, dw_stride, dpt, dpb, dpl, dpr, Co, Ci, H, W))
        return small_hip_conv2d_bias_act_dwconv2d_bias_act_f32(batch, kh, kw, stride, pt, pb, pl, pr, dw_kh, dw_kw, dw_stride, dpt, dpb, dpl,
                                                               dpr, Co, Ci, H, W, in, filt, bias, dw_filt, dw_bias, act, slope, out, stream);
    // the two layers, one after the other
    if (int rc = conv_f32(op, batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, filt, bias, act, slope, 0, intermediate, stream)) return rc;
    const int Ho = out_dim(H, pt, pb, kh, stride), Wo = out_dim(W, pl, pr, kw, stride);
    if (Ho <= 0 || Wo <= 0) return SMALL_HIP_OK;
    return small_hip_depthwise_conv2d_bias_act_f32(batch, dw_kh, dw_kw, dw_stride, dpt, dpb, dpl, dpr, Co, Ho, Wo, intermediate, dw_filt,
                                                   dw_bias, act, slope, out, stream);
}

// One convolution of `channels` -> `channels` per slab of `channels` channels; slab g of image n starts
// (n * groups + g) * channels * H * W elements into the input (the same with Ho * Wo into the output) and
// uses filter block g.  ONE launch: the (image, group) slab is the grid's second dimension, every slab is a
// batch-1 convolution of `channels` channels at its own offsets with its group's filter block.
static int group_conv_f32(const char *op, int batch, int kh, int kw, int stride, int stride_h, int groups, int pt, int pb, int pl,
                          int pr, int channels, int H, int W, const float *in, const float *filt, int accumulate, float *out,
                          small_hip_stream_t stream)
{
    if (channels <= 0 || channels % CB != 0) return SMALL_HIP_ECHANNELS;
    if (stride != 1 && stride != 2) return SMALL_HIP_ESTRIDE;
    if (batch <= 0 || groups <= 0 || kh <= 0 || kw <= 0 || H <= 0 || W <= 0 || !pads_ok(pt, pb, pl, pr))
    { set_error("%s: bad size", op); return SMALL_HIP_EINVAL; }
    if (!in || !filt || !out) { set_error("%s: null pointer", op); return SMALL_HIP_EINVAL; }
    const size_t in_slab = (size_t)channels * H * W;
    const size_t out_slab = (size_t)channels * out_dim(H, pt, pb, kh, stride_h ? stride_h : stride) * out_dim(W, pl, pr, kw, stride);
    const size_t slabs = (size_t)batch * groups;
    // the slabs written must not overlap the slabs read (one slab's workgroups would read another's output)
    if (in + slabs * in_slab > out && out + slabs * out_slab > in)
    { set_error("%s: in-place convolution is not supported", op); return SMALL_HIP_EINVAL; }
    // one launch for up to 65535 slabs: the slab is the grid's second dimension
    for (size_t i = 0; i < slabs; i += 65535)
    {
        GroupSlabs g;
        g.slabs = (int)(slabs - i < 65535 ? slabs - i : 65535);
        g.groups = groups;
        g.slab0 = (int)(i % (size_t)groups);
        g.stride_h = stride_h;
        const int rc = conv_f32(op, 1, kh, kw, stride, pt, pb, pl, pr, channels, channels, H, W, in + i * in_slab, filt,
                                nullptr, SMALL_HIP_ACT_NONE, 0.f, accumulate ? 1 : 0, out + i * out_slab, stream, g);
        if (rc != SMALL_HIP_OK) return rc;
    }
    return SMALL_HIP_OK;
}

int small_hip_group_conv2d_f32(int batch, int kh, int kw, int stride, int groups, int pt, int pb, int pl, int pr,
                               int channels, int H, int W, const float *in, const float *filt, int accumulate,
                               float *out, small_hip_stream_t stream)
{
    return group_conv_f32("small_hip_group_conv2d_f32", batch, kh, kw, stride, 0, groups, pt, pb, pl, pr, channels, H, W, in,
                          filt, accumulate, out, stream);
}

// The 1-D convolutions (interface_abstract_1D.hpp:47-560, 1255-1450): `rows` independent signals of `width` samples in
// one [C/16][rows][width][16] tensor, a 1 x k window moved by `stride` along the width only.  groups == 0: Conv1D /
// PartialConv1D (accumulate) with optional bias and activation; groups > 0: GroupConv1D / PartialGroupConv1D of
// input_channels -> input_channels per group (output_channels, bias and activation are not used).
int small_hip_conv1d_f32(int batch, int k, int stride, int l_pad, int r_pad, int groups, int Co, int Ci, int rows, int width,
                         const float *in, const float *filt, const float *bias, int act, float slope, int accumulate,
                         float *out, small_hip_stream_t stream)
{
    if (groups > 0)
        return group_conv_f32("small_hip_conv1d_f32", batch, 1, k, stride, 1, groups, 0, 0, l_pad, r_pad, Ci, rows, width, in, filt,
                              accumulate, out, stream);
    GroupSlabs g;
    g.stride_h = 1;
    return conv_f32("small_hip_conv1d_f32", batch, 1, k, stride, 0, 0, l_pad, r_pad, Co, Ci, rows, width, in, filt, bias, act,
                    slope, accumulate ? 1 : 0, out, stream, g);
}

int small_hip_dense_f32(int batch, int No, int Ni, const float *in, const float *filt, float *out,
                        small_hip_stream_t stream)
{
    return conv_f32("small_hip_dense_f32", batch, 1, 1, 1, 0, 0, 0, 0, No, Ni, 1, 1, in, filt, nullptr,
                    SMALL_HIP_ACT_NONE, 0.f, 0, out, stream);
}

} // extern "C"
