// Whole-model forward pass of a small float32 CNN in ONE launch for gfx950 (small_hip_fmodel_*).
//
// A keyword-spotting DS-CNN (49x10x1 input, 25x5x64 activations = 32 KB, 87 KB of weights) run layer by layer is
// eleven dependent launches that each sit at the launch-latency floor.  Here one workgroup of 1024 threads owns one
// image from input to logits: the activation tensors stay in the compute unit's LDS, each layer's weights are
// brought into LDS one layer ahead (double buffered, global memory to LDS directly), only the image and the model's output touch global memory and
// the layers are separated by workgroup barriers instead of kernel boundaries.
//
// Layers (the functions of include/small/interface_abstract.hpp on float buffers, fused as Conv2DLayer /
// DepthwiseConv2DLayer::compute_output issue them: bias, convolution, ReLU or LeakyReLU):
//   convolution, input channels % 16 == 0   v_mfma_f32_16x16x4_f32, rows = 16 output channels, columns = 16 pixels
//   convolution, 1..3 input channels        the same instruction on a gathered patch (model input only)
//   depthwise convolution                   vector ALU, a lane = 4 channels of one output pixel
//   depthwise 3x3 -> 1x1 convolution        one layer: a lane's depthwise results ARE its MFMA operand of the 1x1
//                                           convolution (the same pixel, the same four channels), so the depthwise
//                                           tensor is never stored and its arithmetic issues between the MFMAs
//   whole-image average / max pooling       a wave per channel quad: lanes fold pixels, then xor-shuffles (deterministic)
// A fully connected layer is the 1x1 convolution on the 1x1 image pooling leaves.
//
// LDS layout of an activation tensor: [C/16][P][16] floats, the four channel quads of pixel p stored in the order
// q ^ ((p >> 1) & 3).  An MFMA operand read is one 16-byte read per lane at a 64-byte pixel pitch; with that swizzle
// eight neighbouring pixels cover all 32 banks, without it they would share two.  One such read feeds four MFMAs:
// lane (pixel, kq) holds channels 4kq .. 4kq+3, MFMA j of the step contracts channels {j, 4+j, 8+j, 12+j}, and the
// filter is re-ordered once, when the model is created, so that the matching four weights are one 16-byte read too:
//   Wt[co block][tap][ci block][kq][co % 16][j] = F[co][ci = 16 * block + 4 kq + j][tap].
// Numerics: float32 MFMA accumulation, bias added and activation applied on the accumulators.
#include "common.h"

#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

using namespace shp;

namespace
{

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int NT = 1024;                 // 16 waves, 4 per SIMD; one workgroup per compute unit (LDS)
constexpr int NW = NT / WAVE;
constexpr int MAX_LAYERS = 32;
constexpr int MAX_TENSORS = 8;
constexpr int NPRE = 3;                  // 16-byte pieces of the next layer's weights a thread carries: 48 KB per layer
constexpr int LDS_LIMIT = 160 * 1024;

enum { K_STEM = 0, K_CONV = 1, K_DW = 2, K_POOL_AVG = 3, K_POOL_MAX = 4, K_DWPW = 5 };

struct FMLayer
{
    int kind;
    int src_off, dst_off;                // float offsets in LDS; dst_off < 0: the model output in global memory
    int Ci, Co, H, W, Ho, Wo, kh, kw, stride, pt, pl;
    int K, chunks;                       // first layer: reduction length kh*kw*Ci and its chunks of 16 (four MFMA steps)
    int blob_off, blob16;                // the layer's weights in the blob (float offset) and their size in 16-byte pieces
    int next_blob_off, next_blob16;      // the same of the layer after this one (0 pieces after the last): read with this record
    int bias_off, ktab_off;              // float offsets inside the layer's weights
    float nscale;                        // what a negative result is multiplied by: 1 none, 0 ReLU, slope LeakyReLU
    float r_wo, r_cob, r_p, norm;        // 1 / Wo, 1 / (Co / 16), 1 / (Ho * Wo), pooling scale
    // K_DWPW: a 3x3 depthwise convolution whose result feeds the 1x1 convolution that follows without leaving registers
    int Co2, w2_off, bias2_off;          // the 1x1 convolution: output channels, weights and bias inside the layer's weights
    float nscale2, r_cob2;               // ... and 1 / (Co2 / 16)
};

struct FMHeader
{
    int n_layers;
    int in_C, in_H, in_W, in_off;        // the model input and the LDS float offset it is staged at
    int w_lds, w_floats;                 // weights: two buffers of w_floats floats at float offset w_lds
    int pool_off;                        // 4096 + 512 floats of pooling partials
    int zero_off;                        // 16 bytes of zeros: what a tap outside the image reads
    int in_elems, out_elems;             // floats per image in global memory
    int lds_bytes;
    FMLayer layer[MAX_LAYERS];
};
typedef const __attribute__((address_space(4))) FMHeader *HeaderPtr;

__device__ __forceinline__ FMLayer load_layer(HeaderPtr hdr, int li)
{
    FMLayer L;
    __builtin_memcpy(&L, &hdr->layer[li], sizeof(FMLayer));
    return L;
}

// float offset of channel quad q of pixel p in a [C/16][P][16] tensor
__device__ __forceinline__ int apos(int cb, int P, int p, int q) { return ((cb * P + p) * 4 + (q ^ ((p >> 1) & 3))) * 4; }

__device__ __forceinline__ float act_bf(float v, float neg_scale)
{
    const float n = fmaf(v, neg_scale, 0.f);      // "+ 0": the -0 of x * 0 becomes the +0 ReLU gives
    return v > 0.f ? v : n;
}

// ---- model creation: weights into operand order ---------------------------------------------------------------
// kind K_CONV: packed filter [Co/16][Ci/16][taps][16 ci][16 co] -> Wt[Co/16][taps][Ci/16][kq][co16][j]
// kind K_STEM: packed filter [Co/16][K][16 co] -> Wt[Co/16][chunk][kq][co16][j] = F[k = 16 chunk + 4 j + kq], zero from K on
// kind K_DW:   packed filter [C/16][taps][16] unchanged
// followed by the bias (zeros without one)
__global__ __launch_bounds__(256) void fm_prep_kernel(int kind, const float *__restrict__ f, const float *__restrict__ bias,
                                                      float *__restrict__ dst, int Co, int Ci, int taps, int K, int chunks,
                                                      int w_floats)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < w_floats)
    {
        float v = 0.f;
        if (kind == K_CONV)
        {
            const int CiB = Ci / CB;
            const int j = i & 3, co16 = (i >> 2) & 15, kq = (i >> 6) & 3;
            int r = i >> 8;
            const int cib = r % CiB; r /= CiB;
            const int tap = r % taps, cob = r / taps;
            v = f[((((size_t)cob * CiB + cib) * taps + tap) * CB + 4 * kq + j) * CB + co16];
        }
        else if (kind == K_STEM)
        {
            const int j = i & 3, co16 = (i >> 2) & 15, kq = (i >> 6) & 3, r = i >> 8;
            const int chunk = r % chunks, cob = r / chunks, k = 16 * chunk + 4 * j + kq;
            if (k < K) v = f[((size_t)cob * K + k) * CB + co16];
        }
        else
            v = f[i];
        dst[i] = v;
    }
    if (i < Co) dst[w_floats + i] = bias ? bias[i] : 0.f;
}

// ---- device: layers --------------------------------------------------------------------------------------------
// Convolution on MFMA; TP pixel tiles of one channel block per wave step share the filter operand.  The K-steps
// (tap, input channel block) are taken four at a time: all twelve (TP = 2) operand reads of a chunk are issued before
// its first MFMA, so a chunk pays the LDS latency once; a tap outside the image reads the block of zeros.
template <int TP>
__device__ __forceinline__ void conv_layer(const FMLayer &L, float *lds, const float *wl, const float *zero, float *gout,
                                           int wave, int lane)
{
    const int col = lane & 15, kq = lane >> 4;
    const int CoB = L.Co / CB, CiB = L.Ci / CB, S = L.kh * L.kw * CiB;
    const int Pin = L.H * L.W, P = L.Ho * L.Wo;
    const int n_pt = (P + 15) >> 4, n_grp = (n_pt + TP - 1) / TP, n_work = n_grp * CoB;
    const float *src = lds + L.src_off;
    for (int work = wave; work < n_work; work += NW)
    {
        const int pg = (int)(((float)work + 0.5f) * L.r_cob);
        const int cob = work - pg * CoB;
        int ih0[TP], iw0[TP], p[TP];
        bool pv[TP];
#pragma unroll
        for (int t = 0; t < TP; ++t)
        {
            p[t] = (pg * TP + t) * 16 + col;
            pv[t] = p[t] < P;
            const int pc = pv[t] ? p[t] : 0;
            const int oh = (int)(((float)pc + 0.5f) * L.r_wo), ow = pc - oh * L.Wo;
            ih0[t] = oh * L.stride - L.pt;
            iw0[t] = ow * L.stride - L.pl;
        }
        floatx4 acc[TP];
#pragma unroll
        for (int t = 0; t < TP; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
        const float *wrow = wl + ((cob * S * 4 + kq) * 16 + col) * 4;
        int a = 0, b = 0, cib = 0;                       // the next step to load (uniform)
        for (int s0 = 0; s0 < S; s0 += 4)
        {
            float4 A[4], B[TP][4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                const bool live = s0 + u < S;            // uniform
                A[u] = *reinterpret_cast<const float4 *>(live ? wrow + (s0 + u) * 256 : zero);
#pragma unroll
                for (int t = 0; t < TP; ++t)
                {
                    const int ih = ih0[t] + a, iw = iw0[t] + b;
                    const bool ok = live && pv[t] && (unsigned)ih < (unsigned)L.H && (unsigned)iw < (unsigned)L.W;
                    B[t][u] = *reinterpret_cast<const float4 *>(ok ? src + apos(cib, Pin, ih * L.W + iw, kq) : zero);
                }
                // channel block fastest, then the window column, then the row
                const bool w1 = cib + 1 == CiB;
                cib = w1 ? 0 : cib + 1;
                const bool w2 = w1 && b + 1 == L.kw;
                b = w2 ? 0 : b + (w1 ? 1 : 0);
                a += w2 ? 1 : 0;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                const float Av[4] = {A[u].x, A[u].y, A[u].z, A[u].w};
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int t = 0; t < TP; ++t)
                    {
                        const float Bv[4] = {B[t][u].x, B[t][u].y, B[t][u].z, B[t][u].w};
                        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(Av[j], Bv[j], acc[t], 0, 0, 0);
                    }
            }
        }
        const float4 bias = *reinterpret_cast<const float4 *>(wl + L.bias_off + cob * CB + 4 * kq);
#pragma unroll
        for (int t = 0; t < TP; ++t)
        {
            if (!pv[t]) continue;
            const float4 v = make_float4(act_bf(acc[t][0] + bias.x, L.nscale), act_bf(acc[t][1] + bias.y, L.nscale),
                                         act_bf(acc[t][2] + bias.z, L.nscale), act_bf(acc[t][3] + bias.w, L.nscale));
            if (L.dst_off >= 0) *reinterpret_cast<float4 *>(lds + L.dst_off + apos(cob, P, p[t], kq)) = v;
            else *reinterpret_cast<float4 *>(gout + ((size_t)cob * P + p[t]) * CB + 4 * kq) = v;
        }
    }
}

// first layer, 1..3 input channels: the image lies in LDS as it does in memory, [H][W][Ci]; reduction element
// k = (a * kw + b) * Ci + ci.  In MFMA step 4 * chunk + j lane (pixel, kq) supplies element k = 16 chunk + 4 j + kq of
// its pixel's patch; where that element lies comes from a table written with the weights (one 16-byte read per
// chunk), and the gathered operand serves TC output-channel blocks.
template <int TC>
__device__ __forceinline__ void stem_layer(const FMLayer &L, float *lds, const float *wl, const float *zero, float *gout,
                                           int wave, int lane)
{
    const int col = lane & 15, kq = lane >> 4;
    const int CoB = L.Co / CB, P = L.Ho * L.Wo;
    const int n_pt = (P + 15) >> 4, n_cg = CoB / TC, n_work = n_pt * n_cg;
    const float r_ncg = L.r_cob * (float)TC;                 // 1 / n_cg
    const float *src = lds + L.src_off;
    const int4 *ktab = reinterpret_cast<const int4 *>(wl + L.ktab_off);
    for (int work = wave; work < n_work; work += NW)
    {
        const int pt = (int)(((float)work + 0.5f) * r_ncg), cg = work - pt * n_cg;
        const int p = pt * 16 + col;
        const bool pv = p < P;
        const int pc = pv ? p : 0;
        const int oh = (int)(((float)pc + 0.5f) * L.r_wo), ow = pc - oh * L.Wo;
        const int ih0 = oh * L.stride - L.pt, iw0 = ow * L.stride - L.pl;
        floatx4 acc[TC];
#pragma unroll
        for (int c = 0; c < TC; ++c) acc[c] = floatx4{0.f, 0.f, 0.f, 0.f};
        // the operands of chunk ch: where its four patch elements lie (table), the elements, the filter quads
        auto gather = [&](int ch, float4 (&A)[TC], float (&bv)[4]) {
            const int4 e4 = ktab[ch * 4 + kq];               // a | b << 8 | ci << 16 per step; -1 past the end
            const int ev[4] = {e4.x, e4.y, e4.z, e4.w};
#pragma unroll
            for (int c = 0; c < TC; ++c)
                A[c] = *reinterpret_cast<const float4 *>(wl + ((((cg * TC + c) * L.chunks + ch) * 4 + kq) * 16 + col) * 4);
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                const int e = ev[j];
                const int ih = ih0 + (e & 255), iw = iw0 + ((e >> 8) & 255);
                const bool ok = pv && e >= 0 && (unsigned)ih < (unsigned)L.H && (unsigned)iw < (unsigned)L.W;
                bv[j] = *(ok ? src + (ih * L.W + iw) * L.Ci + (e >> 16) : zero);
            }
        };
        auto multiply = [&](const float4 (&A)[TC], const float (&bv)[4]) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int c = 0; c < TC; ++c)
                {
                    const float Av[4] = {A[c].x, A[c].y, A[c].z, A[c].w};
                    acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(Av[j], bv[j], acc[c], 0, 0, 0);
                }
        };
        // chunk ch + 1 is gathered between the MFMAs of chunk ch (a wave issues in order: see dwpw_layer)
        float4 Ac[TC], An[TC];
        float bc[4], bn[4];
        gather(0, Ac, bc);
        for (int ch = 0; ch + 1 < L.chunks; ++ch)
        {
            gather(ch + 1, An, bn);
            multiply(Ac, bc);
#pragma unroll
            for (int c = 0; c < TC; ++c) Ac[c] = An[c];
#pragma unroll
            for (int j = 0; j < 4; ++j) bc[j] = bn[j];
#pragma unroll
            for (int g = 0; g < 4 * TC; ++g)
            {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);
            }
        }
        multiply(Ac, bc);
        if (!pv) continue;
#pragma unroll
        for (int c = 0; c < TC; ++c)
        {
            const int cob = cg * TC + c;
            const float4 bias = *reinterpret_cast<const float4 *>(wl + L.bias_off + cob * CB + 4 * kq);
            const float4 v = make_float4(act_bf(acc[c][0] + bias.x, L.nscale), act_bf(acc[c][1] + bias.y, L.nscale),
                                         act_bf(acc[c][2] + bias.z, L.nscale), act_bf(acc[c][3] + bias.w, L.nscale));
            if (L.dst_off >= 0) *reinterpret_cast<float4 *>(lds + L.dst_off + apos(cob, P, p, kq)) = v;
            else *reinterpret_cast<float4 *>(gout + ((size_t)cob * P + p) * CB + 4 * kq) = v;
        }
    }
}

// Depthwise convolution with a compile-time window: a lane owns 4 channels of one output pixel and walks over a
// share of the channel blocks.  The window's nine positions (offsets into the block, the zeros for taps outside the
// image) are worked out once per lane; per channel block a tap costs two 16-byte LDS reads and four multiply-adds.
template <int KH, int KW>
__device__ __forceinline__ void dw_layer_win(const FMLayer &L, float *lds, const float *wl, const float *zero, float *gout, int tid)
{
    constexpr int T = KH * KW;
    const int CiB = L.Ci / CB;
    const int Pin = L.H * L.W, P = L.Ho * L.Wo, n_lane = P * 4;
    int G = NT / n_lane;                                   // lane groups along the channel blocks
    G = G < 1 ? 1 : (G > CiB ? CiB : G);
    const int per = (CiB + G - 1) / G;                     // channel blocks per group
    const float *src = lds + L.src_off;
    for (int i = tid; i < n_lane * G; i += NT)
    {
        const int g = (int)(((float)i + 0.5f) * L.r_p * 0.25f);      // i / n_lane
        const int r = i - g * n_lane;
        const int q = r & 3, p = r >> 2;
        const int oh = (int)(((float)p + 0.5f) * L.r_wo), ow = p - oh * L.Wo;
        const int ih0 = oh * L.stride - L.pt, iw0 = ow * L.stride - L.pl;
        const int cb0 = g * per, cb1 = cb0 + per < CiB ? cb0 + per : CiB;
        const float *xp[T];
        int xstep[T];
#pragma unroll
        for (int a = 0; a < KH; ++a)
#pragma unroll
            for (int b = 0; b < KW; ++b)
            {
                const int ih = ih0 + a, iw = iw0 + b;
                const bool ok = (unsigned)ih < (unsigned)L.H && (unsigned)iw < (unsigned)L.W;
                xp[a * KW + b] = ok ? src + apos(cb0, Pin, ih * L.W + iw, q) : zero;
                xstep[a * KW + b] = ok ? Pin * CB : 0;
            }
        const float *w = wl + cb0 * T * CB + 4 * q;
        const float *bp = wl + L.bias_off + cb0 * CB + 4 * q;
        int dpos = apos(cb0, P, p, q);
        for (int cb = cb0; cb < cb1; ++cb)
        {
            float4 x[T], k[T];
#pragma unroll
            for (int t = 0; t < T; ++t)
            {
                x[t] = *reinterpret_cast<const float4 *>(xp[t]);
                k[t] = *reinterpret_cast<const float4 *>(w + t * CB);
                xp[t] += xstep[t];
            }
            float4 acc = *reinterpret_cast<const float4 *>(bp);
#pragma unroll
            for (int t = 0; t < T; ++t)
            {
                acc.x = fmaf(x[t].x, k[t].x, acc.x); acc.y = fmaf(x[t].y, k[t].y, acc.y);
                acc.z = fmaf(x[t].z, k[t].z, acc.z); acc.w = fmaf(x[t].w, k[t].w, acc.w);
            }
            acc.x = act_bf(acc.x, L.nscale); acc.y = act_bf(acc.y, L.nscale);
            acc.z = act_bf(acc.z, L.nscale); acc.w = act_bf(acc.w, L.nscale);
            if (L.dst_off >= 0) *reinterpret_cast<float4 *>(lds + L.dst_off + dpos) = acc;
            else *reinterpret_cast<float4 *>(gout + ((size_t)cb * P + p) * CB + 4 * q) = acc;
            w += T * CB; bp += CB; dpos += P * CB;
        }
    }
}

// Depthwise 3x3 + activation feeding a 1x1 convolution + activation.  In the MFMA operand layout lane (pixel, kq) supplies
// channels 4kq .. 4kq+3 of its pixel for each input-channel block: exactly one depthwise result quad.  So the wave
// computes the block's depthwise quad on the vector ALU (nine 16-byte reads of the input, nine of the taps, 36
// multiply-adds) while the MFMAs of the previous block run, and hands it to the MFMAs of all TC output-channel blocks.
// The depthwise tensor never exists in memory, and a layer boundary (barrier, LDS round trip) disappears.
template <int TC>
__device__ __forceinline__ void dwpw_layer(const FMLayer &L, float *lds, const float *wl, const float *zero, float *gout,
                                           int wave, int lane)
{
    constexpr int T = 9;
    const int col = lane & 15, kq = lane >> 4;
    const int CiB = L.Ci / CB, CoB = L.Co2 / CB;
    const int Pin = L.H * L.W, P = L.Ho * L.Wo;
    const int n_pt = (P + 15) >> 4, n_cg = CoB / TC, n_work = n_pt * n_cg;
    const float r_ncg = L.r_cob2 * (float)TC;                // 1 / n_cg
    const float *src = lds + L.src_off;
    for (int work = wave; work < n_work; work += NW)
    {
        const int pt = (int)(((float)work + 0.5f) * r_ncg), cg = work - pt * n_cg;
        const int p = pt * 16 + col;
        const bool pv = p < P;
        const int pc = pv ? p : 0;
        const int oh = (int)(((float)pc + 0.5f) * L.r_wo), ow = pc - oh * L.Wo;
        const int ih0 = oh * L.stride - L.pt, iw0 = ow * L.stride - L.pl;
        const float *xp[T];
        int xstep[T];
#pragma unroll
        for (int a = 0; a < 3; ++a)
#pragma unroll
            for (int b = 0; b < 3; ++b)
            {
                const int ih = ih0 + a, iw = iw0 + b;
                const bool ok = pv && (unsigned)ih < (unsigned)L.H && (unsigned)iw < (unsigned)L.W;
                xp[a * 3 + b] = ok ? src + apos(0, Pin, ih * L.W + iw, kq) : zero;
                xstep[a * 3 + b] = ok ? Pin * CB : 0;
            }
        const float *wk = wl + 4 * kq;                       // depthwise taps [ci block][tap][16]
        const float *bk = wl + L.bias_off + 4 * kq;
        // the depthwise quad of the next input-channel block (advances the pointers)
        auto depthwise = [&]() -> float4 {
            float4 acc = *reinterpret_cast<const float4 *>(bk);
#pragma unroll
            for (int t = 0; t < T; ++t)
            {
                const float4 x = *reinterpret_cast<const float4 *>(xp[t]);
                const float4 k = *reinterpret_cast<const float4 *>(wk + t * CB);
                acc.x = fmaf(x.x, k.x, acc.x); acc.y = fmaf(x.y, k.y, acc.y);
                acc.z = fmaf(x.z, k.z, acc.z); acc.w = fmaf(x.w, k.w, acc.w);
                xp[t] += xstep[t];
            }
            wk += T * CB; bk += CB;
            return make_float4(act_bf(acc.x, L.nscale), act_bf(acc.y, L.nscale), act_bf(acc.z, L.nscale), act_bf(acc.w, L.nscale));
        };
        floatx4 acc[TC];
#pragma unroll
        for (int c = 0; c < TC; ++c) acc[c] = floatx4{0.f, 0.f, 0.f, 0.f};
        const float *arow = wl + L.w2_off + ((cg * TC * CiB * 4 + kq) * 16 + col) * 4;      // + (c * CiB + cib) * 256
        auto filter = [&](int cib, float4 (&A)[TC]) {
#pragma unroll
            for (int c = 0; c < TC; ++c) A[c] = *reinterpret_cast<const float4 *>(arow + (c * CiB + cib) * 256);
        };
        auto multiply = [&](const float4 (&A)[TC], const float4 Bq) {
            const float Bv[4] = {Bq.x, Bq.y, Bq.z, Bq.w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int c = 0; c < TC; ++c)
                {
                    const float Av[4] = {A[c].x, A[c].y, A[c].z, A[c].w};
                    acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(Av[j], Bv[j], acc[c], 0, 0, 0);
                }
        };
        // Software pipeline over the input-channel blocks: while the MFMAs of block cib run, the wave reads the filter
        // of block cib + 1 and does that block's depthwise arithmetic.  A wave issues in order, so the overlap only
        // happens if those instructions sit BETWEEN the MFMAs: the scheduling groups below ask for one MFMA, then a
        // couple of LDS reads and a handful of vector instructions, sixteen times (an MFMA occupies the matrix pipe for
        // 32 cycles = 8 issue slots).
        float4 Ac[TC], An[TC];
        filter(0, Ac);
        float4 Bc = depthwise();
        for (int cib = 0; cib + 1 < CiB; ++cib)
        {
            filter(cib + 1, An);
            multiply(Ac, Bc);
            Bc = depthwise();
#pragma unroll
            for (int c = 0; c < TC; ++c) Ac[c] = An[c];
#pragma unroll
            for (int g = 0; g < 4 * TC; ++g)
            {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);      // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);      // LDS reads
                __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);      // vector ALU
            }
        }
        multiply(Ac, Bc);
        if (!pv) continue;
#pragma unroll
        for (int c = 0; c < TC; ++c)
        {
            const int cob = cg * TC + c;
            const float4 bias = *reinterpret_cast<const float4 *>(wl + L.bias2_off + cob * CB + 4 * kq);
            const float4 v = make_float4(act_bf(acc[c][0] + bias.x, L.nscale2), act_bf(acc[c][1] + bias.y, L.nscale2),
                                         act_bf(acc[c][2] + bias.z, L.nscale2), act_bf(acc[c][3] + bias.w, L.nscale2));
            if (L.dst_off >= 0) *reinterpret_cast<float4 *>(lds + L.dst_off + apos(cob, P, p, kq)) = v;
            else *reinterpret_cast<float4 *>(gout + ((size_t)cob * P + p) * CB + 4 * kq) = v;
        }
    }
}

// depthwise convolution, any window: a lane = one output pixel x 4 channels of one block
__device__ __forceinline__ void dw_layer_any(const FMLayer &L, float *lds, const float *wl, float *gout, int tid)
{
    const int kh = L.kh, kw = L.kw;
    const int Pin = L.H * L.W, P = L.Ho * L.Wo, n = (L.Ci / CB) * P * 4;
    const float *src = lds + L.src_off;
    for (int i = tid; i < n; i += NT)
    {
        const int q = i & 3, r = i >> 2;
        const int cb = (int)(((float)r + 0.5f) * L.r_p), p = r - cb * P;
        const int oh = (int)(((float)p + 0.5f) * L.r_wo), ow = p - oh * L.Wo;
        const int ih0 = oh * L.stride - L.pt, iw0 = ow * L.stride - L.pl;
        const float *w = wl + cb * kh * kw * CB + 4 * q;
        float4 acc = *reinterpret_cast<const float4 *>(wl + L.bias_off + cb * CB + 4 * q);
        for (int a = 0; a < kh; ++a)
            for (int b = 0; b < kw; ++b)
            {
                const int ih = ih0 + a, iw = iw0 + b;
                const bool ok = (unsigned)ih < (unsigned)L.H && (unsigned)iw < (unsigned)L.W;
                float4 x = *reinterpret_cast<const float4 *>(src + apos(cb, Pin, ok ? ih * L.W + iw : 0, q));
                if (!ok) x = make_float4(0.f, 0.f, 0.f, 0.f);
                const float4 k = *reinterpret_cast<const float4 *>(w + (a * kw + b) * CB);
                acc.x = fmaf(x.x, k.x, acc.x); acc.y = fmaf(x.y, k.y, acc.y);
                acc.z = fmaf(x.z, k.z, acc.z); acc.w = fmaf(x.w, k.w, acc.w);
            }
        acc.x = act_bf(acc.x, L.nscale); acc.y = act_bf(acc.y, L.nscale);
        acc.z = act_bf(acc.z, L.nscale); acc.w = act_bf(acc.w, L.nscale);
        if (L.dst_off >= 0) *reinterpret_cast<float4 *>(lds + L.dst_off + apos(cb, P, p, q)) = acc;
        else *reinterpret_cast<float4 *>(gout + ((size_t)cb * P + p) * CB + 4 * q) = acc;
    }
}

__device__ __forceinline__ float4 pool_op(bool is_max, float4 acc, float4 v)
{
    if (is_max)
    {
        acc.x = v.x > acc.x ? v.x : acc.x; acc.y = v.y > acc.y ? v.y : acc.y;
        acc.z = v.z > acc.z ? v.z : acc.z; acc.w = v.w > acc.w ? v.w : acc.w;
    }
    else { acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w; }
    return acc;
}

// window == whole image, no padding (AveragePool2D: sum * float(1 / (H * W)), abstract_layer.hpp:514-569).
// A wave owns a channel quad (wave, wave + 16, ...): its lanes fold the pixels lane, lane + 64, ... in that order, then
// the wave folds its 64 partial sums with xor-shuffles (32, 16, ... 1): a fixed order (deterministic), no barrier and no
// LDS staging inside the layer.  (Three stages through LDS with two barriers took 2.4 us of the DS-CNN's 27.)
__device__ __forceinline__ void pool_layer(const FMLayer &L, float *lds, float *part, float *gout, int tid)
{
    (void)part;
    const int C4 = L.Ci / 4, P = L.H * L.W;
    const bool is_max = L.kind == K_POOL_MAX;
    const float *src = lds + L.src_off;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    for (int c4 = wave; c4 < C4; c4 += NW)
    {
        const int cb = c4 >> 2, q = c4 & 3;
        // a lane without a pixel holds the operation's neutral element: pixel 0 again for the maximum, zero for the sum
        float4 acc = is_max ? *reinterpret_cast<const float4 *>(src + apos(cb, P, 0, q)) : make_float4(0.f, 0.f, 0.f, 0.f);
        for (int p = lane; p < P; p += WAVE)
            acc = pool_op(is_max, acc, *reinterpret_cast<const float4 *>(src + apos(cb, P, p, q)));
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1)
        {
            const float4 o = make_float4(__shfl_xor(acc.x, d, WAVE), __shfl_xor(acc.y, d, WAVE), __shfl_xor(acc.z, d, WAVE),
                                         __shfl_xor(acc.w, d, WAVE));
            acc = pool_op(is_max, acc, o);
        }
        if (lane == 0)
        {
            if (!is_max) { acc.x *= L.norm; acc.y *= L.norm; acc.z *= L.norm; acc.w *= L.norm; }
            if (L.dst_off >= 0) *reinterpret_cast<float4 *>(lds + L.dst_off + apos(cb, 1, 0, q)) = acc;
            else *reinterpret_cast<float4 *>(gout + (size_t)cb * CB + 4 * q) = acc;
        }
    }
}

// n16 16-byte pieces from global memory to LDS without passing through registers (global_load_lds_dwordx4: a wave's
// 64 lanes write 1 KiB of consecutive LDS from the wave-uniform base; each lane supplies its own global address).
// The caller waits (vmcnt) before the data is read.
__device__ __forceinline__ void weights_to_lds(const float *g, float *l, int n16, int tid, int wave)
{
#pragma unroll
    for (int k = 0; k < NPRE; ++k)
    {
        const int i = tid + k * NT;
        if (i < n16)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(g + i * 4),
                                             (__attribute__((address_space(3))) void *)(l + (k * NT + wave * WAVE) * 4), 16, 0, 0);
    }
}

__global__ __launch_bounds__(NT) void fmodel_f32_kernel(const FMHeader *__restrict__ hdr_dev, const float *__restrict__ blob,
                                                        const float *__restrict__ in, float *__restrict__ out)
{
    HeaderPtr hdr = (HeaderPtr)hdr_dev;
    extern __shared__ __align__(16) float lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const size_t n = blockIdx.x;
    const int n_layers = hdr->n_layers;
    float *wbuf = lds + hdr->w_lds;
    const int w_floats = hdr->w_floats;

    // the first layer's weights and the image
    {
        weights_to_lds(blob + hdr->layer[0].blob_off, wbuf, hdr->layer[0].blob16, tid, wave);
        const float *img = in + n * (size_t)hdr->in_elems;
        float *x = lds + hdr->in_off;
        if (hdr->in_C < CB)
            for (int i = tid; i < hdr->in_elems; i += NT) x[i] = img[i];
        else
        {
            const int P = hdr->in_H * hdr->in_W, n4 = hdr->in_elems >> 2;
            for (int i = tid; i < n4; i += NT)
            {
                const int q = i & 3, r = i >> 2, cb = r / P, p = r - cb * P;
                *reinterpret_cast<float4 *>(x + apos(cb, P, p, q)) = reinterpret_cast<const float4 *>(img)[i];
            }
        }
    }
    float *gout = out + n * (size_t)hdr->out_elems;
    float *part = lds + hdr->pool_off;
    const float *zero = lds + hdr->zero_off;
    if (tid < 4) lds[hdr->zero_off + tid] = 0.f;
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();

    for (int li = 0; li < n_layers; ++li)
    {
        const FMLayer L = load_layer(hdr, li);
        const float *wl = wbuf + (li & 1) * w_floats;
        // the next layer's weights go from global memory straight into the other LDS buffer (no registers are held
        // across the layer): in flight while this layer is computed, waited for before the barrier that ends it
        if (L.next_blob16 > 0)
            weights_to_lds(blob + L.next_blob_off, wbuf + ((li + 1) & 1) * w_floats, L.next_blob16, tid, wave);
        if (L.kind == K_CONV)
        {
            const int n_tiles = ((L.Ho * L.Wo + 15) >> 4) * (L.Co / CB);
            if (n_tiles >= 2 * NW) conv_layer<2>(L, lds, wl, zero, gout, wave, lane);
            else conv_layer<1>(L, lds, wl, zero, gout, wave, lane);
        }
        else if (L.kind == K_STEM)
        {
            // as many output-channel blocks per gathered operand as still leave every wave a pixel tile
            const int CoB = L.Co / CB, n_pt = (L.Ho * L.Wo + 15) >> 4;
            if (CoB % 4 == 0 && n_pt * (CoB / 4) >= NW) stem_layer<4>(L, lds, wl, zero, gout, wave, lane);
            else if (CoB % 2 == 0 && n_pt * (CoB / 2) >= NW) stem_layer<2>(L, lds, wl, zero, gout, wave, lane);
            else stem_layer<1>(L, lds, wl, zero, gout, wave, lane);
        }
        else if (L.kind == K_DWPW)
        {
            // as many output-channel blocks per depthwise result as still leave every wave a pixel tile
            const int CoB = L.Co2 / CB, n_pt = (L.Ho * L.Wo + 15) >> 4;
            if (CoB % 4 == 0 && (n_pt * (CoB / 4) >= NW || CoB == 4)) dwpw_layer<4>(L, lds, wl, zero, gout, wave, lane);
            else if (CoB % 2 == 0) dwpw_layer<2>(L, lds, wl, zero, gout, wave, lane);
            else dwpw_layer<1>(L, lds, wl, zero, gout, wave, lane);
        }
        else if (L.kind == K_DW)
        {
            if (L.kh == 3 && L.kw == 3) dw_layer_win<3, 3>(L, lds, wl, zero, gout, tid);
            else dw_layer_any(L, lds, wl, gout, tid);
        }
        else
            pool_layer(L, lds, part, gout, tid);
        __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0): the weights have landed in LDS
        __syncthreads();
    }
}

int align_up(int v, int a) { return (v + a - 1) / a * a; }

} // namespace

struct small_hip_fmodel
{
    FMHeader hdr;
    void *dev = nullptr;        // [FMHeader][weights of every layer, operand order]
    size_t blob_off = 0;
    int device = 0;
};

extern "C" {

int small_hip_fmodel_create(int n_layers, const small_hip_flayer *layers, small_hip_fmodel **model,
                            small_hip_stream_t stream)
{
    const char *op = "small_hip_fmodel_create";
    if (!model) return einval("small_hip_fmodel_create: null result pointer");
    *model = nullptr;
    if (n_layers <= 0 || n_layers > MAX_LAYERS || !layers)
    { set_error("%s: 1..%d layers", op, MAX_LAYERS); return SMALL_HIP_EINVAL; }
    small_hip_fmodel *m = new (std::nothrow) small_hip_fmodel();
    if (!m) return SMALL_HIP_ENOMEM;
    std::memset(&m->hdr, 0, sizeof(m->hdr));
    FMHeader &h = m->hdr;
    auto fail = [&](int rc) { delete m; return rc; };
    std::vector<FMLayer> tmp((size_t)n_layers);          // one record per layer as given; fused pairs are formed below
    std::memset(tmp.data(), 0, sizeof(FMLayer) * (size_t)n_layers);

    int written_by[MAX_TENSORS];
    for (int t = 0; t < MAX_TENSORS; ++t) written_by[t] = -1;
    int blob_floats = 0, max_blob = 0;
    bool any_pool = false;
    std::vector<int> w_floats((size_t)n_layers, 0);
    for (int i = 0; i < n_layers; ++i)
    {
        const small_hip_flayer &l = layers[i];
        FMLayer &L = tmp[(size_t)i];
        const bool pool = l.kind == SMALL_HIP_FL_GLOBAL_AVGPOOL || l.kind == SMALL_HIP_FL_GLOBAL_MAXPOOL;
        if (l.kind != SMALL_HIP_FL_CONV && l.kind != SMALL_HIP_FL_DWCONV && !pool)
        { set_error("%s: layer %d: unknown kind", op, i); return fail(SMALL_HIP_EINVAL); }
        const int Ci = l.input_channels, H = l.input_height, W = l.input_width;
        if (H <= 0 || W <= 0 || Ci <= 0 || H > 4096 || W > 4096) { set_error("%s: layer %d: bad size", op, i); return fail(SMALL_HIP_EINVAL); }
        const bool from_input = l.src == SMALL_HIP_QM_INPUT;
        if (from_input != (i == 0)) { set_error("%s: exactly the first layer reads the model input", op); return fail(SMALL_HIP_EINVAL); }
        if (!from_input && (l.src < 0 || l.src >= MAX_TENSORS || written_by[l.src] < 0))
        { set_error("%s: layer %d reads a tensor that no earlier layer wrote", op, i); return fail(SMALL_HIP_EINVAL); }
        if (l.dst != SMALL_HIP_QM_OUTPUT && (l.dst < 0 || l.dst >= MAX_TENSORS || l.dst == l.src))
        { set_error("%s: layer %d: bad destination tensor", op, i); return fail(SMALL_HIP_EINVAL); }
        if ((l.dst == SMALL_HIP_QM_OUTPUT) != (i == n_layers - 1))
        { set_error("%s: exactly the last layer writes the model output", op); return fail(SMALL_HIP_EINVAL); }
        if (!from_input)
        {
            const FMLayer &S = tmp[(size_t)written_by[l.src]];
            if (S.Ho != H || S.Wo != W || S.Co != Ci)
            { set_error("%s: layer %d: input shape differs from what layer %d produces", op, i, written_by[l.src]); return fail(SMALL_HIP_EINVAL); }
        }
        L.Ci = Ci; L.H = H; L.W = W;
        L.nscale = 1.f;
        if (pool)
        {
            if (Ci % CB != 0 || Ci / 4 > NT) { set_error("%s: layer %d: pooling over %d channels", op, i, Ci); return fail(SMALL_HIP_EUNSUPPORTED); }
            if (l.kernel_height != H || l.kernel_width != W || l.t_pad || l.b_pad || l.l_pad || l.r_pad || from_input ||
                l.act != SMALL_HIP_ACT_NONE)
            { set_error("%s: layer %d: only whole-image pooling without padding or activation, after another layer", op, i); return fail(SMALL_HIP_EUNSUPPORTED); }
            L.kind = l.kind == SMALL_HIP_FL_GLOBAL_AVGPOOL ? K_POOL_AVG : K_POOL_MAX;
            L.Co = Ci; L.Ho = 1; L.Wo = 1; L.kh = H; L.kw = W; L.stride = 1;
            L.norm = (float)(1.0 / ((double)H * W));
            any_pool = true;
        }
        else
        {
            const int kh = l.kernel_height, kw = l.kernel_width, s = l.stride;
            const bool dw = l.kind == SMALL_HIP_FL_DWCONV;
            const int Co = dw ? Ci : l.output_channels;
            const bool stem = !dw && Ci < CB;
            if (stem ? !(Ci >= 1 && Ci <= 3) : Ci % CB != 0) { set_error("%s: layer %d: %d input channels", op, i, Ci); return fail(SMALL_HIP_EUNSUPPORTED); }
            if (stem && !from_input) { set_error("%s: layer %d: 1..3 input channels only on the model input", op, i); return fail(SMALL_HIP_EUNSUPPORTED); }
            if (dw && from_input) { set_error("%s: layer %d: the first layer must be a convolution", op, i); return fail(SMALL_HIP_EUNSUPPORTED); }
            if (s != 1 && s != 2) { set_error("%s: layer %d: stride %d", op, i, s); return fail(SMALL_HIP_EUNSUPPORTED); }
            if (kh <= 0 || kw <= 0 || kh > 255 || kw > 255 || Co <= 0 || Co % CB != 0 || !l.filter || !aligned16(l.filter) ||
                (l.bias && !aligned16(l.bias)) || !pads_ok(l.t_pad, l.b_pad, l.l_pad, l.r_pad))
            { set_error("%s: layer %d: bad convolution arguments", op, i); return fail(SMALL_HIP_EINVAL); }
            if (l.act < SMALL_HIP_ACT_NONE || l.act > SMALL_HIP_ACT_LEAKY) { set_error("%s: layer %d: bad activation", op, i); return fail(SMALL_HIP_EINVAL); }
            const int Ho = out_dim(H, l.t_pad, l.b_pad, kh, s), Wo = out_dim(W, l.l_pad, l.r_pad, kw, s);
            if (Ho <= 0 || Wo <= 0) { set_error("%s: layer %d: empty output", op, i); return fail(SMALL_HIP_EINVAL); }
            L.kind = dw ? K_DW : stem ? K_STEM : K_CONV;
            L.Co = Co; L.Ho = Ho; L.Wo = Wo; L.kh = kh; L.kw = kw; L.stride = s; L.pt = l.t_pad; L.pl = l.l_pad;
            L.nscale = l.act == SMALL_HIP_ACT_RELU ? 0.f : l.act == SMALL_HIP_ACT_LEAKY ? l.slope : 1.f;
            const long taps = (long)kh * kw;
            long wf;
            if (dw) wf = (long)Ci * taps;
            else if (stem)
            {
                L.K = (int)(taps * Ci);
                L.chunks = (L.K + 15) / 16;
                wf = (long)Co * L.chunks * 16;
            }
            else wf = (long)Co * Ci * taps;
            long bf = wf + Co + (stem ? L.chunks * 16 : 0);
            bf = (bf + 3) & ~3L;
            if (bf > (long)NPRE * NT * 4) { set_error("%s: layer %d: more than %d KB of weights", op, i, NPRE * NT * 16 / 1024); return fail(SMALL_HIP_EUNSUPPORTED); }
            w_floats[(size_t)i] = (int)wf;
            L.bias_off = (int)wf;
            L.ktab_off = (int)wf + Co;
            L.blob_off = blob_floats;
            L.blob16 = (int)(bf >> 2);
            blob_floats += (int)bf;
        }
        L.r_wo = 1.0f / (float)L.Wo;
        L.r_cob = 1.0f / (float)(L.Co / CB);
        L.r_p = 1.0f / (float)(L.Ho * L.Wo);
        if ((long)L.Co * L.Ho * L.Wo > LDS_LIMIT / 4)
        { set_error("%s: layer %d: output tensor larger than LDS", op, i); return fail(SMALL_HIP_EUNSUPPORTED); }
        if (l.dst >= 0) written_by[l.dst] = i;
    }

    // The launch's layer list.  A 3x3 depthwise convolution whose only reader is the 1x1 stride-1 convolution right
    // after it becomes one layer with it (their weights already lie back to back in the blob); the depthwise tensor
    // then needs no LDS.  SMALL_HIP_TUNE key fmodel_fuse=0 keeps the layers apart (a measurement aid).
    static const bool fuse_off = tune_int("fmodel_fuse", 1) == 0;
    int tensor_floats[MAX_TENSORS] = {};
    int dev_src[MAX_LAYERS], dev_dst[MAX_LAYERS], n_dev = 0;
    // where a caller's tensor id lives: a fused pair must not write the tensor it reads (callers ping-pong between two
    // ids, so the 1x1 convolution's destination usually IS the depthwise input, whose neighbouring pixels other waves
    // still read); its result then goes to the tensor the depthwise result would have had, and the two ids trade places
    int phys[MAX_TENSORS];
    for (int t = 0; t < MAX_TENSORS; ++t) phys[t] = t;
    for (int i = 0; i < n_layers; ++i)
    {
        FMLayer L = tmp[(size_t)i];
        const int lsrc = layers[i].src, ldst = layers[i].dst;
        int src = lsrc >= 0 ? phys[lsrc] : lsrc, dst = ldst >= 0 ? phys[ldst] : ldst;
        if (!fuse_off && L.kind == K_DW && L.kh == 3 && L.kw == 3 && i + 1 < n_layers)
        {
            const FMLayer &N = tmp[(size_t)i + 1];
            bool ok = N.kind == K_CONV && N.kh == 1 && N.kw == 1 && N.stride == 1 && N.Ho == N.H && N.Wo == N.W &&
                      layers[i + 1].src == ldst && L.blob16 + N.blob16 <= NPRE * NT;
            for (int j = i + 2; ok && j < n_layers; ++j)      // nobody else reads the depthwise result
            {
                if (layers[j].src == ldst) ok = false;
                if (layers[j].dst == ldst) break;
            }
            if (ok)
            {
                L.kind = K_DWPW;
                L.Co2 = N.Co;
                L.w2_off = N.blob_off - L.blob_off;
                L.bias2_off = L.w2_off + N.bias_off;
                L.nscale2 = N.nscale;
                L.r_cob2 = 1.0f / (float)(N.Co / CB);
                L.blob16 += N.blob16;
                const int odst = layers[i + 1].dst;
                if (odst >= 0 && phys[odst] == src)
                {
                    const int free_id = phys[ldst];
                    phys[ldst] = phys[odst];
                    phys[odst] = free_id;
                }
                dst = odst >= 0 ? phys[odst] : odst;
                ++i;
            }
        }
        if (dst >= 0 && dst == src) { set_error("%s: layer %d writes the tensor it reads", op, i); return fail(SMALL_HIP_EINVAL); }
        h.layer[n_dev] = L;
        dev_src[n_dev] = src; dev_dst[n_dev] = dst;
        max_blob = L.blob16 * 4 > max_blob ? L.blob16 * 4 : max_blob;
        if (dst >= 0)
        {
            const int Co = L.kind == K_DWPW ? L.Co2 : L.Co;
            const int fl = Co * L.Ho * L.Wo;
            tensor_floats[dst] = fl > tensor_floats[dst] ? fl : tensor_floats[dst];
        }
        ++n_dev;
    }
    h.n_layers = n_dev;
    for (int i = 0; i + 1 < n_dev; ++i)
    {
        h.layer[i].next_blob_off = h.layer[i + 1].blob_off;
        h.layer[i].next_blob16 = h.layer[i + 1].blob16;
    }

    // LDS plan (floats): [weights x2][pooling partials][input][tensors]
    int off = 0;
    h.w_lds = off; h.w_floats = max_blob; off += 2 * max_blob;
    h.pool_off = off; off += any_pool ? NT * 4 + NT / 2 * 4 : 0;
    h.zero_off = off; off += 4;
    const small_hip_flayer &l0 = layers[0];
    h.in_C = l0.input_channels; h.in_H = l0.input_height; h.in_W = l0.input_width;
    h.in_elems = h.in_C * h.in_H * h.in_W;
    h.in_off = off; off += align_up(h.in_elems, 4);
    int tensor_off[MAX_TENSORS];
    for (int t = 0; t < MAX_TENSORS; ++t) { tensor_off[t] = off; off += tensor_floats[t]; }
    h.lds_bytes = off * 4;
    if ((long)off * 4 > LDS_LIMIT)
    {
        set_error("%s: the model needs %ld bytes of LDS (activations %ld, weights of two layers %d), the limit is %d: run it "
                  "layer by layer", op, (long)off * 4, (long)(off - h.in_off) * 4, 2 * max_blob * 4, LDS_LIMIT);
        return fail(SMALL_HIP_EUNSUPPORTED);
    }
    for (int i = 0; i < n_dev; ++i)
    {
        FMLayer &L = h.layer[i];
        L.src_off = i == 0 ? h.in_off : tensor_off[dev_src[i]];
        L.dst_off = dev_dst[i] >= 0 ? tensor_off[dev_dst[i]] : -1;
    }
    const FMLayer &last = tmp[(size_t)n_layers - 1];
    h.out_elems = last.Co * last.Ho * last.Wo;

    hipStream_t s = as_stream(stream);
    hipError_t e = hipGetDevice(&m->device);
    if (e != hipSuccess) return fail(fail_hip(e, "hipGetDevice"));
    m->blob_off = (sizeof(FMHeader) + 255) & ~(size_t)255;
    e = hipMalloc(&m->dev, m->blob_off + (size_t)blob_floats * 4 + 256);
    if (e != hipSuccess)
    {
        (void)hipGetLastError();
        set_error("%s: hipMalloc: %s", op, hipGetErrorString(e));
        return fail(e == hipErrorOutOfMemory ? SMALL_HIP_ENOMEM : SMALL_HIP_EHIP);
    }
    auto fail_dev = [&](int rc) { (void)hipFree(m->dev); return fail(rc); };
    float *dblob = reinterpret_cast<float *>(static_cast<uint8_t *>(m->dev) + m->blob_off);
    std::vector<std::vector<int>> ktabs((size_t)n_layers);          // alive until the stream has been waited for
    for (int i = 0; i < n_layers; ++i)
    {
        const FMLayer &L = tmp[(size_t)i];
        if (L.kind != K_CONV && L.kind != K_STEM && L.kind != K_DW) continue;
        const int wf = w_floats[(size_t)i];
        const int nthreads = wf > L.Co ? wf : L.Co;
        hipLaunchKernelGGL(fm_prep_kernel, dim3((unsigned)((nthreads + 255) / 256)), dim3(256), 0, s, L.kind, layers[i].filter,
                           layers[i].bias, dblob + L.blob_off, L.Co, L.Ci, L.kh * L.kw, L.K, L.chunks, wf);
        e = hipGetLastError();
        if (e != hipSuccess) return fail_dev(fail_hip(e, "small_hip_fmodel_create: pre-pass"));
        if (L.kind == K_STEM)
        {
            std::vector<int> &kt = ktabs[(size_t)i];
            // entry [chunk][kq][j] describes reduction element k = 16 chunk + 4 j + kq
            kt.assign((size_t)L.chunks * 16, -1);
            for (int k = 0; k < L.K; ++k)
            {
                const int tap = k / L.Ci, ci = k - tap * L.Ci, a = tap / L.kw, b = tap - a * L.kw;
                const int chunk = k / 16, j = (k % 16) / 4, kq = k % 4;
                kt[(size_t)((chunk * 4 + kq) * 4 + j)] = a | (b << 8) | (ci << 16);
            }
            e = hipMemcpyAsync(dblob + L.blob_off + L.ktab_off, kt.data(), kt.size() * sizeof(int), hipMemcpyHostToDevice, s);
            if (e != hipSuccess) return fail_dev(fail_hip(e, "small_hip_fmodel_create: tables"));
        }
    }
    e = hipMemcpyAsync(m->dev, &m->hdr, sizeof(FMHeader), hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);       // the caller's filters and the host-side tables may go
    if (e != hipSuccess) return fail_dev(fail_hip(e, "small_hip_fmodel_create: upload"));
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(fmodel_f32_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            LDS_LIMIT);
    if (e != hipSuccess) return fail_dev(fail_hip(e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)"));
    *model = m;
    return SMALL_HIP_OK;
}

int small_hip_fmodel_forward(const small_hip_fmodel *model, int batch, const float *input, float *output,
                             small_hip_stream_t stream)
{
    if (!model || !model->dev) return einval("small_hip_fmodel_forward: null model");
    if (batch < 0 || !input || !output) return einval("small_hip_fmodel_forward: bad argument");
    if (batch == 0) return SMALL_HIP_OK;
    if (!aligned16(output) || (model->hdr.in_C >= CB && !aligned16(input)))
        return einval("small_hip_fmodel_forward: misaligned pointer");
    const float *dblob = reinterpret_cast<const float *>(static_cast<const uint8_t *>(model->dev) + model->blob_off);
    hipLaunchKernelGGL(fmodel_f32_kernel, dim3((unsigned)batch), dim3(NT), (size_t)model->hdr.lds_bytes, as_stream(stream),
                       static_cast<const FMHeader *>(model->dev), dblob, input, output);
    SHP_LAUNCH_CHECK("small_hip_fmodel_forward");
    return SMALL_HIP_OK;
}

size_t small_hip_fmodel_output_elems(const small_hip_fmodel *model) { return model ? (size_t)model->hdr.out_elems : 0; }
size_t small_hip_fmodel_lds_bytes(const small_hip_fmodel *model) { return model ? (size_t)model->hdr.lds_bytes : 0; }

int small_hip_fmodel_destroy(small_hip_fmodel *model)
{
    if (!model) return SMALL_HIP_OK;
    int rc = SMALL_HIP_OK;
    if (model->dev)
    {
        hipError_t e = hipFree(model->dev);
        if (e != hipSuccess) rc = fail_hip(e, "small_hip_fmodel_destroy: hipFree");
    }
    delete model;
    return rc;
}

} // extern "C"
