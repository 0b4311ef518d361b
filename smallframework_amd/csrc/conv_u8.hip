// Conv2D / Dense (uint8, int32 accumulation, fused requantisation) for gfx950.
//
// The reference accumulates  acc = sum over VALID taps of (I + zI) * (F + zF)  in int32
// (include/small/platforms/reference/intrinsics_quint8.h:191-223; padded taps are skipped, not
// multiplied by the zero point) and requantises in the same pass.  Here the uint8 operands are
// re-biased to signed bytes (x' = x - 128 = x ^ 0x80) so that the contraction runs on
// v_mfma_i32_16x16x64_i8, and the zero-point terms are added back exactly in the epilogue:
//
//   acc = S + ZF * SI[px] + ZI * (SF[co][px] + ZF * Ci * nv[px])         (mod 2^32)
//     S   = sum_valid I' * F'            (MFMA)
//     SI  = sum_valid I'                 (v_sad_u8 on the bytes the lane loads anyway)
//     SF  = sum over the valid taps of Wsum[co][tap],  Wsum = sum_ci F'   (filter pre-pass)
//     nv  = number of valid taps,  ZI = zI + 128,  ZF = zF + 128
//   The valid taps of a pixel form a rectangle [a_lo,a_hi) x [b_lo,b_hi) of the filter window, so
//   SF is read from a 2-D prefix-sum table P[(kh+1)*(kw+1)][Co] with four 16-byte loads per lane
//   (P[hi][hi] - P[lo][hi] - P[hi][lo] + P[lo][lo], exact in wrap-around int32) whatever the
//   border position; interior pixels are the same formula with the full rectangle.
//
// The epilogue can also apply the two element-wise layers that follow a convolution in a residual
// block, both in place on the convolution's output buffer and both with its quantisation parameters:
//   Accum(shortcut, out):  out = requant((shortcut + zS) + (out + zO))
//   ReLUActivation(out, out):  out = requant(max(out + zO, 0))
// which is bit-identical to issuing the three layers one after the other.
//
// A filter pre-pass (one small kernel) turns the packed filter [Co/16][Ci/16][tap][16 ci][16 co]
// into the MFMA A-operand order [Co/16][step][16 co][16 ci] of signed bytes (step = tap*Ci/16 +
// ci block, zero padded to a multiple of 4 steps) and produces Wsum / Wtot.  It does not depend
// on any zero point, so a model can run it once per filter (small_hip_conv2d_u8_prepare_filter)
// and call the prepared entry point per batch.
//
// MFMA mapping (16x16x64): rows = output channels, columns = output pixels, and each of the four
// 16-lane groups of the wave supplies one K-step of 16 bytes -- a pixel's whole 16-channel block
// is one 16-byte load.  A lane ends up with 4 consecutive output channels of one pixel:
// requantise, pack, store one dword; the wave writes 256 contiguous bytes.
#include "common.h"

#include <mutex>
#include "quant.h"

#include <cstdlib>

using namespace shp;

namespace
{

typedef int v4i __attribute__((ext_vector_type(4)));

// n / d for 0 <= n < 2^31, d >= 1, with rcp = 1.0 / d: a double product is within one of the
// quotient, the remainder test fixes it.  A handful of full-rate instructions instead of the
// ~25 of the generic 32-bit division; these kernels are small enough for that to show.
__device__ __forceinline__ int udiv_rcp(int n, int d, double rcp)
{
    int q = (int)((double)n * rcp);
    const int r = n - q * d;
    q += r >= d ? 1 : 0;
    q -= r < 0 ? 1 : 0;
    return q;
}

struct QConvArgs
{
    const uint8_t *in;
    const int8_t *ft;        // prepared filter [Co/16][S_pad][16][16]
    const int32_t *wpre;     // prefix sums of the per-tap filter sums: [(kh+1)*(kw+1)][Co]
    const uint8_t *accum_src; // optional shortcut tensor added after the convolution (same shape as out)
    uint8_t *out;
    int batch, Co, Ci, H, W, Ho, Wo, kh, kw, stride, pt, pl;
    int stride_h;            // vertical stride: `stride`, or 1 for the 1-D layers
    int32_t ZI, ZF;          // zero points + 128
    int32_t zS, zO;          // zero points of the shortcut and of the output buffer (fused Accum / ReLU)
    int relu;
    int use_table;       // tabulate the Accum / ReLU requantisation per workgroup (pays when the launch is ALU-bound)
    QOut q;
    int P, S, S_pad, n_co_groups, n_px_blocks, n_blocks, per_xcd;
    double r_howo, r_wo, r_cib, r_kw;   // reciprocals of Ho*Wo, Wo, Ci/16, kw for udiv_rcp
    // grouped convolution: blockIdx.y walks `slabs` (image, group) slabs that lie in_slab / out_slab bytes apart; slab y
    // uses the prepared filter (slab0 + y) % groups, prep_slab bytes apart.  slabs == 0: an ordinary convolution.
    int slabs, groups, slab0;
    long long in_slab, out_slab, prep_slab;
};

struct GroupSlabs
{
    int slabs = 0, groups = 1, slab0 = 0;
    int stride_h = 0;        // > 0: another vertical stride (1 for the 1-D layers)
};

__device__ __forceinline__ QConvArgs slab_args(QConvArgs a)
{
    if (a.slabs > 0)
    {
        const int y = blockIdx.y;
        a.in += (long long)y * a.in_slab;
        a.out += (long long)y * a.out_slab;
        const long long f = (long long)((a.slab0 + y) % a.groups) * a.prep_slab;
        a.ft += f;
        a.wpre = reinterpret_cast<const int32_t *>(reinterpret_cast<const int8_t *>(a.wpre) + f);
    }
    return a;
}

// ---- filter pre-pass ---------------------------------------------------------------------------
// one lane per (co, step): reads 16 ci bytes at stride 16, writes 16 contiguous signed bytes
__global__ __launch_bounds__(256) void prep_filter_u8_kernel(const uint8_t *__restrict__ f,
                                                             int8_t *__restrict__ ft, int Co, int CiB,
                                                             int taps, int S_pad)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= Co * S_pad) return;
    const int co16 = i & 15;
    const int s = (i >> 4) % S_pad;
    const int cob = (i >> 4) / S_pad;
    uint32_t w[4] = {0, 0, 0, 0};
    if (s < taps * CiB)
    {
        const int tap = s / CiB, cib = s - tap * CiB;
        const uint8_t *src = f + (((size_t)cob * CiB + cib) * taps + tap) * 256 + co16;
#pragma unroll
        for (int ci = 0; ci < 16; ++ci) w[ci >> 2] |= (uint32_t)(src[ci * 16] ^ 0x80u) << (8 * (ci & 3));
    }
    reinterpret_cast<uint4 *>(ft)[(size_t)(cob * S_pad + s) * 16 + co16] = make_uint4(w[0], w[1], w[2], w[3]);
}

// one lane per output channel: per-tap sums Wsum[a][b] = sum_ci (F - 128), then the inclusive 2-D
// prefix table P[a][b] = sum_{a' < a, b' < b} Wsum[a'][b'] stored as [(kh+1)*(kw+1)][Co]
__global__ __launch_bounds__(256) void wprefix_u8_kernel(const uint8_t *__restrict__ f, int32_t *__restrict__ wpre,
                                                         int Co, int CiB, int kh, int kw)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= Co) return;
    const int cob = i >> 4, co16 = i & 15;
    const int taps = kh * kw;
    for (int b = 0; b <= kw; ++b) wpre[(size_t)b * Co + i] = 0;
    for (int a = 0; a < kh; ++a)
    {
        wpre[(size_t)((a + 1) * (kw + 1)) * Co + i] = 0;
        uint32_t row = 0;
        for (int b = 0; b < kw; ++b)
        {
            int32_t sum = 0;
            for (int cib = 0; cib < CiB; ++cib)
            {
                const uint8_t *src = f + (((size_t)cob * CiB + cib) * taps + a * kw + b) * 256 + co16;
#pragma unroll
                for (int ci = 0; ci < 16; ++ci) sum += (int32_t)src[ci * 16] - 128;
            }
            row += (uint32_t)sum;
            wpre[(size_t)((a + 1) * (kw + 1) + b + 1) * Co + i] =
                (int32_t)((uint32_t)wpre[(size_t)(a * (kw + 1) + b + 1) * Co + i] + row);
        }
    }
}

// The Accum and ReLU stages that follow a convolution in a residual block requantise values from a
// tiny domain (a sum of two bytes, a byte), so a workgroup tabulates them once instead of running
// the 64-bit requantisation per element: post[t], t = accumulated byte + convolution byte (0..510)
// or, without Accum, t = convolution byte (0..255), holds the byte the op-by-op sequence produces.
struct PostArgs
{
    int has_accum, relu;
    int32_t zS, zO;
    QOut q;
};

__device__ __forceinline__ void build_post_table(uint8_t (&post)[512], const PostArgs pa)
{
    for (int t = threadIdx.x; t < (pa.has_accum ? 511 : 256); t += blockDim.x)
    {
        uint32_t y = (uint32_t)t;
        if (pa.has_accum) y = requant_u8((int32_t)((uint32_t)t + (uint32_t)pa.zS + (uint32_t)pa.zO), pa.q);
        if (pa.relu)
        {
            const int32_t z = (int32_t)y + pa.zO;
            y = requant_u8(z > 0 ? z : 0, pa.q);
        }
        post[t] = (uint8_t)y;
    }
}

// ---- main kernel --------------------------------------------------------------------------------
// 16 bytes of 0x80, the re-biased zero: masked taps load from here instead of being patched after
// the load (a select on the loaded value would make the wave wait for the data where it was issued)
__device__ __align__(16) uint8_t g_bias_block[16] = {0x80, 0x80, 0x80, 0x80, 0x80, 0x80, 0x80, 0x80,
                                                    0x80, 0x80, 0x80, 0x80, 0x80, 0x80, 0x80, 0x80};

template <int COT, int PXT>
__global__ __launch_bounds__(256) void conv_mfma_u8_kernel(const QConvArgs a0)
{
    const QConvArgs a = slab_args(a0);
    const int bid = blockIdx.x;
    const int lid = (bid % NUM_XCD) * a.per_xcd + bid / NUM_XCD;
    if (lid >= a.n_blocks) return;
    const int cg = lid % a.n_co_groups;
    const int pxb = lid / a.n_co_groups;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = lane & 15;
    const int grp = lane >> 4;

    __shared__ uint8_t post[512];
    const bool use_post = a.use_table && (a.accum_src != nullptr || a.relu);     // uniform

    const int HoWo = a.Ho * a.Wo;
    const int CiB = a.Ci / CB;
    const int CoB = a.Co / CB;
    const size_t in_blk = (size_t)a.H * a.W * CB;

    const uint8_t *in_img[PXT];
    int ih0[PXT], iw0[PXT], rem_of[PXT], n_of[PXT];
    bool pvalid[PXT];
    uint32_t sumI[PXT];
#pragma unroll
    for (int t = 0; t < PXT; ++t)
    {
        const int p = ((pxb * 4 + wave) * PXT + t) * 16 + col;
        pvalid[t] = p < a.P;
        const int pc = pvalid[t] ? p : 0;
        const int n = udiv_rcp(pc, HoWo, a.r_howo);
        const int rem = pc - n * HoWo;
        const int oh = udiv_rcp(rem, a.Wo, a.r_wo);
        const int ow = rem - oh * a.Wo;
        ih0[t] = oh * a.stride_h - a.pt;
        iw0[t] = ow * a.stride - a.pl;
        in_img[t] = a.in + (size_t)n * CiB * in_blk;
        rem_of[t] = rem;
        n_of[t] = n;
        sumI[t] = 0;
    }
    // A rows: channel block (cg*COT + c), row `col`; blocks past Co are clamped and never stored
    const int8_t *w_row[COT];
#pragma unroll
    for (int c = 0; c < COT; ++c)
    {
        int cob = cg * COT + c;
        cob = cob < CoB ? cob : CoB - 1;
        w_row[c] = a.ft + ((size_t)cob * a.S_pad * 16 + col) * 16;
    }

    v4i acc[COT][PXT];
#pragma unroll
    for (int c = 0; c < COT; ++c)
#pragma unroll
        for (int t = 0; t < PXT; ++t) acc[c][t] = v4i{0, 0, 0, 0};

    // Software pipeline of depth D over the K loop (4 K-steps per iteration, one per 16-lane group):
    // the loads of iteration i+D are issued right after iteration i has been multiplied, so D
    // iterations' worth of loads are always in flight.  These layers are small and latency-bound:
    // without it every iteration paid a full memory round trip.  Masked taps load the 0x80 block
    // (re-biased zero, contributes nothing to the product or to sumI).
    constexpr int D = 3;
    uint4 Bq[D][PXT], Wq[D][COT];
    auto load = [&](int s0, uint4 (&Bv)[PXT], uint4 (&Wv)[COT]) {
        if (s0 >= a.S_pad) return;        // uniform: nothing left to fetch, the registers are not consumed again
        const int s = s0 + grp;
        const bool svalid = s < a.S;
        const int sc = svalid ? s : 0;
        const int tap = udiv_rcp(sc, CiB, a.r_cib);
        const int cib = sc - tap * CiB;
        const int ta = udiv_rcp(tap, a.kw, a.r_kw);
        const int tb = tap - ta * a.kw;
#pragma unroll
        for (int t = 0; t < PXT; ++t)
        {
            const int ih = ih0[t] + ta, iw = iw0[t] + tb;
            const bool ok = svalid && pvalid[t] && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
            const size_t off = (size_t)cib * in_blk + ((size_t)ih * a.W + iw) * CB;
            Bv[t] = *reinterpret_cast<const uint4 *>(ok ? in_img[t] + off : g_bias_block);
        }
        const int sw = s < a.S_pad ? s : 0;          // past the end: any valid filter step (B is zero)
#pragma unroll
        for (int c = 0; c < COT; ++c) Wv[c] = *reinterpret_cast<const uint4 *>(w_row[c] + (size_t)sw * 256);
    };
    auto consume = [&](const uint4 (&Bv)[PXT], const uint4 (&Wv)[COT]) {
        v4i B[PXT];
#pragma unroll
        for (int t = 0; t < PXT; ++t)
        {
            const uint4 v = Bv[t];
            // sum of the 16 raw bytes minus 16*128 = sum of the signed bytes (0 for masked taps)
            uint32_t sb = __builtin_amdgcn_sad_u8(v.x, 0u, 0u);
            sb = __builtin_amdgcn_sad_u8(v.y, 0u, sb);
            sb = __builtin_amdgcn_sad_u8(v.z, 0u, sb);
            sb = __builtin_amdgcn_sad_u8(v.w, 0u, sb);
            sumI[t] += sb - 2048u;
            B[t] = v4i{(int)(v.x ^ 0x80808080u), (int)(v.y ^ 0x80808080u), (int)(v.z ^ 0x80808080u),
                       (int)(v.w ^ 0x80808080u)};
        }
#pragma unroll
        for (int c = 0; c < COT; ++c)
        {
            const v4i A = v4i{(int)Wv[c].x, (int)Wv[c].y, (int)Wv[c].z, (int)Wv[c].w};
#pragma unroll
            for (int t = 0; t < PXT; ++t)
                acc[c][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, B[t], acc[c][t], 0, 0, 0);
        }
    };
#pragma unroll
    for (int d = 0; d < D; ++d) load(4 * d, Bq[d], Wq[d]);
    // tabulate the post-ops while the first loads are in flight
    if (use_post)
    {
        build_post_table(post, PostArgs{a.accum_src != nullptr, a.relu, a.zS, a.zO, a.q});
        __syncthreads();                  // use_post is uniform over the launch
    }
    for (int s0 = 0; s0 < a.S_pad; s0 += 4 * D)
    {
#pragma unroll
        for (int d = 0; d < D; ++d)
        {
            if (s0 + 4 * d >= a.S_pad) break;        // uniform
            consume(Bq[d], Wq[d]);
            load(s0 + 4 * (d + D), Bq[d], Wq[d]);
        }
    }

    // ---- epilogue: zero-point terms, requantise, optional Accum / ReLU, pack, store ----------------
    const int pw = a.kw + 1;
#pragma unroll
    for (int t = 0; t < PXT; ++t)
    {
        // total over the four K groups of this pixel column
        uint32_t si = sumI[t];
        si += (uint32_t)__shfl_xor((int)si, 16);
        si += (uint32_t)__shfl_xor((int)si, 32);
        if (!pvalid[t]) continue;
        // valid tap rectangle of this pixel
        const int a_lo = ih0[t] < 0 ? -ih0[t] : 0;
        int a_hi = (a.H - ih0[t]) < a.kh ? (a.H - ih0[t]) : a.kh;
        const int b_lo = iw0[t] < 0 ? -iw0[t] : 0;
        int b_hi = (a.W - iw0[t]) < a.kw ? (a.W - iw0[t]) : a.kw;
        a_hi = a_hi > a_lo ? a_hi : a_lo;
        b_hi = b_hi > b_lo ? b_hi : b_lo;
        const uint32_t base = (uint32_t)a.ZF * si;
        const uint32_t cnt = (uint32_t)a.ZF * (uint32_t)(a.Ci * (a_hi - a_lo) * (b_hi - b_lo));
        const int32_t *p_hh = a.wpre + (size_t)(a_hi * pw + b_hi) * a.Co;
        const int32_t *p_lh = a.wpre + (size_t)(a_lo * pw + b_hi) * a.Co;
        const int32_t *p_hl = a.wpre + (size_t)(a_hi * pw + b_lo) * a.Co;
        const int32_t *p_ll = a.wpre + (size_t)(a_lo * pw + b_lo) * a.Co;
#pragma unroll
        for (int c = 0; c < COT; ++c)
        {
            const int cob = cg * COT + c;
            if (cob >= CoB) continue;
            const int co4 = cob * CB + 4 * grp;
            const uint4 hh = *reinterpret_cast<const uint4 *>(p_hh + co4);
            const uint4 lh = *reinterpret_cast<const uint4 *>(p_lh + co4);
            const uint4 hl = *reinterpret_cast<const uint4 *>(p_hl + co4);
            const uint4 ll = *reinterpret_cast<const uint4 *>(p_ll + co4);
            const uint32_t sf4[4] = {hh.x - lh.x - hl.x + ll.x, hh.y - lh.y - hl.y + ll.y,
                                     hh.z - lh.z - hl.z + ll.z, hh.w - lh.w - hl.w + ll.w};
            uint32_t *o = reinterpret_cast<uint32_t *>(
                a.out + (((size_t)n_of[t] * CoB + cob) * HoWo + rem_of[t]) * CB + 4 * grp);
            uint32_t sc = 0;
            if (a.accum_src)
                sc = *reinterpret_cast<const uint32_t *>(
                    a.accum_src + (((size_t)n_of[t] * CoB + cob) * HoWo + rem_of[t]) * CB + 4 * grp);
            uint32_t packed = 0;
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
                const uint32_t v = (uint32_t)acc[c][t][r] + base + (uint32_t)a.ZI * (sf4[r] + cnt);
                uint32_t y = requant_u8((int32_t)v, a.q);
                if (use_post) y = post[y + ((sc >> (8 * r)) & 0xffu)];      // sc is 0 without Accum
                else
                {
                    if (a.accum_src)
                        y = requant_u8((int32_t)(((sc >> (8 * r)) & 0xffu) + (uint32_t)a.zS + y + (uint32_t)a.zO), a.q);
                    if (a.relu)
                    {
                        const int32_t z = (int32_t)y + a.zO;
                        y = requant_u8(z > 0 ? z : 0, a.q);
                    }
                }
                packed |= y << (8 * r);
            }
            *o = packed;
        }
    }
}

// ---- first layers (Ci in {1,2,3}): vector ALU, direct (I + zI) * (F + zF) ----------------------------
struct QSmallArgs
{
    const uint8_t *in;
    const uint8_t *filt;
    uint8_t *out;
    int batch, Co, H, W, Ho, Wo, kh, kw, stride, pt, pl, P;
    int stride_h;
    int32_t zi, zf;
    const uint8_t *accum_src;
    int32_t zS, zO;
    int relu;
    int use_table;       // tabulate the Accum / ReLU requantisation per workgroup (pays when the launch is ALU-bound)
    QOut q;
};

// M24: both zero points are small enough (|z| < 2^22) that (byte + z) fits 24 signed bits; the
// products then use the full-rate 24-bit multiply-add (its low 32 bits equal those of the 32-bit
// wrap-around product), four times the rate of the 32-bit integer multiply.
template <int CI, bool M24>
__global__ __launch_bounds__(256) void conv_smallci_u8_kernel(const QSmallArgs a)
{
    __shared__ uint8_t post[512];
    const bool use_post = a.use_table && (a.accum_src != nullptr || a.relu);     // uniform
    const int p0 = blockIdx.x * 256 + threadIdx.x;
    const bool live = p0 < a.P;                                 // lanes past the end compute nothing, store nothing
    const int p = live ? p0 : 0;
    const int cob = blockIdx.y;
    const int HoWo = a.Ho * a.Wo;
    const int n = p / HoWo;
    const int rem = p - n * HoWo;
    const int oh = rem / a.Wo;
    const int ow = rem - oh * a.Wo;
    const int ih0 = oh * a.stride_h - a.pt, iw0 = ow * a.stride - a.pl;
    const uint8_t *img = a.in + (size_t)n * a.H * a.W * CI;
    const uint8_t *w = a.filt + (size_t)cob * a.kh * a.kw * CI * CB;
    uint32_t acc[CB];
#pragma unroll
    for (int j = 0; j < CB; ++j) acc[j] = 0;
    for (int ta = 0; ta < (live ? a.kh : 0); ++ta)
    {
        const int ih = ih0 + ta;
        if (ih < 0 || ih >= a.H) continue;
        for (int tb = 0; tb < a.kw; ++tb)
        {
            const int iw = iw0 + tb;
            if (iw < 0 || iw >= a.W) continue;
            const uint8_t *ip = img + ((size_t)ih * a.W + iw) * CI;
            const uint8_t *wp = w + (size_t)(ta * a.kw + tb) * CI * CB;
#pragma unroll
            for (int ci = 0; ci < CI; ++ci)
            {
                const int32_t xs = (int32_t)ip[ci] + a.zi;
#pragma unroll
                for (int j = 0; j < CB; ++j)
                {
                    const int32_t ws = (int32_t)wp[ci * CB + j] + a.zf;
                    if (M24) acc[j] += (uint32_t)__mul24(xs, ws);
                    else acc[j] += (uint32_t)xs * (uint32_t)ws;
                }
            }
        }
    }
    if (use_post)
    {
        build_post_table(post, PostArgs{a.accum_src != nullptr, a.relu, a.zS, a.zO, a.q});
        __syncthreads();                  // use_post is uniform over the launch
    }
    const size_t opos = (((size_t)n * (a.Co / CB) + cob) * HoWo + rem) * CB;
    uint4 sc4 = make_uint4(0, 0, 0, 0);
    if (a.accum_src && live) sc4 = *reinterpret_cast<const uint4 *>(a.accum_src + opos);
    const uint32_t scw[4] = {sc4.x, sc4.y, sc4.z, sc4.w};
    uint32_t pk[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < CB; ++j)
    {
        uint32_t y = requant_u8((int32_t)acc[j], a.q);
        if (use_post) y = post[y + ((scw[j >> 2] >> (8 * (j & 3))) & 0xffu)];   // scw is 0 without Accum
        else
        {
            if (a.accum_src)
                y = requant_u8((int32_t)(((scw[j >> 2] >> (8 * (j & 3))) & 0xffu) + (uint32_t)a.zS + y + (uint32_t)a.zO), a.q);
            if (a.relu)
            {
                const int32_t z = (int32_t)y + a.zO;
                y = requant_u8(z > 0 ? z : 0, a.q);
            }
        }
        pk[j >> 2] |= y << (8 * (j & 3));
    }
    if (live) *reinterpret_cast<uint4 *>(a.out + opos) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
}

// workgroups from which the post-op table pays (below, the launch is latency-bound and the table only adds a barrier)
long table_min_wg()
{
    static const long v = tune_int("convq_table_min_wg", 2 * NUM_CU);
    return v;
}

size_t ws_ft_bytes(int Co, int S_pad) { return (size_t)Co * S_pad * 16; }

size_t prepared_bytes(int kh, int kw, int Co, int Ci)
{
    const int S = kh * kw * (Ci / CB), S_pad = (S + 3) & ~3;
    size_t b = ws_ft_bytes(Co, S_pad);                 // multiple of 64
    b += (size_t)Co * (kh + 1) * (kw + 1) * sizeof(int32_t);   // prefix sums of the per-tap filter sums
    return (b + 255) & ~(size_t)255;
}

int prepare_filter(int kh, int kw, int Co, int Ci, const uint8_t *filt, void *ws, hipStream_t s)
{
    const int CiB = Ci / CB, taps = kh * kw, S = taps * CiB, S_pad = (S + 3) & ~3;
    int8_t *ft = static_cast<int8_t *>(ws);
    int32_t *wpre = reinterpret_cast<int32_t *>(ft + ws_ft_bytes(Co, S_pad));
    const int n1 = Co * S_pad;
    hipLaunchKernelGGL(prep_filter_u8_kernel, dim3((n1 + 255) / 256), dim3(256), 0, s, filt, ft, Co, CiB, taps, S_pad);
    SHP_LAUNCH_CHECK("prep_filter_u8_kernel");
    hipLaunchKernelGGL(wprefix_u8_kernel, dim3((Co + 255) / 256), dim3(256), 0, s, filt, wpre, Co, CiB, kh, kw);
    SHP_LAUNCH_CHECK("wprefix_u8_kernel");
    return SMALL_HIP_OK;
}

template <int COT, int PXT>
void launch_q(QConvArgs &a, hipStream_t s)
{
    a.n_co_groups = (a.Co / CB + COT - 1) / COT;
    a.n_px_blocks = (a.P + 16 * PXT * 4 - 1) / (16 * PXT * 4);
    a.n_blocks = a.n_co_groups * a.n_px_blocks;
    a.per_xcd = (a.n_blocks + NUM_XCD - 1) / NUM_XCD;
    a.use_table = a.n_blocks >= table_min_wg();
    hipLaunchKernelGGL((conv_mfma_u8_kernel<COT, PXT>), dim3(a.per_xcd * NUM_XCD, a.slabs > 0 ? a.slabs : 1), dim3(256), 0, s, a);
}

int conv_u8_check(const char *op, int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int Co,
                  int Ci, int H, int W, const void *in, const void *filt, const void *out,
                  const small_hip_quant *iq, const small_hip_quant *fq, const small_hip_quant *oq)
{
    const bool blocked = Ci > 0 && Ci % CB == 0;
    const bool small_ci = Ci == 1 || Ci == 2 || Ci == 3;
    if (!blocked && !small_ci) return SMALL_HIP_ECHANNELS;
    if (stride != 1 && stride != 2) return SMALL_HIP_ESTRIDE;
    if (batch <= 0 || kh <= 0 || kw <= 0 || H <= 0 || W <= 0 || Co <= 0 || !pads_ok(pt, pb, pl, pr))
    { set_error("%s: bad size", op); return SMALL_HIP_EINVAL; }
    if (Co % CB != 0) { set_error("%s: output_channels must be a multiple of 16 (pad the filter)", op); return SMALL_HIP_EINVAL; }
    if (!iq || !fq || !oq) { set_error("%s: null quantisation parameters", op); return SMALL_HIP_EINVAL; }
    if (oq->rshift < 0 || oq->rshift > 31 || oq->lshift < 0 || oq->lshift > 31)
    { set_error("%s: shift out of range", op); return SMALL_HIP_EINVAL; }
    if (!in || !filt || !out || !aligned16(filt) || !aligned16(out) || (blocked && !aligned16(in)))
    { set_error("%s: null or misaligned pointer", op); return SMALL_HIP_EINVAL; }
    if (in == out) { set_error("%s: in-place convolution is not supported", op); return SMALL_HIP_EINVAL; }
    return SMALL_HIP_OK;
}

// ---- scratch of the entry point that allocates nothing -------------------------------------------------------
// The filter pre-pass of small_hip_conv2d_u8_noalloc writes here instead of into an allocated block.  Every GPU the
// library runs on holds its own copy of the array at its own address until the process ends; in host code the array's
// name is only a handle for hipGetSymbolAddress, whose per-device result is what kernels and copies are given.
constexpr size_t NOALLOC_SCRATCH_BYTES = size_t(SMALL_HIP_NOALLOC_MAX_PREPARED_BYTES);
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

// Calls on different streams of one GPU share the array: the library orders them on the device (the later call's
// pre-pass waits for the earlier call's convolution through one event per GPU, created at the first call; no host wait).
// The lock is held from the wait to the record, so that two host threads cannot interleave their launches.  A call
// recorded into a HIP graph is not ordered this way (an event of ordinary work must not enter a capture): replays that
// overlap other users of the array are the caller's to order.
struct StaticScratchUse
{
    std::unique_lock<std::mutex> lock;
    void *ptr = nullptr;
    int dev = -1;
    bool capturing = false;
};
struct StaticScratchState
{
    static constexpr int MAX_DEV = 64;
    std::mutex mu;
    void *addr[MAX_DEV] = {};
    hipEvent_t done[MAX_DEV] = {};
    hipStream_t last[MAX_DEV] = {};
    bool pending[MAX_DEV] = {};
};
StaticScratchState &static_state()
{
    static StaticScratchState st;
    return st;
}

int static_scratch_begin(const char *op, size_t bytes, hipStream_t s, StaticScratchUse *use)
{
    if (bytes > NOALLOC_SCRATCH_BYTES)
    {
        set_error("%s: the prepared filter needs %zu bytes, the static scratch holds %zu (use "
                  "small_hip_conv2d_u8_prepare_filter + small_hip_conv2d_u8_prepared for larger filters)",
                  op, bytes, NOALLOC_SCRATCH_BYTES);
        return SMALL_HIP_EINVAL;
    }
    int dev = 0;
    SHP_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= StaticScratchState::MAX_DEV) { set_error("%s: device index out of range", op); return SMALL_HIP_EINVAL; }
    StaticScratchState &st = static_state();
    use->lock = std::unique_lock<std::mutex>(st.mu);
    use->dev = dev;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    SHP_HIP(hipStreamIsCapturing(s, &cs));
    use->capturing = cs != hipStreamCaptureStatusNone;
    if (!st.addr[dev])
    {
        if (use->capturing)
        { set_error("%s: the first call on a GPU looks up the static array and cannot be recorded into a graph: call once before the capture", op); return SMALL_HIP_EINVAL; }
        void *p = nullptr;
        SHP_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));      // the current device's copy
        if (!p) { set_error("%s: hipGetSymbolAddress returned null", op); return SMALL_HIP_EHIP; }
        SHP_HIP(hipEventCreateWithFlags(&st.done[dev], hipEventDisableTiming));
        st.addr[dev] = p;
    }
    if (!use->capturing && st.pending[dev] && st.last[dev] != s) SHP_HIP(hipStreamWaitEvent(s, st.done[dev], 0));
    use->ptr = st.addr[dev];
    return SMALL_HIP_OK;
}

// after the call's last launch has been enqueued on s
int static_scratch_end(StaticScratchUse *use, hipStream_t s)
{
    if (use->capturing || use->dev < 0) return SMALL_HIP_OK;
    StaticScratchState &st = static_state();
    SHP_HIP(hipEventRecord(st.done[use->dev], s));
    st.last[use->dev] = s;
    st.pending[use->dev] = true;
    return SMALL_HIP_OK;
}

struct Fuse
{
    const uint8_t *accum_src = nullptr;
    int32_t zS = 0;
    int relu = 0;
};

int conv_u8_run(const char *op, int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int Co,
                int Ci, int H, int W, const uint8_t *in, const small_hip_quant *iq, const void *prepared,
                const small_hip_quant *fq, uint8_t *out, const small_hip_quant *oq, const Fuse &fz,
                hipStream_t s, const GroupSlabs grp = GroupSlabs{})
{
    QConvArgs a{};
    const int CiB = Ci / CB, taps = kh * kw;
    a.S = taps * CiB;
    a.S_pad = (a.S + 3) & ~3;
    a.r_cib = 1.0 / CiB; a.r_kw = 1.0 / kw;
    a.in = in; a.out = out;
    a.ft = static_cast<const int8_t *>(prepared);
    a.wpre = reinterpret_cast<const int32_t *>(a.ft + ws_ft_bytes(Co, a.S_pad));
    a.accum_src = fz.accum_src;
    a.zS = fz.zS;
    a.zO = oq->zero;
    a.relu = fz.relu;
    a.batch = batch; a.Co = Co; a.Ci = Ci; a.H = H; a.W = W; a.kh = kh; a.kw = kw;
    a.stride = stride; a.pt = pt; a.pl = pl;
    a.stride_h = grp.stride_h > 0 ? grp.stride_h : stride;
    a.Ho = out_dim(H, pt, pb, kh, a.stride_h);
    a.Wo = out_dim(W, pl, pr, kw, stride);
    a.r_howo = 1.0 / ((double)a.Ho * a.Wo); a.r_wo = 1.0 / a.Wo;
    a.ZI = (int32_t)((uint32_t)iq->zero + 128u);
    a.ZF = (int32_t)((uint32_t)fq->zero + 128u);
    a.q = make_qout(oq->multiplier, oq->lshift, oq->rshift);
    const long P = (long)batch * a.Ho * a.Wo;
    if (P == 0) return SMALL_HIP_OK;
    if (P > 0x7fffffffL / 64) { set_error("%s: batch*Ho*Wo too large for one launch", op); return SMALL_HIP_EINVAL; }
    a.P = (int)P;
    const long n_slabs = grp.slabs > 0 ? grp.slabs : 1;
    if (grp.slabs > 0)
    {
        if (batch != 1 || grp.slabs > 65535) { set_error("%s: bad slab launch", op); return SMALL_HIP_EINVAL; }
        a.slabs = grp.slabs; a.groups = grp.groups; a.slab0 = grp.slab0;
        a.in_slab = (long long)Ci * H * W;
        a.out_slab = (long long)Co * a.Ho * a.Wo;
        a.prep_slab = (long long)prepared_bytes(kh, kw, Co, Ci);
    }
    const int CoB = Co / CB;
    // The largest wave tile (COT channel blocks x PXT pixel groups of 16) that still leaves at least
    // `want` workgroups: these layers are small and latency-bound, so filling the chip with waves
    // comes before operand re-use.
    static const long want = tune_int("convq_min_wg", 512);
    auto nwg = [&](int cot, int pxt) { return (long)((CoB + cot - 1) / cot) * ((P + 64 * pxt - 1) / (64 * pxt)) * n_slabs; };
    if (CoB % 4 == 0 && nwg(4, 2) >= want) launch_q<4, 2>(a, s);
    else if (CoB % 2 == 0 && nwg(2, 2) >= want) launch_q<2, 2>(a, s);
    else if (nwg(1, 2) >= want) launch_q<1, 2>(a, s);
    else launch_q<1, 1>(a, s);
    SHP_LAUNCH_CHECK(op);
    return SMALL_HIP_OK;
}

int conv_u8(const char *op, int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int Co, int Ci,
            int H, int W, const uint8_t *in, const small_hip_quant *iq, const uint8_t *filt,
            const small_hip_quant *fq, uint8_t *out, const small_hip_quant *oq, const Fuse &fz,
            small_hip_stream_t stream, bool static_ws = false, const GroupSlabs grp = GroupSlabs{})
{
    const int stride_h = grp.stride_h > 0 ? grp.stride_h : stride;
    if (int rc = conv_u8_check(op, batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, filt, out, iq, fq, oq))
        return rc;
    hipStream_t s = as_stream(stream);
    if (Ci < CB)
    {
        QSmallArgs a{};
        a.in = in; a.filt = filt; a.out = out; a.batch = batch; a.Co = Co; a.H = H; a.W = W;
        a.kh = kh; a.kw = kw; a.stride = stride; a.pt = pt; a.pl = pl;
        a.stride_h = stride_h;
        a.Ho = out_dim(H, pt, pb, kh, stride_h);
        a.Wo = out_dim(W, pl, pr, kw, stride);
        a.zi = iq->zero; a.zf = fq->zero;
        a.accum_src = fz.accum_src; a.zS = fz.zS; a.zO = oq->zero; a.relu = fz.relu;
        a.q = make_qout(oq->multiplier, oq->lshift, oq->rshift);
        const long P = (long)batch * a.Ho * a.Wo;
        if (P == 0) return SMALL_HIP_OK;
        if (P > 0x7fffffffL / 64) { set_error("%s: batch*Ho*Wo too large for one launch", op); return SMALL_HIP_EINVAL; }
        a.P = (int)P;
        const dim3 grid((unsigned)((a.P + 255) / 256), (unsigned)(Co / CB));
        a.use_table = (long)grid.x * grid.y >= table_min_wg();
        void (*k)(const QSmallArgs) = nullptr;
        const auto small = [](int32_t z) { return z > -(1 << 22) && z < (1 << 22); };
        if (small(a.zi) && small(a.zf)) k = Ci == 1 ? conv_smallci_u8_kernel<1, true> : Ci == 2 ? conv_smallci_u8_kernel<2, true> : conv_smallci_u8_kernel<3, true>;
        else k = Ci == 1 ? conv_smallci_u8_kernel<1, false> : Ci == 2 ? conv_smallci_u8_kernel<2, false> : conv_smallci_u8_kernel<3, false>;
        hipLaunchKernelGGL(k, grid, dim3(256), 0, s, a);
        SHP_LAUNCH_CHECK(op);
        return SMALL_HIP_OK;
    }
    // refuse what conv_u8_run would refuse before anything is enqueued
    const long P = (long)batch * out_dim(H, pt, pb, kh, stride_h) * out_dim(W, pl, pr, kw, stride);
    if (P == 0) return SMALL_HIP_OK;
    if (P > 0x7fffffffL / 64) { set_error("%s: batch*Ho*Wo too large for one launch", op); return SMALL_HIP_EINVAL; }
    void *ws = nullptr;
    WorkspaceLease lease;            // held until the launches below are enqueued
    StaticScratchUse use;            // the same for the static array
    if (static_ws)
    {
        if (int rc = static_scratch_begin(op, prepared_bytes(kh, kw, Co, Ci), s, &use)) return rc;
        ws = use.ptr;
    }
    else
    {
        if (int rc = lease_workspace(prepared_bytes(kh, kw, Co, Ci), s, &lease)) return rc;
        ws = lease.ptr;
    }
    if (int rc = prepare_filter(kh, kw, Co, Ci, filt, ws, s)) return rc;
    if (int rc = conv_u8_run(op, batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, iq, ws, fq, out, oq, fz, s, grp)) return rc;
    return static_ws ? static_scratch_end(&use, s) : SMALL_HIP_OK;
}

int fuse_check(const char *op, const uint8_t *accum_input, const small_hip_quant *accum_q, const void *out, Fuse *fz,
               int relu)
{
    fz->relu = relu ? 1 : 0;
    if (accum_input)
    {
        if (!accum_q) { set_error("%s: accum_input without quantisation parameters", op); return SMALL_HIP_EINVAL; }
        if (!aligned16(accum_input) || accum_input == out)
        { set_error("%s: misaligned or aliased accum_input", op); return SMALL_HIP_EINVAL; }
        fz->accum_src = accum_input;
        fz->zS = accum_q->zero;
    }
    return SMALL_HIP_OK;
}

} // namespace

namespace shp
{
// the filter pre-pass for other translation units (the whole-model kernel prepares its layers with it)
size_t prepared_bytes_u8(int kh, int kw, int Co, int Ci) { return prepared_bytes(kh, kw, Co, Ci); }
size_t prepared_table_offset_u8(int kh, int kw, int Co, int Ci)
{
    const int S = kh * kw * (Ci / CB), S_pad = (S + 3) & ~3;
    return ws_ft_bytes(Co, S_pad);
}
int prepare_filter_u8(int kh, int kw, int Co, int Ci, const uint8_t *filt, void *ws, hipStream_t s)
{
    return prepare_filter(kh, kw, Co, Ci, filt, ws, s);
}
} // namespace shp

extern "C" {

int small_hip_conv2d_u8(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int Co, int Ci,
                        int H, int W, const uint8_t *in, const small_hip_quant *iq, const uint8_t *filt,
                        const small_hip_quant *fq, uint8_t *out, const small_hip_quant *oq,
                        small_hip_stream_t stream)
{
    return conv_u8("small_hip_conv2d_u8", batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, iq, filt, fq,
                   out, oq, Fuse{}, stream);
}

int small_hip_conv2d_u8_noalloc(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int Co, int Ci,
                                int H, int W, const uint8_t *in, const small_hip_quant *iq, const uint8_t *filt,
                                const small_hip_quant *fq, uint8_t *out, const small_hip_quant *oq,
                                small_hip_stream_t stream)
{
    return conv_u8("small_hip_conv2d_u8_noalloc", batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, iq, filt,
                   fq, out, oq, Fuse{}, stream, true);
}

// The quantised form of the grouped convolution: the filters of all groups prepared once, then one launch over the
// (image, group) slabs of `channels` channels.
static int group_conv_u8(const char *op, int batch, int kh, int kw, int stride, int stride_h, int groups, int pt, int pb, int pl,
                         int pr, int channels, int H, int W, const uint8_t *in, const small_hip_quant *iq,
                         const uint8_t *filt, const small_hip_quant *fq, uint8_t *out, const small_hip_quant *oq,
                         small_hip_stream_t stream)
{
    if (channels <= 0 || channels % CB != 0) return SMALL_HIP_ECHANNELS;
    if (stride != 1 && stride != 2) return SMALL_HIP_ESTRIDE;
    if (batch <= 0 || groups <= 0 || kh <= 0 || kw <= 0 || H <= 0 || W <= 0 || !pads_ok(pt, pb, pl, pr))
    { set_error("%s: bad size", op); return SMALL_HIP_EINVAL; }
    if (!in || !filt || !out) { set_error("%s: null pointer", op); return SMALL_HIP_EINVAL; }
    const size_t in_slab = (size_t)channels * H * W;
    const size_t out_slab = (size_t)channels * out_dim(H, pt, pb, kh, stride_h ? stride_h : stride) * out_dim(W, pl, pr, kw, stride);
    const size_t filt_slab = (size_t)channels * channels * kh * kw;
    const size_t slabs = (size_t)batch * groups;
    if (in + slabs * in_slab > out && out + slabs * out_slab > in)
    { set_error("%s: in-place convolution is not supported", op); return SMALL_HIP_EINVAL; }
    if (int rc = conv_u8_check(op, 1, kh, kw, stride, pt, pb, pl, pr, channels, channels, H, W, in, filt, out, iq, fq, oq))
        return rc;
    if (out_slab == 0) return SMALL_HIP_OK;
    if (out_slab / channels > (size_t)(0x7fffffffL / 64)) { set_error("%s: Ho*Wo too large for one launch", op); return SMALL_HIP_EINVAL; }
    // every group's filter is prepared once into the leased block, then the (image, group) slabs are the second grid
    // dimension of ONE convolution launch (65535 slabs at most per launch)
    hipStream_t s = as_stream(stream);
    const size_t prep = prepared_bytes(kh, kw, channels, channels);
    WorkspaceLease lease;
    if (int rc = lease_workspace(prep * (size_t)groups, s, &lease)) return rc;
    for (int g = 0; g < groups; ++g)
        if (int rc = prepare_filter(kh, kw, channels, channels, filt + (size_t)g * filt_slab,
                                    static_cast<uint8_t *>(lease.ptr) + (size_t)g * prep, s))
            return rc;
    for (size_t i = 0; i < slabs; i += 65535)
    {
        GroupSlabs g;
        g.slabs = (int)(slabs - i < 65535 ? slabs - i : 65535);
        g.groups = groups;
        g.slab0 = (int)(i % (size_t)groups);
        g.stride_h = stride_h;
        const int rc = conv_u8_run(op, 1, kh, kw, stride, pt, pb, pl, pr, channels, channels, H, W, in + i * in_slab, iq,
                                   lease.ptr, fq, out + i * out_slab, oq, Fuse{}, s, g);
        if (rc != SMALL_HIP_OK) return rc;
    }
    return SMALL_HIP_OK;
}

int small_hip_group_conv2d_u8(int batch, int kh, int kw, int stride, int groups, int pt, int pb, int pl, int pr,
                              int channels, int H, int W, const uint8_t *in, const small_hip_quant *iq,
                              const uint8_t *filt, const small_hip_quant *fq, uint8_t *out,
                              const small_hip_quant *oq, small_hip_stream_t stream)
{
    return group_conv_u8("small_hip_group_conv2d_u8", batch, kh, kw, stride, 0, groups, pt, pb, pl, pr, channels, H, W, in, iq,
                         filt, fq, out, oq, stream);
}

// The quantised 1-D convolutions (interface_abstract_1D.hpp:229, 1320): `rows` independent signals of `width` samples, a
// 1 x k window moved by `stride` along the width only; groups > 0: the grouped form (input_channels per group).
int small_hip_conv1d_u8(int batch, int k, int stride, int l_pad, int r_pad, int groups, int Co, int Ci, int rows, int width,
                        const uint8_t *in, const small_hip_quant *iq, const uint8_t *filt, const small_hip_quant *fq,
                        uint8_t *out, const small_hip_quant *oq, small_hip_stream_t stream)
{
    if (groups > 0)
        return group_conv_u8("small_hip_conv1d_u8", batch, 1, k, stride, 1, groups, 0, 0, l_pad, r_pad, Ci, rows, width, in, iq,
                             filt, fq, out, oq, stream);
    GroupSlabs g;
    g.stride_h = 1;
    return conv_u8("small_hip_conv1d_u8", batch, 1, k, stride, 0, 0, l_pad, r_pad, Co, Ci, rows, width, in, iq, filt, fq, out, oq,
                   Fuse{}, stream, false, g);
}

int small_hip_dense_u8(int batch, int No, int Ni, const uint8_t *in, const small_hip_quant *iq,
                       const uint8_t *filt, const small_hip_quant *fq, uint8_t *out, const small_hip_quant *oq,
                       small_hip_stream_t stream)
{
    return conv_u8("small_hip_dense_u8", batch, 1, 1, 1, 0, 0, 0, 0, No, Ni, 1, 1, in, iq, filt, fq, out, oq,
                   Fuse{}, stream);
}

size_t small_hip_conv2d_u8_prepared_filter_bytes(int kh, int kw, int Co, int Ci)
{
    if (kh <= 0 || kw <= 0 || Co <= 0 || Co % CB != 0 || Ci <= 0 || Ci % CB != 0) return 0;
    return prepared_bytes(kh, kw, Co, Ci);
}

int small_hip_conv2d_u8_prepare_filter(int kh, int kw, int Co, int Ci, const uint8_t *filt, void *prepared,
                                       small_hip_stream_t stream)
{
    if (kh <= 0 || kw <= 0 || Co <= 0 || Co % CB != 0) return einval("small_hip_conv2d_u8_prepare_filter: bad size");
    if (Ci <= 0 || Ci % CB != 0) return SMALL_HIP_ECHANNELS;
    if (!filt || !prepared || !aligned16(filt) || !aligned16(prepared))
        return einval("small_hip_conv2d_u8_prepare_filter: null or misaligned pointer");
    return prepare_filter(kh, kw, Co, Ci, filt, prepared, as_stream(stream));
}

int small_hip_conv2d_u8_prepared(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int Co,
                                 int Ci, int H, int W, const uint8_t *in, const small_hip_quant *iq,
                                 const void *prepared, const small_hip_quant *fq, uint8_t *out,
                                 const small_hip_quant *oq, small_hip_stream_t stream)
{
    const char *op = "small_hip_conv2d_u8_prepared";
    if (Ci <= 0 || Ci % CB != 0) return SMALL_HIP_ECHANNELS;
    if (int rc = conv_u8_check(op, batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, prepared, out, iq, fq, oq))
        return rc;
    return conv_u8_run(op, batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, iq, prepared, fq, out, oq,
                       Fuse{}, as_stream(stream));
}

int small_hip_conv2d_accum_relu_u8(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr, int Co,
                                   int Ci, int H, int W, const uint8_t *in, const small_hip_quant *iq,
                                   const uint8_t *filt, const small_hip_quant *fq, const uint8_t *accum_input,
                                   const small_hip_quant *accum_q, int relu, uint8_t *out,
                                   const small_hip_quant *oq, small_hip_stream_t stream)
{
    const char *op = "small_hip_conv2d_accum_relu_u8";
    Fuse fz;
    if (int rc = fuse_check(op, accum_input, accum_q, out, &fz, relu)) return rc;
    return conv_u8(op, batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, iq, filt, fq, out, oq, fz, stream);
}

int small_hip_conv2d_accum_relu_u8_prepared(int batch, int kh, int kw, int stride, int pt, int pb, int pl, int pr,
                                            int Co, int Ci, int H, int W, const uint8_t *in,
                                            const small_hip_quant *iq, const void *prepared,
                                            const small_hip_quant *fq, const uint8_t *accum_input,
                                            const small_hip_quant *accum_q, int relu, uint8_t *out,
                                            const small_hip_quant *oq, small_hip_stream_t stream)
{
    const char *op = "small_hip_conv2d_accum_relu_u8_prepared";
    if (Ci <= 0 || Ci % CB != 0) return SMALL_HIP_ECHANNELS;
    if (int rc = conv_u8_check(op, batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, prepared, out, iq, fq, oq))
        return rc;
    Fuse fz;
    if (int rc = fuse_check(op, accum_input, accum_q, out, &fz, relu)) return rc;
    return conv_u8_run(op, batch, kh, kw, stride, pt, pb, pl, pr, Co, Ci, H, W, in, iq, prepared, fq, out, oq, fz,
                       as_stream(stream));
}

} // extern "C"
