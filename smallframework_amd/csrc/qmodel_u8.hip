// Whole-model forward pass of a small quantised (uint8) CNN in ONE launch for gfx950.
//
// The layer-by-layer path runs a model like ResNet-8 (32x32x3 input, <= 16 KB per activation tensor, 77 KB of
// weights) as eleven dependent launches of 4-18 us, each a round trip through HBM for a tensor that would fit in a
// corner of one CU's LDS.  Here one workgroup owns one image from input to logits: the prepared filters of every
// layer and all activation tensors live in the CU's 160 KB of LDS, only the input image and the model's output
// touch global memory, and the layers are separated by workgroup barriers instead of kernel boundaries.
//
// Arithmetic is the layer functions' own, bit for bit (small::Conv2D / ReLUActivation<QUInt8Buffer>:
// include/small/q_abstract_layer.hpp:894-1567, include/small/platforms/reference/intrinsics_quint8.h:191-223, 481-531;
// Accum / AveragePool2D on uint8 as small_hip_accum_u8 / small_hip_avgpool2d_u8 define them):
//   acc = sum over VALID taps of (I + zI) * (F + zF),   out = requant(acc)   [+ Accum] [+ ReLU in place]
// evaluated as in conv_u8.hip: operands re-biased to signed bytes (x' = x ^ 0x80) for v_mfma_i32_16x16x64_i8 and the
// zero-point terms restored exactly in the epilogue,
//   acc = S + ZF * SI[px] + ZI * (SF[co][px] + ZF * Ci * nv[px])    (mod 2^32),   ZI = zI + 128, ZF = zF + 128.
//
// LDS layout.  Activations are kept re-biased, channel-blocked and with a one-pixel ring of zeros:
// [C/16][H + 2][W + 2][16] signed bytes.  A zero in that encoding is "this tap contributes nothing" to S and SI, so
// padded taps need no masks: every operand is one aligned 16-byte LDS read at pixel base + a per-step constant, and
// SI is the plain box sum of what the lane loads anyway (v_dot4 with a vector of ones).  The last term depends on the
// pixel's border case only (which of the first / last window row and column fall outside the image: with a ring of
// one pixel 4 x 4 cases) and on the output channel: it is tabulated per layer when the model is created,
// T[case][co], fetched into LDS one layer ahead, and costs the epilogue one 16-byte LDS read.  A first layer with
// 1..3 input channels is staged as [H + 2][W + 2][4] (channel padded with zeros) and one window row (kw * 4 <= 16
// bytes) is one K group of the MFMA, so a 3x3 stem is a single MFMA per 16 x 16 output tile.
//
// MFMA mapping as in conv_u8.hip: rows = 16 output channels, columns = 16 output pixels, the four 16-lane groups of a
// wave supply four K-steps; a lane ends with 4 consecutive channels of one pixel = one dword store into the next
// layer's LDS tensor.  The 16 waves of the workgroup take (channel block, pixel tile) pairs round robin, two pixel
// tiles at a time on one filter operand while there are enough tiles.
//
// Nothing waits on device memory between the first and the last layer: the filters of layers >= 1 are loaded into
// registers before the first layer is computed and stored to LDS after it; each layer's tables (K-step offsets,
// the Accum / ReLU byte table, T) are written by the previous layer's waves as they finish, into the other half of a
// double buffer, so a layer costs one barrier.
#include "common.h"
#include "quant.h"

#include <cstring>
#include <mutex>
#include <new>
#include <vector>

using namespace shp;

namespace
{

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int NT = 1024;                 // threads per workgroup: 16 waves, 4 per SIMD (one workgroup per CU: LDS)
constexpr int NW = NT / WAVE;
constexpr int MAX_LAYERS = 32;
constexpr int MAX_TENSORS = 8;
constexpr int MAX_STEPS = 256;           // K-steps (taps x channel blocks) of one layer
constexpr int MAX_CO = 128;              // a layer's tables are fetched by one 16-byte load per thread
constexpr int LDS_LIMIT = 160 * 1024;
constexpr int FIN_ENTRIES = 514, FIN_BYTES = 528;   // the short epilogue's table (conv_tiles), padded to 16 bytes

enum { K_STEM = 0, K_CONV = 1, K_POOL_AVG = 2, K_POOL_MAX = 3 };

// One layer.  The descriptors live in device memory and are read through a pointer to the CONSTANT address space, which
// the compiler reads with scalar loads into scalar registers (the memory is written once, when the model is created).
// Read through an ordinary pointer, every use inside the tile loops became a fresh vector load (the loops' stores may
// alias it as far as the compiler can tell); copied out of LDS lane by lane, a descriptor cost more vector instructions
// than a small layer's arithmetic; passed by value as a kernel argument, the whole block was copied to scratch memory
// as soon as the layer index was dynamic.
struct QMLayer
{
    int kind;
    int src_off, dst_off, acc_off;       // LDS byte offsets of the tensors; dst_off < 0: the model's output in global
                                         // memory; acc_off < 0: no Accum
    int Ci, Co, H, W, Ho, Wo, kh, kw, stride, pt, pl;
    int S_pad;                           // K-steps padded to a multiple of 4
    int w_off;                           // prepared filter: offset in LDS == offset in the filter image of the blob
    int tab_off, tab16;                  // the layer's tables in the blob: T[16][Co] int32 | steps[S_pad] int32 | post[512] |
                                         // fin[528] | postx[512] | pixel table [Ho*Wo][2] uint16, and their size in 16-byte pieces
    int32_t ZF;                          // filter zero point + 128 (convolutions)
    int32_t zI;                          // zero point of the input (pooling)
    int has_post;                        // Accum and / or ReLU follow: the convolution's byte goes through post[]
    int idx_shift;                       // >= 0: the short epilogue (rshift - 2, see conv_tiles); -1: the general one
    int geo_off;                         // the pixel table's offset inside the layer's tables (the short epilogue's layers)
    float r_wo, r_cob;                   // 1 / Wo, 1 / (Co / 16)
    int wo_shift;                        // log2(Wo) when Wo is a power of two, else -1
    QOut q;
};

struct QMHeader
{
    int n_layers;
    int filter_bytes;                    // LDS image of all prepared filters (blob offset 0 -> LDS offset 0)
    int first_bytes;                     // ... of which the first layer's (needed before anything else)
    int later_kib;                       // KiB behind it that hold the later layers' filters (the last one rounded up)
    int in_C, in_H, in_W, in_off;        // the model input and the LDS offset it is staged at
    int tab_lds, tab_bytes, pool_off;    // LDS scratch: tables[2][tab_bytes], pooling sums
    int in_elems, out_elems;             // bytes per image in global memory
    int lds_bytes;
    QMLayer layer[MAX_LAYERS];
};
typedef const __attribute__((address_space(4))) QMHeader *HeaderPtr;

// a descriptor out of constant memory into (scalar) registers
__device__ __forceinline__ QMLayer load_layer(HeaderPtr hdr, int li)
{
    QMLayer L;
    __builtin_memcpy(&L, &hdr->layer[li], sizeof(QMLayer));
    return L;
}

__device__ __forceinline__ int sdot_ones(uint32_t v, int acc)
{
    return __builtin_amdgcn_sdot4((int)v, 0x01010101, acc, false);
}

// ---- model creation: filter pre-passes ------------------------------------------------------------------------
// first layer: packed filter [Co/16][kh][kw][Ci][16 co] (Ci in 1..3) -> [Co/16][4 rows][16 co][16 bytes = kw x 4
// channels] signed, zero padded (rows >= kh, channels >= Ci, columns >= kw), and the prefix table
// P[(kh+1)*(kw+1)][Co] of the per-tap sums of F - 128
__global__ __launch_bounds__(256) void qm_prep_stem_kernel(const uint8_t *__restrict__ f, int8_t *__restrict__ ft,
                                                           int32_t *__restrict__ wpre, int Co, int Ci, int kh, int kw)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < Co * 4)
    {
        const int co16 = i & 15, row = (i >> 4) & 3, cob = i >> 6;
        uint32_t w[4] = {0, 0, 0, 0};
        if (row < kh)
            for (int b = 0; b < kw; ++b)
                for (int ci = 0; ci < Ci; ++ci)
                {
                    const uint32_t v = f[(((size_t)cob * kh + row) * kw + b) * Ci * 16 + ci * 16 + co16];
                    w[b] |= ((v ^ 0x80u) & 0xffu) << (8 * ci);
                }
        reinterpret_cast<uint4 *>(ft)[(size_t)(cob * 4 + row) * 16 + co16] = make_uint4(w[0], w[1], w[2], w[3]);
    }
    if (i < Co)
    {
        const int cob = i >> 4, co16 = i & 15;
        for (int b = 0; b <= kw; ++b) wpre[(size_t)b * Co + i] = 0;
        for (int a = 0; a < kh; ++a)
        {
            wpre[(size_t)((a + 1) * (kw + 1)) * Co + i] = 0;
            uint32_t row = 0;
            for (int b = 0; b < kw; ++b)
            {
                int32_t sum = 0;
                for (int ci = 0; ci < Ci; ++ci)
                    sum += (int32_t)f[(((size_t)cob * kh + a) * kw + b) * Ci * 16 + ci * 16 + co16] - 128;
                row += (uint32_t)sum;
                wpre[(size_t)((a + 1) * (kw + 1) + b + 1) * Co + i] =
                    (int32_t)((uint32_t)wpre[(size_t)(a * (kw + 1) + b + 1) * Co + i] + row);
            }
        }
    }
}

// T[case][co] = ZI * (SF + ZF * Ci * nv) for the 16 border cases of a pixel: case = ra * 4 + rb,
// ra = 2 * (first window row outside the image) + (last window row outside), rb likewise for columns;
// SF = sum of F - 128 over the valid taps, from the prefix table; wrap-around 32-bit arithmetic throughout.
__global__ __launch_bounds__(256) void qm_case_table_kernel(const int32_t *__restrict__ wpre, int32_t *__restrict__ T,
                                                            int Co, int Ci, int kh, int kw, int32_t ZI, int32_t ZF)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= 16 * Co) return;
    const int cs = i / Co, co = i - cs * Co;
    const int ra = cs >> 2, rb = cs & 3;
    const int a_lo = ra >> 1, b_lo = rb >> 1;
    int a_hi = kh - (ra & 1), b_hi = kw - (rb & 1);
    a_hi = a_hi > a_lo ? a_hi : a_lo;
    b_hi = b_hi > b_lo ? b_hi : b_lo;
    const int pw = kw + 1;
    const uint32_t sf = (uint32_t)wpre[(size_t)(a_hi * pw + b_hi) * Co + co] - (uint32_t)wpre[(size_t)(a_lo * pw + b_hi) * Co + co] -
                        (uint32_t)wpre[(size_t)(a_hi * pw + b_lo) * Co + co] + (uint32_t)wpre[(size_t)(a_lo * pw + b_lo) * Co + co];
    const uint32_t cnt = (uint32_t)ZF * (uint32_t)(Ci * (a_hi - a_lo) * (b_hi - b_lo));
    T[i] = (int32_t)((uint32_t)ZI * (sf + cnt));
}

__global__ __launch_bounds__(256) void qm_copy16_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, int n16)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}

// ---- device: one layer -----------------------------------------------------------------------------------------
__device__ __forceinline__ void zero_ring(uint8_t *t, int Cb, int H, int W, int tid)
{
    const int Hp = H + 2, Wp = W + 2;
    const int per = 2 * Wp + 2 * H;
    for (int i = tid; i < Cb * per; i += NT)
    {
        const int cb = i / per, r = i - cb * per;
        int h, w;
        if (r < Wp) { h = 0; w = r; }
        else if (r < 2 * Wp) { h = Hp - 1; w = r - Wp; }
        else { const int rr = r - 2 * Wp; h = 1 + (rr >> 1); w = (rr & 1) ? Wp - 1 : 0; }
        *reinterpret_cast<uint4 *>(t + ((cb * Hp + h) * Wp + w) * 16) = make_uint4(0, 0, 0, 0);
    }
}

// requant_u8's short form (positive multiplier) with the layer's constants hoisted, in signed arithmetic: a
// non-positive accumulator gives v <= 0, the rounding shift keeps it <= 0 and the clamp returns 0, exactly as the
// unsigned form's explicit test does; a positive one is the same computation.
// The rounding term: the remainder v mod 2^rs exceeds (2^rs - 1) / 2 exactly when its top bit, bit rs - 1 of v, is set
// (never for rs == 0): one bit-field extract instead of a mask, a compare and a carry.
struct FastQ
{
    int32_t mult;
    int ls, rs, bit, width;              // bit = (rs - 1) & 31, width = rs > 0
};
__device__ __forceinline__ uint32_t requant_fast(int32_t acc, const FastQ f)
{
    const int32_t shifted = (int32_t)((uint32_t)acc << f.ls);
    const long long prod = (long long)shifted * (long long)f.mult + (1ll << 30);
    const int32_t v = (int32_t)(prod >> 31);
    const int32_t r = (v >> f.rs) - (int32_t)__builtin_amdgcn_ubfe((uint32_t)v, (uint32_t)f.bit, (uint32_t)f.width);
    return (uint32_t)(r < 0 ? 0 : (r > 255 ? 255 : r));      // v_med3_i32
}

// TP pixel tiles (16 pixels each) of one channel block per wave step, sharing the filter operand.
// NM > 0: the layer has exactly NM MFMA steps (4 K-steps each), the loop is unrolled and the lane's K-step offsets
// live in registers; NM == 0: any count, offsets read from the table per step.
// POST: what follows the requantisation, fixed per instantiation so that the epilogue is straight-line code:
// 3 the short epilogue (see there) without Accum, 4 with Accum: postx[byte + shortcut byte]; -1 decided per layer at run
// time (the general form, also the only one that writes the model's output to global memory); 0 / 1 / 2 are the general
// form's cases nothing / post[] / Accum as compile-time variants (kept for measurements).
template <bool STEM, int TP, int NM, bool FAST, int POST = -1>
__device__ __forceinline__ void conv_tiles(const QMLayer &L, uint8_t *lds, const uint8_t *tab, uint8_t *gout, int tid, int wave,
                                           int n_waves)
{
    const int lane = tid & 63, col = lane & 15, grp = lane >> 4;
    const int CoB = L.Co / CB;
    const int Wp = L.W + 2, Hop = L.Ho + 2, Wop = L.Wo + 2;
    const int P = L.Ho * L.Wo;
    const int n_pt = (P + 15) >> 4;
    const int n_grp = (n_pt + TP - 1) / TP;
    const int n_work = n_grp * CoB;
    const uint8_t *src = lds + L.src_off;
    const int nm = NM > 0 ? NM : (L.S_pad >> 2);
    const int32_t *T = reinterpret_cast<const int32_t *>(tab);
    const int *steps = reinterpret_cast<const int *>(tab + 64 * L.Co);
    const uint8_t *post = tab + 64 * L.Co + 4 * L.S_pad;
    const FastQ fq{L.q.multiplier, L.q.lshift & 31, L.q.rshift, (L.q.rshift - 1) & 31, L.q.rshift > 0 ? 1 : 0};
    constexpr bool GEO = POST >= 3;                   // the short epilogue's layers carry a pixel table
    const uint8_t *geo = tab + L.geo_off;
    // the lane's K-steps: offset from the window origin, and the vector the box sum multiplies by (0 past the end:
    // such a step reads valid memory, its filter rows are zero, and it must not count towards the box sum)
    int so[NM > 0 ? NM : 1], ones[NM > 0 ? NM : 1];
    if (!STEM && NM > 0)
    {
#pragma unroll
        for (int m = 0; m < NM; ++m)
        {
            const int v = steps[4 * m + grp];
            so[m] = v >= 0 ? v : 0;
            ones[m] = v >= 0 ? 0x01010101 : 0;
        }
    }
    const int wo_shift = L.wo_shift;
    const int s_shift = L.stride - 1;                 // stride is 1 or 2

    for (int work = wave; work < n_work; work += n_waves)
    {
        const int pg = (int)(((float)work + 0.5f) * L.r_cob);
        const int cob = work - pg * CoB;
        const uint8_t *wrow = lds + L.w_off + (cob * L.S_pad * 16 + col) * 16 + grp * 256;
        int oh[TP], ow[TP], ih0[TP], iw0[TP];
        int srcoff[TP], dstoff[TP], casoff[TP];      // GEO: the pixel's three offsets out of the layer's pixel table
        bool pvalid[TP];
#pragma unroll
        for (int t = 0; t < TP; ++t)
        {
            const int p = (pg * TP + t) * 16 + col;
            pvalid[t] = p < P;
            const int pc = pvalid[t] ? p : P - 1;
            if (GEO)
            {
                const uint16_t *ge = reinterpret_cast<const uint16_t *>(geo + pc * 4);
                srcoff[t] = ge[0];
                dstoff[t] = ge[1] & 0xfff0;
                casoff[t] = ge[1] & 15;
                oh[t] = ow[t] = ih0[t] = iw0[t] = 0;
                continue;
            }
            srcoff[t] = dstoff[t] = casoff[t] = 0;
            if (wo_shift >= 0) { oh[t] = pc >> wo_shift; ow[t] = pc & (L.Wo - 1); }
            else { oh[t] = (int)(((float)pc + 0.5f) * L.r_wo); ow[t] = pc - oh[t] * L.Wo; }
            ih0[t] = (oh[t] << s_shift) - L.pt;
            iw0[t] = (ow[t] << s_shift) - L.pl;
        }
        // si: the pixel's box sum, from the matrix pipe too (a filter block of ones: every row of the product is the sum
        // of the pixel's bytes over all K-steps, so each lane finds its pixel's sum in its own registers; the pipe is
        // idle most of the time here, the vector ALU is what these layers wait for)
        v4i acc[TP], si[TP];
#pragma unroll
        for (int t = 0; t < TP; ++t) { acc[t] = v4i{0, 0, 0, 0}; si[t] = v4i{0, 0, 0, 0}; }
        if (STEM)
        {
            // one MFMA: K group g = window row g (kw pixels x 4 channels), rows >= kh are zero
            const uint4 A = *reinterpret_cast<const uint4 *>(wrow);
#pragma unroll
            for (int t = 0; t < TP; ++t)
            {
                uint32_t b[4] = {0, 0, 0, 0};
                if (grp < L.kh)
                {
                    const uint32_t *row = GEO ? reinterpret_cast<const uint32_t *>(src + srcoff[t] + __mul24(grp, Wp) * 4)
                                              : reinterpret_cast<const uint32_t *>(src + (__mul24(ih0[t] + grp + 1, Wp) + iw0[t] + 1) * 4);
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (j < L.kw) b[j] = row[j];
                }
                const v4i bv{(int)b[0], (int)b[1], (int)b[2], (int)b[3]};
                si[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{0x01010101, 0x01010101, 0x01010101, 0x01010101}, bv, si[t], 0, 0, 0);
                acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{(int)A.x, (int)A.y, (int)A.z, (int)A.w}, bv, acc[t], 0, 0, 0);
            }
        }
        else
        {
            const uint8_t *pix[TP];
#pragma unroll
            for (int t = 0; t < TP; ++t) pix[t] = GEO ? src + srcoff[t] : src + (__mul24(ih0[t] + 1, Wp) + iw0[t] + 1) * 16;
            if (NM > 0)
            {
#pragma unroll
                for (int m = 0; m < NM; ++m)
                {
                    const uint4 A = *reinterpret_cast<const uint4 *>(wrow + m * 1024);
#pragma unroll
                    for (int t = 0; t < TP; ++t)
                    {
                        const uint4 B = *reinterpret_cast<const uint4 *>(pix[t] + so[m]);
                        const v4i bv{(int)B.x, (int)B.y, (int)B.z, (int)B.w};
                        si[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{ones[m], ones[m], ones[m], ones[m]}, bv, si[t], 0, 0, 0);
                        acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{(int)A.x, (int)A.y, (int)A.z, (int)A.w}, bv, acc[t], 0, 0, 0);
                    }
                }
            }
            else
            {
                for (int m = 0; m < nm; ++m)
                {
                    const int sv = steps[4 * m + grp];
                    const int one = sv >= 0 ? 0x01010101 : 0;
                    const uint4 A = *reinterpret_cast<const uint4 *>(wrow + m * 1024);
#pragma unroll
                    for (int t = 0; t < TP; ++t)
                    {
                        const uint4 B = *reinterpret_cast<const uint4 *>(pix[t] + (sv >= 0 ? sv : 0));
                        const v4i bv{(int)B.x, (int)B.y, (int)B.z, (int)B.w};
                        si[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{one, one, one, one}, bv, si[t], 0, 0, 0);
                        acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{(int)A.x, (int)A.y, (int)A.z, (int)A.w}, bv, acc[t], 0, 0, 0);
                    }
                }
            }
        }
#pragma unroll
        for (int t = 0; t < TP; ++t)
        {
            const int sit = si[t][0];
            if (!pvalid[t]) continue;
            // border case of the pixel -> T
            uint4 tc;
            int opos;
            if (GEO)
            {
                tc = *reinterpret_cast<const uint4 *>(tab + __mul24(casoff[t], L.Co * 4) + (cob * CB + 4 * grp) * 4);
                opos = dstoff[t] + __mul24(cob * Hop, Wop) * 16 + 4 * grp;
            }
            else
            {
                const int ra = (ih0[t] < 0 ? 2 : 0) + (ih0[t] + L.kh > L.H ? 1 : 0);
                const int rb = (iw0[t] < 0 ? 2 : 0) + (iw0[t] + L.kw > L.W ? 1 : 0);
                tc = *reinterpret_cast<const uint4 *>(T + __mul24(ra * 4 + rb, L.Co) + cob * CB + 4 * grp);
                opos = (__mul24(cob * Hop + oh[t] + 1, Wop) + ow[t] + 1) * 16 + 4 * grp;
            }
            const uint32_t tc4[4] = {tc.x, tc.y, tc.z, tc.w};
            const uint32_t base = (uint32_t)L.ZF * (uint32_t)sit;
            if (POST == 3 || POST == 4)
            {
                // The short epilogue (positive multiplier, rshift >= 2, result in LDS).  The requantised byte depends on
                // idx = product >> (30 + rshift) alone, which is the product's high word shifted by rshift - 2: one
                // shift instead of the 64-bit shift, the rounding bit, the subtraction and the post[] address; the clamp
                // is the table's domain.  fin[] holds the byte as the tensors store it, so the four bytes go out as four
                // byte stores with nothing to pack (LDS instructions do not take vector-ALU issue slots; the vector ALU
                // is what this kernel waits for).
                const uint8_t *fin = post + 512, *postx = fin + FIN_BYTES;
                uint8_t *dstp = lds + L.dst_off + opos;
                uint32_t sc = 0;
                if (POST == 4) sc = *reinterpret_cast<const uint32_t *>(lds + L.acc_off + opos) ^ 0x80808080u;
                // all table reads first, then the stores: a store between them would have to be assumed to change the
                // tables (both are LDS) and each read would wait for its own round trip
                uint32_t y[4];
#pragma unroll
                for (int r = 0; r < 4; ++r)
                {
                    const int32_t v = (int32_t)((uint32_t)acc[t][r] + base + tc4[r]);
                    const int32_t shifted = (int32_t)((uint32_t)v << fq.ls);
                    const long long prod = (long long)shifted * (long long)fq.mult + (1ll << 30);
                    int idx = (int32_t)(prod >> 32) >> L.idx_shift;
                    idx = idx < 0 ? 0 : (idx > FIN_ENTRIES - 1 ? FIN_ENTRIES - 1 : idx);
                    y[r] = fin[idx];
                }
                if (POST == 4)
                {
#pragma unroll
                    for (int r = 0; r < 4; ++r) y[r] = postx[y[r] + ((sc >> (8 * r)) & 0xffu)];
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) dstp[r] = (uint8_t)y[r];
                continue;
            }
            uint32_t packed = 0;
            const bool with_acc = POST >= 0 ? POST == 2 : L.acc_off >= 0;
            const bool with_post = POST >= 0 ? POST != 0 : L.has_post != 0;
            if (with_acc)
            {
                const uint32_t sc = *reinterpret_cast<const uint32_t *>(lds + L.acc_off + opos) ^ 0x80808080u;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                {
                    const int32_t v = (int32_t)((uint32_t)acc[t][r] + base + tc4[r]);
                    const uint32_t y = FAST ? requant_fast(v, fq) : requant_u8(v, L.q);
                    packed |= (uint32_t)post[y + ((sc >> (8 * r)) & 0xffu)] << (8 * r);
                }
            }
            else
            {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                {
                    const int32_t v = (int32_t)((uint32_t)acc[t][r] + base + tc4[r]);
                    uint32_t y = FAST ? requant_fast(v, fq) : requant_u8(v, L.q);
                    if (with_post) y = post[y];
                    packed |= y << (8 * r);
                }
            }
            if (POST >= 0) { *reinterpret_cast<uint32_t *>(lds + L.dst_off + opos) = packed ^ 0x80808080u; continue; }
            if (L.dst_off >= 0) *reinterpret_cast<uint32_t *>(lds + L.dst_off + opos) = packed ^ 0x80808080u;
            else *reinterpret_cast<uint32_t *>(gout + ((size_t)(cob * L.Ho + oh[t]) * L.Wo + ow[t]) * 16 + 4 * grp) = packed;
        }
    }
}

template <bool STEM, int TP, int POST>
__device__ __forceinline__ void conv_tiles_nm(const QMLayer &L, uint8_t *lds, const uint8_t *tab, uint8_t *gout, int tid, int wave,
                                              int n_waves)
{
    // the step counts of 3x3 windows over 16, 32 and 64 channels and of 1x1 windows get unrolled loops
    if (STEM) return conv_tiles<true, TP, 1, true, POST>(L, lds, tab, gout, tid, wave, n_waves);
    const int nm = L.S_pad >> 2;
    if (nm == 1) conv_tiles<false, TP, 1, true, POST>(L, lds, tab, gout, tid, wave, n_waves);
    else if (nm == 3) conv_tiles<false, TP, 3, true, POST>(L, lds, tab, gout, tid, wave, n_waves);
    else if (nm == 5) conv_tiles<false, TP, 5, true, POST>(L, lds, tab, gout, tid, wave, n_waves);
    else if (nm == 9) conv_tiles<false, TP, 9, true, POST>(L, lds, tab, gout, tid, wave, n_waves);
    else conv_tiles<false, TP, 0, true, -1>(L, lds, tab, gout, tid, wave, n_waves);
}

template <bool STEM, int TP>
__device__ __forceinline__ void conv_tiles_post(const QMLayer &L, uint8_t *lds, const uint8_t *tab, uint8_t *gout, int tid, int wave,
                                                int n_waves)
{
    // the model's output, and layers the short epilogue does not cover (rshift < 2, no room for a pixel table): the general form
    if (L.dst_off < 0 || L.idx_shift < 0) conv_tiles<STEM, TP, STEM ? 1 : 0, true, -1>(L, lds, tab, gout, tid, wave, n_waves);
    else if (L.acc_off >= 0) conv_tiles_nm<STEM, TP, 4>(L, lds, tab, gout, tid, wave, n_waves);
    else conv_tiles_nm<STEM, TP, 3>(L, lds, tab, gout, tid, wave, n_waves);
}

// waves [wave0, wave0 + n_waves) of the workgroup compute the layer (all 16 but for the first layer)
template <bool STEM>
__device__ __forceinline__ void conv_layer(const QMLayer &L, uint8_t *lds, const uint8_t *tab, uint8_t *gout, int tid, int wave,
                                           int n_waves)
{
    const int n_tiles = ((L.Ho * L.Wo + 15) >> 4) * (L.Co / CB);
    if (L.q.fast)
    {
        if (n_tiles >= 2 * n_waves) conv_tiles_post<STEM, 2>(L, lds, tab, gout, tid, wave, n_waves);
        else conv_tiles_post<STEM, 1>(L, lds, tab, gout, tid, wave, n_waves);
    }
    else
        conv_tiles<STEM, 1, 0, false>(L, lds, tab, gout, tid, wave, n_waves);   // any int32 multiplier: general requantisation
}

// window == whole image: AveragePool2D (sum of x + zI, the caller folds 1/(H*W) into the output scale) or MaxPool2D
// (q_abstract_layer.hpp:286-293: an un-padded window starts from its first RAW byte, then max over x + zI)
__device__ __forceinline__ void pool_layer(const QMLayer &L, uint8_t *lds, int *pool, uint8_t *gout, int tid)
{
    const int C = L.Ci, Cb = C / CB, Hp = L.H + 2, Wp = L.W + 2;
    const uint8_t *src = lds + L.src_off;
    const bool is_max = L.kind == K_POOL_MAX;
    for (int c = tid; c < C; c += NT)
        pool[c] = is_max ? (int)((uint32_t)(src[(((c >> 4) * Hp + 1) * Wp + 1) * 16 + (c & 15)] ^ 0x80u)) : 0;
    if (L.dst_off >= 0)
        for (int i = tid; i < Cb * 9; i += NT)
            *reinterpret_cast<uint4 *>(lds + L.dst_off + i * 16) = make_uint4(0, 0, 0, 0);
    __syncthreads();
    const int parts = NT / C;             // C <= NT is checked when the model is created
    const int HW = L.H * L.W;
    const int c = tid % C, part = tid / C;
    if (part < parts)
    {
        int acc = is_max ? (int)0x80000000 : 0;
        for (int px = part; px < HW; px += parts)
        {
            const int h = px / L.W, w = px - h * L.W;
            const int x = (int)(uint32_t)(src[(((c >> 4) * Hp + h + 1) * Wp + w + 1) * 16 + (c & 15)] ^ 0x80u) + L.zI;
            acc = is_max ? (x > acc ? x : acc) : (int)((uint32_t)acc + (uint32_t)x);
        }
        if (is_max) atomicMax(&pool[c], acc);
        else atomicAdd(&pool[c], acc);
    }
    __syncthreads();
    for (int ch = tid; ch < C; ch += NT)
    {
        const uint32_t y = requant_u8(pool[ch], L.q);
        if (L.dst_off >= 0) lds[L.dst_off + (((ch >> 4) * 3 + 1) * 3 + 1) * 16 + (ch & 15)] = (uint8_t)(y ^ 0x80u);
        else gout[ch] = (uint8_t)y;
    }
}

__global__ __launch_bounds__(NT) void qmodel_u8_kernel(const QMHeader *__restrict__ hdr_dev, const uint8_t *__restrict__ blob,
                                                       const uint8_t *__restrict__ in, uint8_t *__restrict__ out)
{
    HeaderPtr hdr = (HeaderPtr)hdr_dev;
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);       // uniform: tile bookkeeping stays on the scalar unit
    const size_t n = blockIdx.x;
    const int n_layers = hdr->n_layers;

    // the first layer's filter and tables
    {
        const uint4 *s = reinterpret_cast<const uint4 *>(blob);
        uint4 *d = reinterpret_cast<uint4 *>(lds);
        for (int i = tid; i < (hdr->first_bytes >> 4); i += NT) d[i] = s[i];
        if (tid < hdr->layer[0].tab16)
            reinterpret_cast<uint4 *>(lds + hdr->tab_lds)[tid] = reinterpret_cast<const uint4 *>(blob + hdr->layer[0].tab_off)[tid];
    }
    // The filters of all later layers: requested now, by the memory pipeline itself (global memory to LDS without
    // passing through registers, a wave moves one KiB per instruction), and awaited after the first layer has been
    // computed by all sixteen waves: the copy costs the layer neither waves nor registers.
    {
        const int lane = tid & 63;
        const int first = hdr->first_bytes, kib = hdr->later_kib;
        for (int c = wave; c < kib; c += NW)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(blob + first + c * 1024 + lane * 16),
                                             (__attribute__((address_space(3))) void *)(lds + first + c * 1024), 16, 0, 0);
    }
    // the image, re-biased, with its ring of zeros
    {
        const int C = hdr->in_C, H = hdr->in_H, W = hdr->in_W, Hp = H + 2, Wp = W + 2;
        const uint8_t *img = in + n * (size_t)hdr->in_elems;
        if (C < CB)
        {
            uint32_t *d = reinterpret_cast<uint32_t *>(lds + hdr->in_off);
            for (int i = tid; i < Hp * Wp; i += NT)
            {
                const int hp = i / Wp, wp = i - hp * Wp;
                uint32_t v = 0;
                if (hp >= 1 && hp <= H && wp >= 1 && wp <= W)
                {
                    const uint8_t *px = img + ((size_t)(hp - 1) * W + (wp - 1)) * C;
                    for (int c = 0; c < C; ++c) v |= (uint32_t)(px[c] ^ 0x80u) << (8 * c);
                }
                d[i] = v;
            }
        }
        else
        {
            uint4 *d = reinterpret_cast<uint4 *>(lds + hdr->in_off);
            const int Cb = C / CB;
            for (int i = tid; i < Cb * Hp * Wp; i += NT)
            {
                const int wp = i % Wp, hp = (i / Wp) % Hp, cb = i / (Wp * Hp);
                uint4 v = make_uint4(0, 0, 0, 0);
                if (hp >= 1 && hp <= H && wp >= 1 && wp <= W)
                {
                    v = *reinterpret_cast<const uint4 *>(img + ((size_t)(cb * H + hp - 1) * W + (wp - 1)) * 16);
                    v.x ^= 0x80808080u; v.y ^= 0x80808080u; v.z ^= 0x80808080u; v.w ^= 0x80808080u;
                }
                d[i] = v;
            }
        }
    }
    uint8_t *tabs = lds + hdr->tab_lds;
    const int tab_bytes = hdr->tab_bytes;
    int *pool = reinterpret_cast<int *>(lds + hdr->pool_off);
    uint8_t *gout = out + n * (size_t)hdr->out_elems;
    __syncthreads();

    for (int li = 0; li < n_layers; ++li)
    {
        const QMLayer L = load_layer(hdr, li);
        const int cur = li & 1, nxt = cur ^ 1;
        const bool more = li + 1 < n_layers;
        // the next layer's tables: in flight while this layer is computed, stored into the other half afterwards
        uint4 tpre = make_uint4(0, 0, 0, 0);
        const int next_tab16 = more ? hdr->layer[li + 1].tab16 : 0;
        if (tid < next_tab16) tpre = reinterpret_cast<const uint4 *>(blob + hdr->layer[li + 1].tab_off)[tid];
        const uint8_t *tab = tabs + cur * tab_bytes;
        if (L.kind == K_POOL_AVG || L.kind == K_POOL_MAX) pool_layer(L, lds, pool, gout, tid);
        else
        {
            if (L.dst_off >= 0) zero_ring(lds + L.dst_off, L.Co / CB, L.Ho, L.Wo, tid);
            if (L.kind == K_STEM) conv_layer<true>(L, lds, tab, gout, tid, wave, NW);
            else conv_layer<false>(L, lds, tab, gout, tid, wave, NW);
        }
        if (tid < next_tab16) reinterpret_cast<uint4 *>(tabs + nxt * tab_bytes)[tid] = tpre;
        if (li == 0) __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0): this wave's share of the later layers' filters has landed
        __syncthreads();
    }
}

int align_up(int v, int a) { return (v + a - 1) / a * a; }

} // namespace

namespace
{
struct Post
{
    int has_accum, relu;
    int32_t zS, zO;
};
} // namespace

struct small_hip_qmodel
{
    QMHeader hdr;
    void *dev = nullptr;        // [QMHeader][filters (LDS image)][tables of every layer][scratch of the pre-passes]
    size_t blob_off = 0;
    int device = 0;
};

extern "C" {

int small_hip_qmodel_create(int n_layers, const small_hip_qlayer *layers, small_hip_qmodel **model,
                            small_hip_stream_t stream)
{
    const char *op = "small_hip_qmodel_create";
    if (!model) return einval("small_hip_qmodel_create: null result pointer");
    *model = nullptr;
    if (n_layers <= 0 || n_layers > MAX_LAYERS || !layers)
    { set_error("%s: 1..%d layers", op, MAX_LAYERS); return SMALL_HIP_EINVAL; }

    small_hip_qmodel *m = new (std::nothrow) small_hip_qmodel();
    if (!m) return SMALL_HIP_ENOMEM;
    std::memset(&m->hdr, 0, sizeof(m->hdr));
    QMHeader &h = m->hdr;
    h.n_layers = n_layers;
    auto fail = [&](int rc) { delete m; return rc; };

    // geometry, tensor sizes, filter image
    int tensor_bytes[MAX_TENSORS] = {};
    bool written[MAX_TENSORS] = {};
    struct Geo { int Ho, Wo, Co; };
    std::vector<Geo> geo((size_t)n_layers);
    std::vector<int32_t> ZI((size_t)n_layers, 0);
    std::vector<Post> posts((size_t)n_layers);
    int lds_filters = 0, tables = 0, max_t = 0;
    size_t scratch = 0;
    for (int i = 0; i < n_layers; ++i)
    {
        const small_hip_qlayer &l = layers[i];
        QMLayer &L = h.layer[i];
        const bool pool = l.kind == SMALL_HIP_QL_GLOBAL_AVGPOOL || l.kind == SMALL_HIP_QL_GLOBAL_MAXPOOL;
        if (l.kind != SMALL_HIP_QL_CONV && !pool) { set_error("%s: layer %d: unknown kind", op, i); return fail(SMALL_HIP_EINVAL); }
        const int Ci = l.input_channels, H = l.input_height, W = l.input_width;
        if (H <= 0 || W <= 0 || Ci <= 0) { set_error("%s: layer %d: bad size", op, i); return fail(SMALL_HIP_EINVAL); }
        const bool from_input = l.src == SMALL_HIP_QM_INPUT;
        if (from_input != (i == 0)) { set_error("%s: exactly the first layer reads the model input", op); return fail(SMALL_HIP_EINVAL); }
        if (!from_input && (l.src < 0 || l.src >= MAX_TENSORS || !written[l.src]))
        { set_error("%s: layer %d reads a tensor that no earlier layer wrote", op, i); return fail(SMALL_HIP_EINVAL); }
        if (l.dst != SMALL_HIP_QM_OUTPUT && (l.dst < 0 || l.dst >= MAX_TENSORS || l.dst == l.src))
        { set_error("%s: layer %d: bad destination tensor", op, i); return fail(SMALL_HIP_EINVAL); }
        if ((l.dst == SMALL_HIP_QM_OUTPUT) != (i == n_layers - 1))
        { set_error("%s: exactly the last layer writes the model output", op); return fail(SMALL_HIP_EINVAL); }
        if (l.output_q.rshift < 0 || l.output_q.rshift > 31 || l.output_q.lshift < 0 || l.output_q.lshift > 31)
        { set_error("%s: layer %d: shift out of range", op, i); return fail(SMALL_HIP_EINVAL); }
        L.Ci = Ci; L.H = H; L.W = W;
        posts[(size_t)i] = Post{0, l.relu ? 1 : 0, 0, l.output_q.zero};
        L.q = make_qout(l.output_q.multiplier, l.output_q.lshift, l.output_q.rshift);
        L.has_post = l.relu ? 1 : 0;
        L.acc_off = -1;
        if (pool)
        {
            if (Ci % CB != 0 || Ci > NT) { set_error("%s: layer %d: pooling over %d channels", op, i, Ci); return fail(SMALL_HIP_EUNSUPPORTED); }
            if (l.kernel_height != H || l.kernel_width != W || l.t_pad || l.b_pad || l.l_pad || l.r_pad || l.relu ||
                l.accum_src != SMALL_HIP_QM_NONE || from_input)
            { set_error("%s: layer %d: only whole-image pooling without padding, after a convolution", op, i); return fail(SMALL_HIP_EUNSUPPORTED); }
            L.kind = l.kind == SMALL_HIP_QL_GLOBAL_AVGPOOL ? K_POOL_AVG : K_POOL_MAX;
            L.Co = Ci; L.Ho = 1; L.Wo = 1; L.kh = H; L.kw = W; L.stride = 1;
            L.zI = l.input_q.zero;
        }
        else
        {
            const int kh = l.kernel_height, kw = l.kernel_width, s = l.stride, Co = l.output_channels;
            const bool stem = Ci < CB;
            if (stem ? !(Ci >= 1 && Ci <= 3) : Ci % CB != 0) { set_error("%s: layer %d: %d input channels", op, i, Ci); return fail(SMALL_HIP_EUNSUPPORTED); }
            if (stem && !from_input) { set_error("%s: layer %d: 1..3 input channels only on the model input", op, i); return fail(SMALL_HIP_EUNSUPPORTED); }
            if (s != 1 && s != 2) { set_error("%s: layer %d: stride %d", op, i, s); return fail(SMALL_HIP_EUNSUPPORTED); }
            if (kh <= 0 || kw <= 0 || Co <= 0 || Co % CB != 0 || !l.filter || !aligned16(l.filter) ||
                !pads_ok(l.t_pad, l.b_pad, l.l_pad, l.r_pad))
            { set_error("%s: layer %d: bad convolution arguments (output channels: multiples of 16)", op, i); return fail(SMALL_HIP_EINVAL); }
            if (Co > MAX_CO) { set_error("%s: layer %d: more than %d output channels", op, i, MAX_CO); return fail(SMALL_HIP_EUNSUPPORTED); }
            if (stem && (kh > 4 || kw > 4))
            { set_error("%s: layer %d: first-layer windows up to 4x4", op, i); return fail(SMALL_HIP_EUNSUPPORTED); }
            const int Ho = out_dim(H, l.t_pad, l.b_pad, kh, s), Wo = out_dim(W, l.l_pad, l.r_pad, kw, s);
            if (Ho <= 0 || Wo <= 0) { set_error("%s: layer %d: empty output", op, i); return fail(SMALL_HIP_EINVAL); }
            // the tensors carry a ring of one pixel: no tap may fall further outside the image
            if (l.t_pad > 1 || l.l_pad > 1 || (Ho - 1) * s + kh - 1 - l.t_pad > H || (Wo - 1) * s + kw - 1 - l.l_pad > W)
            { set_error("%s: layer %d: padding beyond one pixel", op, i); return fail(SMALL_HIP_EUNSUPPORTED); }
            L.kind = stem ? K_STEM : K_CONV;
            L.Co = Co; L.Ho = Ho; L.Wo = Wo; L.kh = kh; L.kw = kw; L.stride = s; L.pt = l.t_pad; L.pl = l.l_pad;
            const int S = stem ? 4 : kh * kw * (Ci / CB);
            L.S_pad = (S + 3) & ~3;
            if (L.S_pad > MAX_STEPS) { set_error("%s: layer %d: window x channels too large", op, i); return fail(SMALL_HIP_EUNSUPPORTED); }
            ZI[(size_t)i] = (int32_t)((uint32_t)l.input_q.zero + 128u);
            L.ZF = (int32_t)((uint32_t)l.filter_q.zero + 128u);
            L.w_off = lds_filters;
            lds_filters += stem ? Co * 64 : (int)prepared_table_offset_u8(kh, kw, Co, Ci);
            if (i == 0) h.first_bytes = lds_filters;
            L.geo_off = 64 * Co + 4 * L.S_pad + 512 + FIN_BYTES + 512;     // the tables' offsets and sizes: assign_tables below
            const size_t need = stem ? (size_t)Co * (kh + 1) * (kw + 1) * 4 : prepared_bytes_u8(kh, kw, Co, Ci);
            scratch = need > scratch ? need : scratch;
            if (l.accum_src != SMALL_HIP_QM_NONE)
            {
                // the Accum source may be the destination itself (a residual sum accumulated in place, as the reference's
                // PartialConv2DLayer does): a lane reads its four bytes of it before it writes them
                if (l.accum_src < 0 || l.accum_src >= MAX_TENSORS || !written[l.accum_src] || l.accum_src == l.src ||
                    l.dst == SMALL_HIP_QM_OUTPUT)
                { set_error("%s: layer %d: bad Accum source", op, i); return fail(SMALL_HIP_EINVAL); }
                posts[(size_t)i].has_accum = 1;
                posts[(size_t)i].zS = l.accum_q.zero;
                L.has_post = 1;
            }
        }
        // the short epilogue: positive multiplier, rshift >= 2, the result stays in LDS (conv_tiles)
        // (and the pixel table's 16-bit offsets must reach every pixel of the input and output tensors)
        L.idx_shift = (!pool && L.q.fast && L.q.rshift >= 2 && l.dst != SMALL_HIP_QM_OUTPUT && (H + 2) * (W + 2) * 16 <= 0xffff &&
                       (L.Ho + 2) * (L.Wo + 2) * 16 <= 0xffff)
                          ? L.q.rshift - 2
                          : -1;
        L.r_wo = 1.0f / (float)L.Wo;
        L.r_cob = 1.0f / (float)(L.Co / CB);
        L.wo_shift = -1;
        for (int b = 0; b < 16; ++b)
            if (L.Wo == (1 << b)) L.wo_shift = b;
        geo[(size_t)i] = Geo{L.Ho, L.Wo, L.Co};
        if (l.dst >= 0)
        {
            const int bytes = (L.Co / CB) * (L.Ho + 2) * (L.Wo + 2) * 16;
            tensor_bytes[l.dst] = bytes > tensor_bytes[l.dst] ? bytes : tensor_bytes[l.dst];
            written[l.dst] = true;
        }
    }
    // a layer's input (and Accum source) is what the last writer of that tensor produced: shapes must agree
    for (int i = 1; i < n_layers; ++i)
    {
        int w = -1;
        for (int j = 0; j < i; ++j)
            if (layers[j].dst == layers[i].src) w = j;
        if (w < 0 || geo[(size_t)w].Ho != layers[i].input_height || geo[(size_t)w].Wo != layers[i].input_width ||
            geo[(size_t)w].Co != layers[i].input_channels)
        { set_error("%s: layer %d: input shape differs from what layer %d produces", op, i, w); return fail(SMALL_HIP_EINVAL); }
        if (layers[i].kind != SMALL_HIP_QL_CONV || layers[i].accum_src == SMALL_HIP_QM_NONE) continue;
        w = -1;
        for (int j = 0; j < i; ++j)
            if (layers[j].dst == layers[i].accum_src) w = j;
        if (w < 0 || geo[(size_t)w].Ho != geo[(size_t)i].Ho || geo[(size_t)w].Wo != geo[(size_t)i].Wo || geo[(size_t)w].Co != geo[(size_t)i].Co)
        { set_error("%s: layer %d: Accum source has another shape", op, i); return fail(SMALL_HIP_EINVAL); }
    }

    // LDS plan: [filters][tables x2][pooling sums][input][tensors]; the later layers' filters are copied in whole KiB
    h.filter_bytes = lds_filters;
    h.later_kib = (lds_filters - h.first_bytes + 1023) >> 10;
    const int filters_end = h.first_bytes + (h.later_kib << 10);
    const small_hip_qlayer &l0 = layers[0];
    h.in_C = l0.input_channels; h.in_H = l0.input_height; h.in_W = l0.input_width;
    h.in_elems = h.in_C * h.in_H * h.in_W;
    int tensor_off[MAX_TENSORS];
    int off = 0;
    // The pixel tables of the short epilogue are the one part of the plan that is optional: a layer whose table would
    // not fit the table fetch (one 16-byte piece per thread) goes without, and so do all layers when the model would not
    // fit LDS with them; those layers take the general epilogue.
    for (int with_pixels = 1; with_pixels >= 0; --with_pixels)
    {
        tables = 0; max_t = 0;
        for (int i = 0; i < n_layers; ++i)
        {
            QMLayer &L = h.layer[i];
            if (L.kind != K_STEM && L.kind != K_CONV) continue;
            int tb = L.geo_off;
            const int with_table = tb + ((L.Ho * L.Wo * 4 + 15) & ~15);
            if (with_pixels && L.idx_shift >= 0 && (with_table >> 4) <= NT) tb = with_table;
            else L.idx_shift = -1;
            L.tab_off = tables;                    // relative to the table area, fixed up below
            L.tab16 = tb >> 4;
            tables += tb;
            max_t = tb > max_t ? tb : max_t;
        }
        off = align_up(filters_end, 16);
        h.tab_lds = off; h.tab_bytes = max_t; off += 2 * max_t;
        int pool_c = 0;
        for (int i = 0; i < n_layers; ++i)
            if (h.layer[i].kind == K_POOL_AVG || h.layer[i].kind == K_POOL_MAX) pool_c = h.layer[i].Ci > pool_c ? h.layer[i].Ci : pool_c;
        h.pool_off = off; off += align_up(pool_c * 4, 16);
        h.in_off = off;
        off += align_up((h.in_C < CB ? 4 : h.in_C) * (h.in_H + 2) * (h.in_W + 2), 16);
        for (int t = 0; t < MAX_TENSORS; ++t) { tensor_off[t] = off; off += tensor_bytes[t]; }
        h.lds_bytes = off;
        if (off <= LDS_LIMIT) break;
    }
    if (off > LDS_LIMIT)
    {
        set_error("%s: the model needs %d bytes of LDS (filters %d), the limit is %d: run it layer by layer", op, off,
                  lds_filters, LDS_LIMIT);
        return fail(SMALL_HIP_EUNSUPPORTED);
    }
    const int table_base = align_up(filters_end, 256);      // the copy reads the blob up to filters_end
    for (int i = 0; i < n_layers; ++i)
    {
        QMLayer &L = h.layer[i];
        L.src_off = i == 0 ? h.in_off : tensor_off[layers[i].src];
        L.dst_off = layers[i].dst >= 0 ? tensor_off[layers[i].dst] : -1;
        if (L.kind == K_STEM || L.kind == K_CONV) L.tab_off += table_base;
        if (layers[i].kind == SMALL_HIP_QL_CONV && layers[i].accum_src != SMALL_HIP_QM_NONE) L.acc_off = tensor_off[layers[i].accum_src];
    }
    const QMLayer &last = h.layer[n_layers - 1];
    h.out_elems = last.Co * last.Ho * last.Wo;

    // device side: header, filter image, T tables; the pre-passes work through a scratch block behind them
    hipStream_t s = as_stream(stream);
    hipError_t e = hipGetDevice(&m->device);
    if (e != hipSuccess) return fail(fail_hip(e, "hipGetDevice"));
    m->blob_off = (sizeof(QMHeader) + 255) & ~(size_t)255;
    const size_t scratch_off = ((size_t)table_base + (size_t)tables + 255) & ~(size_t)255;
    e = hipMalloc(&m->dev, m->blob_off + scratch_off + scratch + 256);
    if (e != hipSuccess)
    {
        (void)hipGetLastError();
        set_error("%s: hipMalloc: %s", op, hipGetErrorString(e));
        return fail(e == hipErrorOutOfMemory ? SMALL_HIP_ENOMEM : SMALL_HIP_EHIP);
    }
    auto fail_dev = [&](int rc) { (void)hipFree(m->dev); return fail(rc); };
    uint8_t *dblob = static_cast<uint8_t *>(m->dev) + m->blob_off;
    uint8_t *tmp = dblob + scratch_off;
    std::vector<std::vector<uint8_t>> host_tabs((size_t)n_layers);     // alive until the stream has been waited for
    for (int i = 0; i < n_layers; ++i)
    {
        const QMLayer &L = h.layer[i];
        const small_hip_qlayer &l = layers[i];
        const int32_t *P = nullptr;
        if (L.kind == K_CONV)
        {
            // filter + prefix table into the scratch block, the filter part from there into the image
            if (int rc = prepare_filter_u8(L.kh, L.kw, L.Co, L.Ci, l.filter, tmp, s)) return fail_dev(rc);
            const int n16 = (int)(prepared_table_offset_u8(L.kh, L.kw, L.Co, L.Ci) >> 4);
            hipLaunchKernelGGL(qm_copy16_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, s,
                               reinterpret_cast<const uint4 *>(tmp), reinterpret_cast<uint4 *>(dblob + L.w_off), n16);
            P = reinterpret_cast<const int32_t *>(tmp + prepared_table_offset_u8(L.kh, L.kw, L.Co, L.Ci));
        }
        else if (L.kind == K_STEM)
        {
            hipLaunchKernelGGL(qm_prep_stem_kernel, dim3((unsigned)((L.Co * 4 + 255) / 256)), dim3(256), 0, s, l.filter,
                               reinterpret_cast<int8_t *>(dblob + L.w_off), reinterpret_cast<int32_t *>(tmp), L.Co, L.Ci,
                               L.kh, L.kw);
            P = reinterpret_cast<const int32_t *>(tmp);
        }
        else
            continue;
        hipLaunchKernelGGL(qm_case_table_kernel, dim3((unsigned)((16 * L.Co + 255) / 256)), dim3(256), 0, s, P,
                           reinterpret_cast<int32_t *>(dblob + L.tab_off), L.Co, L.Ci, L.kh, L.kw, ZI[(size_t)i], L.ZF);
        e = hipGetLastError();
        if (e != hipSuccess) return fail_dev(fail_hip(e, "small_hip_qmodel_create: pre-pass"));
        // steps[s]: LDS offset of K-step s (tap a, b; channel block) relative to the pixel's window origin, -1 past
        // the end; post[t]: what Accum (t = convolution byte + shortcut byte) and / or the in-place ReLU make of a
        // convolution's byte.  Both are plain functions of the layer's constants: computed here, once.
        std::vector<uint8_t> &hb = host_tabs[(size_t)i];
        hb.assign((size_t)(L.tab16 * 16 - 64 * L.Co), 0);
        int32_t *st = reinterpret_cast<int32_t *>(hb.data());
        const int CiB = L.kind == K_CONV ? L.Ci / CB : 1, Hp = L.H + 2, Wp = L.W + 2, S = L.kind == K_CONV ? L.kh * L.kw * CiB : 4;
        for (int k = 0; k < L.S_pad; ++k)
        {
            st[k] = -1;
            if (k < S && L.kind == K_CONV)
            {
                const int tap = k / CiB, cib = k - tap * CiB, a = tap / L.kw, b = tap - a * L.kw;
                st[k] = ((cib * Hp + a) * Wp + b) * 16;
            }
        }
        const Post &pa = posts[(size_t)i];
        uint8_t *po = hb.data() + 4 * L.S_pad;
        for (int t = 0; t < 511; ++t)
        {
            uint32_t y = (uint32_t)t;
            if (pa.has_accum) y = requant_u8((int32_t)((uint32_t)t + (uint32_t)pa.zS + (uint32_t)pa.zO), L.q);
            else if (t > 255) break;
            if (pa.relu)
            {
                const int32_t z = (int32_t)y + pa.zO;
                y = requant_u8(z > 0 ? z : 0, L.q);
            }
            po[t] = (uint8_t)y;
        }
        // The short epilogue's tables.  With a positive multiplier and rshift >= 2 the requantised byte is a function of
        // idx = product >> (30 + rshift) alone: idx = 2 q + b with q = v >> rshift and b = bit rshift - 1 of v, and the
        // reference's result is clamp(q - b, 0, 255) (its rounding term is -1).  fin[clamp(idx, 0, 513)] is that byte after
        // post[] and in the tensors' encoding (^ 0x80); in front of an Accum it is the plain byte, and postx[] is post[]
        // in the tensors' encoding.
        {
            uint8_t *fin = po + 512, *postx = fin + FIN_BYTES;
            for (int idx = 0; idx < FIN_ENTRIES; ++idx)
            {
                const int r = (idx >> 1) - (idx & 1);
                const uint8_t y = (uint8_t)(r < 0 ? 0 : r > 255 ? 255 : r);
                fin[idx] = pa.has_accum ? y : (uint8_t)((L.has_post ? po[y] : y) ^ 0x80u);
            }
            for (int t = 0; t < 512; ++t) postx[t] = (uint8_t)(po[t] ^ 0x80u);
            // The pixel table: everything the kernel needs to know about output pixel p, as two 16-bit words: the LDS
            // offset of its window origin in the input tensor's first channel block, and the offset of the pixel in the
            // output tensor's first channel block (a multiple of 16) with its border case (the row of T) in the low four
            // bits.  Two LDS reads from one address instead of some thirty vector instructions of index arithmetic per tile.
            uint16_t *ge = reinterpret_cast<uint16_t *>(postx + 512);
            const int Wop = L.Wo + 2, esz = L.kind == K_STEM ? 4 : 16;
            for (int pp = 0; L.idx_shift >= 0 && pp < L.Ho * L.Wo; ++pp)
            {
                const int oh = pp / L.Wo, ow = pp - oh * L.Wo;
                const int ih0 = oh * L.stride - L.pt, iw0 = ow * L.stride - L.pl;
                const int ra = (ih0 < 0 ? 2 : 0) + (ih0 + L.kh > L.H ? 1 : 0), rb = (iw0 < 0 ? 2 : 0) + (iw0 + L.kw > L.W ? 1 : 0);
                ge[2 * pp + 0] = (uint16_t)(((ih0 + 1) * Wp + iw0 + 1) * esz);
                ge[2 * pp + 1] = (uint16_t)((((oh + 1) * Wop + ow + 1) * 16) | (ra * 4 + rb));
            }
        }
        e = hipMemcpyAsync(dblob + L.tab_off + 64 * L.Co, hb.data(), hb.size(), hipMemcpyHostToDevice, s);
        if (e != hipSuccess) return fail_dev(fail_hip(e, "small_hip_qmodel_create: tables"));
    }
    e = hipMemcpyAsync(m->dev, &m->hdr, sizeof(QMHeader), hipMemcpyHostToDevice, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);       // the caller's filters and the host-side tables may go
    if (e != hipSuccess) return fail_dev(fail_hip(e, "small_hip_qmodel_create: upload"));
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(qmodel_u8_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            LDS_LIMIT);
    if (e != hipSuccess) return fail_dev(fail_hip(e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)"));
    *model = m;
    return SMALL_HIP_OK;
}

int small_hip_qmodel_forward(const small_hip_qmodel *model, int batch, const uint8_t *input, uint8_t *output,
                             small_hip_stream_t stream)
{
    if (!model || !model->dev) return einval("small_hip_qmodel_forward: null model");
    if (batch < 0 || !input || !output) return einval("small_hip_qmodel_forward: bad argument");
    if (batch == 0) return SMALL_HIP_OK;
    if (model->hdr.in_C >= CB && !aligned16(input)) return einval("small_hip_qmodel_forward: misaligned input");
    if (!aligned16(output)) return einval("small_hip_qmodel_forward: misaligned output");
    const uint8_t *dblob = static_cast<const uint8_t *>(model->dev) + model->blob_off;
    hipLaunchKernelGGL(qmodel_u8_kernel, dim3((unsigned)batch), dim3(NT), (size_t)model->hdr.lds_bytes, as_stream(stream),
                       static_cast<const QMHeader *>(model->dev), dblob, input, output);
    SHP_LAUNCH_CHECK("small_hip_qmodel_forward");
    return SMALL_HIP_OK;
}

size_t small_hip_qmodel_output_bytes(const small_hip_qmodel *model) { return model ? (size_t)model->hdr.out_elems : 0; }
size_t small_hip_qmodel_lds_bytes(const small_hip_qmodel *model) { return model ? (size_t)model->hdr.lds_bytes : 0; }

int small_hip_qmodel_destroy(small_hip_qmodel *model)
{
    if (!model) return SMALL_HIP_OK;
    int rc = SMALL_HIP_OK;
    if (model->dev)
    {
        hipError_t e = hipFree(model->dev);
        if (e != hipSuccess) rc = fail_hip(e, "small_hip_qmodel_destroy: hipFree");
    }
    delete model;
    return rc;
}

} // extern "C"
