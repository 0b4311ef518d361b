// Requantisation int32 -> uint8 (device code; also callable on the host for tables built at set-up), bit-for-bit the reference's
// VQRDMULH + RNDRSHIFT + clamp (include/small/platforms/reference/intrinsics_quint8.h:481-531).
#pragma once

#include <hip/hip_runtime.h>
#include <cstdint>

namespace shp
{

struct QOut
{
    int32_t multiplier;
    int32_t lshift;
    int32_t rshift;
    int32_t fast;      // multiplier > 0 and 0 <= rshift <= 30: requant_u8 may take its short form
};

// host side: the requantisation fields of an output buffer
inline QOut make_qout(int32_t multiplier, int32_t lshift, int32_t rshift)
{
    return QOut{multiplier, lshift, rshift, (multiplier > 0 && rshift >= 0 && rshift <= 30) ? 1 : 0};
}

__host__ __device__ __forceinline__ int32_t requant_i32(int32_t acc, const QOut q)
{
    // val * (1 << lshift) in 32-bit wrap-around arithmetic, then widened to 64 bits
    const int32_t shifted = (int32_t)((uint32_t)acc << (q.lshift & 31));
    const long long a = (long long)shifted;
    const long long b = (long long)q.multiplier;
    const bool overflow = (a == b) && (a == -2147483648LL);
    const long long prod = a * b;
    const long long nudged = prod + (prod >= 0 ? (long long)(1 << 30) : (long long)(1 - (1 << 30)));
    // C++ '/' by 2^31: truncation toward zero
    const long long adj = nudged + ((nudged >> 63) & 0x7fffffffLL);
    int32_t v = overflow ? 2147483647 : (int32_t)(adj >> 31);
    const int rs = q.rshift;
    const int32_t mask = (int32_t)((1LL << rs) - 1);
    const int32_t mod = v & mask;
    const int32_t threshold = (mask >> 1) + ((v < 0) ? -1 : 0);
    // the reference's rounding term is -1 ("one" is ~0 there), reproduced on purpose
    return (v >> rs) + ((mod > threshold) ? -1 : 0);
}

// requant_i32 clamped to 0..255.  With a positive multiplier (every practical scale) the clamp makes
// most of the general form redundant, and the short form below returns the same byte:
//   - a non-positive (shifted) accumulator gives a product <= 0, VQRDMULH then returns v <= 0, the
//     rounding shift keeps it <= 0 and the clamp makes it 0;
//   - a positive one gives 0 < product < 2^62, the overflow case (both factors INT32_MIN) cannot
//     occur, truncation equals the arithmetic shift, v = (product + 2^30) >> 31 fits 31 bits, and
//     the rounding term is -1 exactly when (v & mask) > (mask >> 1).
// About 10 instructions instead of 25; these kernels are bound by this arithmetic.
__host__ __device__ __forceinline__ uint32_t requant_u8(int32_t acc, const QOut q)
{
    if (q.fast)
    {
        const int32_t shifted = (int32_t)((uint32_t)acc << (q.lshift & 31));
        const uint64_t prod = (uint64_t)(uint32_t)shifted * (uint64_t)(uint32_t)q.multiplier + (1ull << 30);
        const uint32_t v = (uint32_t)(prod >> 31);
        // (v mod 2^rshift) > (2^rshift - 1) / 2 exactly when bit rshift - 1 of v is set (never for rshift == 0)
        const uint32_t round_bit = (v >> ((q.rshift - 1) & 31)) & (q.rshift > 0 ? 1u : 0u);
        const int32_t r = (int32_t)(v >> q.rshift) - (int32_t)round_bit;   // -1 is possible
        const int32_t c = r < 0 ? 0 : (r > 255 ? 255 : r);
        return shifted > 0 ? (uint32_t)c : 0u;
    }
    const int32_t r = requant_i32(acc, q);
    return (uint32_t)(r > 0 ? (r < 255 ? r : 255) : 0);
}

} // namespace shp
