// Device-side requantisation int32 -> uint8, bit-for-bit the reference's
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
};

__device__ __forceinline__ int32_t requant_i32(int32_t acc, const QOut q)
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

__device__ __forceinline__ uint32_t requant_u8(int32_t acc, const QOut q)
{
    const int32_t r = requant_i32(acc, q);
    return (uint32_t)(r > 0 ? (r < 255 ? r : 255) : 0);
}

} // namespace shp
