/*
 * conv_inl.h -- software 16-bit <-> 32-bit float conversions shared by the CPU checker's
 * translation units (test infrastructure, see ft_oracle.h). Integer arithmetic only, so the
 * result does not depend on which conversion instructions the host CPU has.
 *
 * fp32 -> fp16 reproduces what the reference's copy-out instruction does
 * (flextrain/ops/csrc/includes/simd.h:35-37: _mm512_cvtps_ph(..., _MM_FROUND_TO_NEAREST_INT)):
 * IEEE round-to-nearest-even, overflow to infinity, gradual underflow, NaN quieted with the top
 * mantissa bits kept.
 */
#ifndef FT_ORACLE_CONV_INL_H
#define FT_ORACLE_CONV_INL_H

#include <stdint.h>
#include <string.h>

static inline uint32_t fto_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    return u;
}

static inline float fto_float(uint32_t u)
{
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

static inline uint16_t fto_f32_to_f16(float f)
{
    const uint32_t x = fto_bits(f);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t a = x & 0x7fffffffu;

    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x03ffu)); /* NaN */
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 2^16 (inf included) */

    const uint32_t e = a >> 23;
    uint32_t h, rem, half;
    if (e >= 113u) { /* normal half: 2^-14 <= |f| */
        const uint32_t mant = a & 0x007fffffu;
        h = ((e - 112u) << 10) | (mant >> 13);
        rem = mant & 0x1fffu;
        half = 0x1000u;
    } else if (e >= 102u) { /* subnormal half (or rounds up into the smallest normal) */
        const uint32_t mant = (a & 0x007fffffu) | 0x00800000u;
        const uint32_t shift = 126u - e; /* 14 .. 24 */
        h = mant >> shift;
        rem = mant & ((1u << shift) - 1u);
        half = 1u << (shift - 1u);
    } else {
        return sign; /* |f| < 2^-25 rounds to zero */
    }
    if (rem > half || (rem == half && (h & 1u))) h += 1u; /* carry may reach 0x7c00 = inf */
    return (uint16_t)(sign | h);
}

static inline uint16_t fto_f32_to_bf16(float f)
{
    const uint32_t x = fto_bits(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u); /* NaN */
    return (uint16_t)((x + 0x7fffu + ((x >> 16) & 1u)) >> 16);
}

static inline float fto_bf16_to_f32(uint16_t h)
{
    return fto_float((uint32_t)h << 16);
}

static inline float fto_f16_to_f32(uint16_t h)
{
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu;
    uint32_t mant = h & 0x03ffu;
    if (e == 0x1fu) return fto_float(sign | 0x7f800000u | (mant << 13));
    if (e != 0u) return fto_float(sign | ((e + 112u) << 23) | (mant << 13));
    if (mant == 0u) return fto_float(sign);
    /* subnormal half: value = mant * 2^-24, exact in fp32 */
    uint32_t shift = 0;
    while (!(mant & 0x0400u)) {
        mant <<= 1;
        ++shift;
    }
    return fto_float(sign | ((113u - shift) << 23) | ((mant & 0x03ffu) << 13));
}

#endif
