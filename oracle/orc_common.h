/*
 * orc_common.h -- number formats and the seeded generator shared by the CPU oracle.
 *
 * TEST INFRASTRUCTURE. The oracle is a CPU restatement of the definitions the routed-expert path is held to.
 * It is the checker of tests, of the smoke run and of the benchmark's CPU baseline; it is never the product
 * path and nothing under anemone_amd/ links or calls it.
 *
 * Every conversion here is written from the IEEE 754 / OCP definitions of the formats:
 *   binary16  1 sign, 5 exponent (bias 15), 10 fraction bits
 *   bfloat16  the upper 16 bits of a binary32
 *   E4M3      1 sign, 4 exponent (bias 7), 3 fraction bits, no infinities, 0x7F/0xFF not a number, largest 448
 *   E2M1      1 sign, 2 exponent, 1 fraction bit: magnitudes {0, .5, 1, 1.5, 2, 3, 4, 6}
 *   E8M0      a power of two, 2^(code - 127)
 * Reference citations: tools/measure/trellis_reference.h:57-104 (binary16 and E4M3 by their fields),
 * tests/weight_format_reference.c:73,99-119 (E2M1 / E4M3 / E8M0 tables).
 */
#ifndef ORC_COMMON_H
#define ORC_COMMON_H

#include <math.h>
#include <stdint.h>
#include <string.h>

static inline uint32_t orc_f32_bits(float value)
{
    uint32_t bits;
    memcpy(&bits, &value, sizeof bits);
    return bits;
}

static inline float orc_f32_from_bits(uint32_t bits)
{
    float value;
    memcpy(&value, &bits, sizeof value);
    return value;
}

/* binary16 -> double, exact */
static inline double orc_half_value(uint16_t bits)
{
    const uint32_t exponent = (bits >> 10) & 31u, fraction = bits & 1023u;
    double magnitude;
    if (exponent == 31u) {
        magnitude = fraction == 0 ? INFINITY : NAN;
    } else if (exponent == 0u) {
        magnitude = ldexp((double)fraction, -24);
    } else {
        magnitude = ldexp((double)(fraction + 1024u), (int)exponent - 25);
    }
    return (bits & 0x8000u) ? -magnitude : magnitude;
}

/* double -> binary16, one rounding: to nearest, ties to even; 65520 and above to infinity; NaN to 0x7E00 */
static inline uint16_t orc_half_from_double(double value)
{
    if (value != value) {
        return 0x7E00u;
    }
    const uint16_t sign = signbit(value) ? 0x8000u : 0u;
    const double magnitude = fabs(value);
    if (magnitude >= 65520.0) {
        return (uint16_t)(sign | 0x7C00u);
    }
    if (magnitude == 0.0) {
        return sign;
    }
    int exponent;
    (void)frexp(magnitude, &exponent); /* magnitude in [2^(exponent-1), 2^exponent) */
    int binade = exponent - 1;
    if (binade < -14) {
        binade = -14;
    }
    /* units of the last place of the binade; nearbyint rounds ties to even in the default mode */
    const double units = nearbyint(ldexp(magnitude, 10 - binade));
    const uint32_t whole = (uint32_t)units; /* 0..2048 */
    uint32_t bits;
    if (exponent - 1 < -14) {
        bits = whole; /* subnormal, or 1024 = the least normal */
    } else {
        bits = ((uint32_t)(binade + 15) << 10) + (whole - 1024u); /* a carry to 2048 steps the exponent */
    }
    return (uint16_t)(sign | bits);
}

static inline float orc_half_to_float(uint16_t bits)
{
    return (float)orc_half_value(bits); /* every binary16 is a binary32 */
}

static inline uint16_t orc_half_from_float(float value)
{
    return orc_half_from_double((double)value); /* float -> double is exact, so this is one rounding */
}

static inline float orc_bf16_to_float(uint16_t bits)
{
    return orc_f32_from_bits((uint32_t)bits << 16);
}

/* binary32 -> bfloat16: to nearest, ties to even; a NaN becomes 0x7FC0 */
static inline uint16_t orc_bf16_from_float(float value)
{
    const uint32_t bits = orc_f32_bits(value);
    if (value != value) {
        return 0x7FC0u;
    }
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

/* E4M3 code -> double by its fields (0x7F and 0xFF read by their fields give 480; callers never store them) */
static inline double orc_e4m3_value(uint32_t code)
{
    const uint32_t exponent = (code >> 3) & 15u, fraction = code & 7u;
    const double magnitude =
        exponent == 0 ? ldexp((double)fraction, -9) : ldexp((double)(8u + fraction), (int)exponent - 10);
    return (code & 0x80u) ? -magnitude : magnitude;
}

/* E2M1 code (4 bits) -> double */
static inline double orc_e2m1_value(uint32_t code)
{
    static const double magnitudes[8] = {0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0};
    const double magnitude = magnitudes[code & 7u];
    return (code & 8u) ? -magnitude : magnitude;
}

static inline double orc_e8m0_value(uint32_t code)
{
    return ldexp(1.0, (int)code - 127);
}

/* splitmix64: the one generator of every synthetic tensor (the reference's tests seed theirs the same way,
 * tests/exl3_widths_test.c:103-110). */
static inline uint64_t orc_splitmix64(uint64_t *state)
{
    uint64_t z = (*state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* FNV-1a over bytes, 64 bits: digests of the larger fixtures */
static inline uint64_t orc_fnv1a64(const void *bytes, uint64_t count)
{
    const unsigned char *p = (const unsigned char *)bytes;
    uint64_t hash = 0xCBF29CE484222325ull;
    for (uint64_t i = 0; i < count; i++) {
        hash = (hash ^ p[i]) * 0x100000001B3ull;
    }
    return hash;
}

#endif
