/*
 * quantize_device.cuh -- one value of the per-32 activation quantizer (source/kernel_activation_quantize.cuh:52-133,
 * include/anemone/linear_records.h:20-44 of the reference), shared by the quantizer's own kernel and by the producer
 * (gate with up and the quantization of the hidden vectors in one launch). The 32 values of a block sit in 32
 * consecutive lanes of a wavefront (lane % 32 = index % 32); every lane calls with its value.
 */
#ifndef QUANTIZE_DEVICE_CUH
#define QUANTIZE_DEVICE_CUH

#include "exl3_device.cuh"

/* the scale code of a block whose largest magnitude is `largest`: the smallest power of two at least
 * max(largest, 1e-4) / 448, as its biased exponent */
__device__ static __forceinline__ uint32_t quantize_exponent_code(float largest)
{
    const uint32_t ratio = __float_as_uint(__fmul_rn(fmaxf(largest, 1e-4f), 1.0f / 448.0f));
    return ((ratio >> 23) & 255u) + ((ratio & 0x7FFFFFu) != 0u ? 1u : 0u);
}

/* one bfloat16 value under its block's scale code: its E4M3 code (to nearest even, clamped at 448) and its operand.
 * The definition, in plain arithmetic; the kernels use quantize_codes4 below, which the library's arithmetic_selfcheck
 * kernel compares with it over every value and every scale code. */
__device__ static __forceinline__ void quantize_code_defined(uint32_t bits, uint32_t code_exponent, uint32_t &code_out, uint32_t &operand_out)
{
    const float value = bf16_to_float((uint16_t)bits);
    const float scaled = __fmul_rn(value, __uint_as_float((254u - code_exponent) << 23)); /* exact: a power of two */
    const float magnitude = fminf(fabsf(scaled), 448.0f);
    const uint32_t field = __float_as_uint(fmaxf(magnitude, 0.015625f)) >> 23; /* at least 2^-6's */
    /* units of 1/8 of the binade (2^-9 below 2^-6): 0 .. 16, to nearest even */
    const uint32_t units = (uint32_t)__builtin_rintf(__fmul_rn(magnitude, __uint_as_float((257u - field) << 23)));
    const uint32_t sign = (bits >> 8) & 0x80u;
    code_out = (((field - 120u) << 3) + units - 8u) | sign;
    /* the operand: units x 2^(field - 130) x 2^(c - 127) x 2^100, exact, its upper half a bfloat16 */
    const float carried = __fmul_rn((float)units, __uint_as_float((field + code_exponent - 30u) << 23));
    operand_out = (code_exponent <= 146u ? __float_as_uint(carried) >> 16 : 0x7F80u) | (sign << 8);
}

/* Four values of one block at once, by the card's own conversions: the scaled value, limited to 448 in magnitude (a
 * NaN becomes 448) under the value's sign, goes through v_cvt_pk_fp8_f32 (E4M3, to nearest even, subnormals of 2^-9);
 * the operand is the code converted back (v_cvt_pk_f32_fp8) times 2^(c - 27), exact, whose upper half is the
 * bfloat16. codes: byte i the code of bits[i]; carried[i]: the operand of bits[i] in the upper half of the word, to be
 * paired by quantize_operand_pair. */
__device__ static __forceinline__ void quantize_codes4(const uint32_t (&bits)[4], uint32_t code_exponent, uint32_t &codes, uint32_t (&carried)[4])
{
    const float down = __uint_as_float((254u - code_exponent) << 23);
    const float up = __uint_as_float(((code_exponent <= 146u ? code_exponent : 146u) + 100u) << 23);
    float held[4];
#pragma unroll
    for (uint32_t i = 0; i < 4u; i++) {
        const uint32_t value = bits[i] << 16;
        const float magnitude = fminf(fabsf(__fmul_rn(__uint_as_float(value), down)), 448.0f);
        held[i] = __uint_as_float((__float_as_uint(magnitude) & 0x7FFFFFFFu) | (value & 0x80000000u));
    }
    int packed = __builtin_amdgcn_cvt_pk_fp8_f32(held[0], held[1], 0, false);
    packed = __builtin_amdgcn_cvt_pk_fp8_f32(held[2], held[3], packed, true);
    codes = (uint32_t)packed;
    const auto low = __builtin_amdgcn_cvt_pk_f32_fp8(packed, false), high = __builtin_amdgcn_cvt_pk_f32_fp8(packed, true);
    carried[0] = __float_as_uint(__fmul_rn(low[0], up));
    carried[1] = __float_as_uint(__fmul_rn(low[1], up));
    carried[2] = __float_as_uint(__fmul_rn(high[0], up));
    carried[3] = __float_as_uint(__fmul_rn(high[1], up));
}

/* two operands as one word (first in the low half); a scale code above 146 makes every operand an infinity of its sign */
__device__ static __forceinline__ uint32_t quantize_operand_pair(uint32_t first, uint32_t second, uint32_t code_exponent)
{
    const uint32_t pair = __builtin_amdgcn_perm(second, first, 0x07060302u);
    return code_exponent <= 146u ? pair : (pair & 0x80008000u) | 0x7F807F80u;
}

/* one value by the same route (the three others zero) */
__device__ static __forceinline__ void quantize_code(uint32_t bits, uint32_t code_exponent, uint32_t &code_out, uint32_t &operand_out)
{
    const uint32_t four[4] = {bits, 0u, 0u, 0u};
    uint32_t codes, carried[4];
    quantize_codes4(four, code_exponent, codes, carried);
    code_out = codes & 0xFFu;
    operand_out = quantize_operand_pair(carried[0], 0u, code_exponent) & 0xFFFFu;
}

/* where the values of a vector go: value `index` = 64 load + 16 step + u lies in word ((4 load + t) 4 + step) with
 * t = (u % 8) / 2: its code at byte 2 (u % 2) + u / 8 of the word, its operand at halfword 2 (u / 8) + u % 2 of the
 * word's four */
__device__ static __forceinline__ uint32_t quantize_word_of(uint32_t load, uint32_t step, uint32_t t)
{
    return ((4u * load + t) * 4u + step) * 4u;
}

/* bits: the bfloat16 value at `index` of a vector of `width` values; codes, exponents, operands: the vector's arrays */
__device__ static __forceinline__ void quantize_value(uint32_t bits, uint32_t index, unsigned char *codes, unsigned char *exponents,
                                                      uint16_t *operands)
{
    float largest = fabsf(bf16_to_float((uint16_t)bits));
#pragma unroll
    for (uint32_t distance = 16u; distance != 0u; distance >>= 1u) {
        largest = fmaxf(largest, __shfl_xor(largest, (int)distance, 32));
    }
    const uint32_t code_exponent = quantize_exponent_code(largest);
    uint32_t code, operand;
    quantize_code(bits, code_exponent, code, operand);
    const uint32_t u = index % 16u, word = quantize_word_of(index / 64u, (index % 64u) / 16u, (u % 8u) / 2u);
    codes[word + 2u * (u % 2u) + u / 8u] = (unsigned char)code;
    operands[word + 2u * (u / 8u) + u % 2u] = (uint16_t)operand;
    if (index % 32u == 0u) {
        exponents[index / 32u] = (unsigned char)code_exponent;
    }
}

/* thread q of a vector's width / 4 (four values, a word of codes) of vector `vector`: activation_quantize_entry's work of
 * one thread; the eight threads of a block of 32 values are neighbours in one wavefront and call together */
__device__ static __forceinline__ void activation_quantize_body(const struct activation_quantize_arguments &arguments, unsigned char *arena,
                                                                uint32_t q, uint64_t vector)
{
    /* thread q = (16 l + 4 s + t) takes the four values 64 l + 16 s + 2 t + {0, 1, 8, 9}: the four codes of one word of
     * the lane order and the four operands of one pair of words; the 32 values of a block of the quantization are those
     * of eight neighbouring threads (s = 2 b, 2 b + 1; t = 0 .. 3) */
    const uint32_t l = q / 16u, s = (q / 4u) % 4u, t = q % 4u, first = 64u * l + 16u * s + 2u * t;
    if (first >= arguments.width) {
        return; /* the width is a multiple of 64: whole groups of sixteen threads leave together */
    }
    const uint16_t *values = (const uint16_t *)(arena + arguments.values_offset) + vector * arguments.width + first;
    const uint32_t near_pair = *(const uint32_t *)values, far_pair = *(const uint32_t *)(values + 8);
    const uint32_t bits[4] = {near_pair & 0xFFFFu, near_pair >> 16, far_pair & 0xFFFFu, far_pair >> 16}; /* values +0, +1, +8, +9 */
    float largest = fmaxf(fmaxf(fabsf(bf16_to_float((uint16_t)bits[0])), fabsf(bf16_to_float((uint16_t)bits[1]))),
                          fmaxf(fabsf(bf16_to_float((uint16_t)bits[2])), fabsf(bf16_to_float((uint16_t)bits[3]))));
#pragma unroll
    for (uint32_t distance = 4u; distance != 0u; distance >>= 1u) {
        largest = fmaxf(largest, __shfl_xor(largest, (int)distance, 8));
    }
    const uint32_t code_exponent = quantize_exponent_code(largest);
    /* the word's bytes j = 0 .. 3 hold values +0 (j = 0), +8 (1), +1 (2), +9 (3); its operands' halfwords 2 r + h hold
     * value + h + 8 r */
    const uint32_t in_word_order[4] = {bits[0], bits[2], bits[1], bits[3]};
    uint32_t codes, carried[4];
    quantize_codes4(in_word_order, code_exponent, codes, carried);
    const uint32_t word = quantize_word_of(l, s, t);
    *(uint32_t *)(arena + arguments.codes_offset + vector * arguments.width + word) = codes;
    *(uint2_t *)((uint16_t *)(arena + arguments.operands_offset) + vector * arguments.width + word) =
        (uint2_t){quantize_operand_pair(carried[0], carried[2], code_exponent), quantize_operand_pair(carried[1], carried[3], code_exponent)};
    if (q % 8u == 0u) {
        (arena + arguments.exponents_offset)[vector * (arguments.width / 32u) + first / 32u] = (unsigned char)code_exponent;
    }
}

#endif
