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

/* one bfloat16 value under its block's scale code: its E4M3 code (to nearest even, clamped at 448) and its operand */
__device__ static __forceinline__ void quantize_code(uint32_t bits, uint32_t code_exponent, uint32_t &code_out, uint32_t &operand_out)
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

#endif
