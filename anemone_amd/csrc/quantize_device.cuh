/*
 * quantize_device.cuh -- one value of the per-32 activation quantizer (source/kernel_activation_quantize.cuh:52-133,
 * include/anemone/linear_records.h:20-44 of the reference), shared by the quantizer's own kernel and by the producer
 * (gate with up and the quantization of the hidden vectors in one launch). The 32 values of a block sit in 32
 * consecutive lanes of a wavefront (lane % 32 = index % 32); every lane calls with its value.
 */
#ifndef QUANTIZE_DEVICE_CUH
#define QUANTIZE_DEVICE_CUH

#include "exl3_device.cuh"

/* bits: the bfloat16 value at `index` of a vector of `width` values; codes, exponents, operands: the vector's arrays */
__device__ static __forceinline__ void quantize_value(uint32_t bits, uint32_t index, unsigned char *codes, unsigned char *exponents,
                                                      uint16_t *operands)
{
    const float value = bf16_to_float((uint16_t)bits);
    float largest = fabsf(value);
#pragma unroll
    for (uint32_t distance = 16u; distance != 0u; distance >>= 1u) {
        largest = fmaxf(largest, __shfl_xor(largest, (int)distance, 32));
    }
    const uint32_t ratio = __float_as_uint(__fmul_rn(fmaxf(largest, 1e-4f), 1.0f / 448.0f));
    const uint32_t code_exponent = ((ratio >> 23) & 255u) + ((ratio & 0x7FFFFFu) != 0u ? 1u : 0u);
    const float scaled = __fmul_rn(value, __uint_as_float((254u - code_exponent) << 23)); /* exact: a power of two */
    const float magnitude = fminf(fabsf(scaled), 448.0f);
    const uint32_t field = __float_as_uint(fmaxf(magnitude, 0.015625f)) >> 23; /* at least 2^-6's */
    /* units of 1/8 of the binade (2^-9 below 2^-6): 0 .. 16, to nearest even */
    const uint32_t units = (uint32_t)__builtin_rintf(__fmul_rn(magnitude, __uint_as_float((257u - field) << 23)));
    const uint32_t sign = (bits >> 8) & 0x80u;
    const uint32_t code = (((field - 120u) << 3) + units - 8u) | sign;
    /* the operand: units x 2^(field - 130) x 2^(c - 127) x 2^100, exact, its upper half a bfloat16 */
    const float carried = __fmul_rn((float)units, __uint_as_float((field + code_exponent - 30u) << 23));
    const uint32_t operand = (code_exponent <= 146u ? __float_as_uint(carried) >> 16 : 0x7F80u) | (sign << 8);

    const uint32_t load = index / 64u, step = (index % 64u) / 16u, u = index % 16u, t = (u % 8u) / 2u;
    const uint32_t word = ((4u * load + t) * 4u + step) * 4u;
    codes[word + 2u * (u % 2u) + u / 8u] = (unsigned char)code;
    operands[word + 2u * (u / 8u) + u % 2u] = (uint16_t)operand;
    if (index % 32u == 0u) {
        exponents[index / 32u] = (unsigned char)code_exponent;
    }
}

#endif
