/*
 * kernel_activation_quantize.hip -- the per-32 activation quantizer of the FP4 / FP8 linears on gfx950.
 * Entry name, record and every written byte follow the reference (source/kernel_activation_quantize.cuh:52-133,
 * include/anemone/linear_records.h:20-44): for each block of 32 consecutive bfloat16 values, all in float32,
 *   m = max(largest magnitude, 1e-4) x float32(1 / 448); the exponent code c is the exponent of m, one more unless
 *   m is a power of two; each value is divided by 2^(c - 127) (exact), limited to 448 and rounded to the nearest E4M3
 *   number, a tie to the even code, the sign kept also on a zero.
 * Written: codes [v][width] in LANE ORDER (byte ((4 l + t) 4 + s) 4 + j holds value 64 l + 16 s + 2 t + j / 2 +
 * 8 (j % 2)), exponents [v][width / 32], operands [v][width] (bfloat16 of the value's code x scale x 2^100, in
 * OPERAND ORDER; an infinity of the sign where c is above 146). The operands are not read by this library's own
 * kernels; they are written because the record's contract writes them on every card.
 * Launch: grid (ceil(width / 256), vectors), block 256; a thread a value, 32 lanes a block of values.
 */
#include "exl3_device.cuh"
#include "kernel_registry.h"

extern "C" __global__ void __launch_bounds__(LINEAR_ELEMENT_THREADS)
    activation_quantize_entry(struct activation_quantize_arguments arguments, unsigned char *arena)
{
    const uint32_t index = blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= arguments.width) {
        return; /* the width is a multiple of 64: whole groups of 32 lanes leave together */
    }
    const uint64_t vector = blockIdx.y;
    const uint32_t bits = ((const uint16_t *)(arena + arguments.values_offset))[vector * arguments.width + index];
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
    unsigned char *codes = arena + arguments.codes_offset + vector * arguments.width;
    uint16_t *operands = (uint16_t *)(arena + arguments.operands_offset) + vector * arguments.width;
    codes[word + 2u * (u % 2u) + u / 8u] = (unsigned char)code;
    operands[word + 2u * (u / 8u) + u % 2u] = (uint16_t)operand;
    if (index % 32u == 0u) {
        (arena + arguments.exponents_offset)[vector * (arguments.width / 32u) + index / 32u] = (unsigned char)code_exponent;
    }
}
ANEMONE_KERNEL(KERNEL_FILE_ACTIVATION_QUANTIZE, activation_quantize_entry, activation_quantize_arguments);
