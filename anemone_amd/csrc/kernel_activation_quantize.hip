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
 * Launch: grid (ceil(width / 1024), vectors), block 256; a thread four values (a word of codes), eight threads a block
 * of 32 values.
 */
#include "kernel_registry.h"
#include "quantize_device.cuh"

extern "C" __global__ void __launch_bounds__(LINEAR_ELEMENT_THREADS)
    activation_quantize_entry(struct activation_quantize_arguments arguments, unsigned char *arena)
{
    activation_quantize_body(arguments, arena, blockIdx.x * blockDim.x + threadIdx.x, blockIdx.y);
}
ANEMONE_KERNEL(KERNEL_FILE_ACTIVATION_QUANTIZE, activation_quantize_entry, activation_quantize_arguments);

/* The quantizer of WEIGHT_FORMAT_E4M3_BLOCK128's vectors (no counterpart in the reference): for each 128 consecutive
 * bfloat16 values, all in float32, scale = max(largest magnitude, 1e-4) / 448; each value is divided by the scale
 * (one rounding), limited to 448 and rounded to the nearest E4M3 number, a tie to the even code, the sign kept.
 * Written: codes [v][width] in the same lane order; the scales, float32 [v][width / 128], where the record names the
 * exponents (the same bytes a vector: width / 32); the operands are not written.
 * Launch: grid (ceil(width / 1024), vectors), block 256: a thread four values (a word of codes), 32 threads a scale. */
extern "C" __global__ void __launch_bounds__(LINEAR_ELEMENT_THREADS)
    activation_quantize_128_entry(struct activation_quantize_arguments arguments, unsigned char *arena)
{
    /* the threads' values as in activation_quantize_entry: thread q = 16 l + 4 s + t takes 64 l + 16 s + 2 t + {0, 1, 8, 9},
     * one word of codes; the 128 values of a scale are those of 32 neighbouring threads */
    const uint32_t q = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t l = q / 16u, s = (q / 4u) % 4u, t = q % 4u, first = 64u * l + 16u * s + 2u * t;
    if (first >= arguments.width) {
        return; /* the width is a multiple of 128: whole groups of 32 threads leave together */
    }
    const uint64_t vector = blockIdx.y;
    const uint16_t *values = (const uint16_t *)(arena + arguments.values_offset) + vector * arguments.width + first;
    const uint32_t near_pair = *(const uint32_t *)values, far_pair = *(const uint32_t *)(values + 8);
    const uint32_t bits[4] = {near_pair & 0xFFFFu, near_pair >> 16, far_pair & 0xFFFFu, far_pair >> 16};
    float largest = fmaxf(fmaxf(fabsf(bf16_to_float((uint16_t)bits[0])), fabsf(bf16_to_float((uint16_t)bits[1]))),
                          fmaxf(fabsf(bf16_to_float((uint16_t)bits[2])), fabsf(bf16_to_float((uint16_t)bits[3]))));
#pragma unroll
    for (uint32_t distance = 16u; distance != 0u; distance >>= 1u) {
        largest = fmaxf(largest, __shfl_xor(largest, (int)distance, 32));
    }
    const float scale = __fdiv_rn(fmaxf(largest, 1e-4f), 448.0f);
    uint32_t code[4];
#pragma unroll
    for (uint32_t i = 0; i < 4u; i++) {
        const float scaled = __fdiv_rn(bf16_to_float((uint16_t)bits[i]), scale);
        const float magnitude = fminf(fabsf(scaled), 448.0f);
        const uint32_t field = __float_as_uint(fmaxf(magnitude, 0.015625f)) >> 23;
        const uint32_t units = (uint32_t)__builtin_rintf(__fmul_rn(magnitude, __uint_as_float((257u - field) << 23)));
        code[i] = (((field - 120u) << 3) + units - 8u) | ((bits[i] >> 8) & 0x80u);
    }
    *(uint32_t *)(arena + arguments.codes_offset + vector * arguments.width + quantize_word_of(l, s, t)) =
        code[0] | (code[2] << 8) | (code[1] << 16) | (code[3] << 24); /* bytes: values +0, +8, +1, +9 */
    if (q % 32u == 0u) {
        ((float *)(arena + arguments.exponents_offset))[vector * (arguments.width / 128u) + first / 128u] = scale;
    }
}
ANEMONE_KERNEL(KERNEL_FILE_ACTIVATION_QUANTIZE, activation_quantize_128_entry, activation_quantize_arguments);
