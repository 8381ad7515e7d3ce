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
#include "kernel_registry.h"
#include "quantize_device.cuh"

extern "C" __global__ void __launch_bounds__(LINEAR_ELEMENT_THREADS)
    activation_quantize_entry(struct activation_quantize_arguments arguments, unsigned char *arena)
{
    const uint32_t index = blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= arguments.width) {
        return; /* the width is a multiple of 64: whole groups of 32 lanes leave together */
    }
    const uint64_t vector = blockIdx.y;
    const uint32_t bits = ((const uint16_t *)(arena + arguments.values_offset))[vector * arguments.width + index];
    quantize_value(bits, index, arena + arguments.codes_offset + vector * arguments.width,
                   arena + arguments.exponents_offset + vector * (arguments.width / 32u),
                   (uint16_t *)(arena + arguments.operands_offset) + vector * arguments.width);
}
ANEMONE_KERNEL(KERNEL_FILE_ACTIVATION_QUANTIZE, activation_quantize_entry, activation_quantize_arguments);

/* The quantizer of WEIGHT_FORMAT_E4M3_BLOCK128's vectors (no counterpart in the reference): for each 128 consecutive
 * bfloat16 values, all in float32, scale = max(largest magnitude, 1e-4) / 448; each value is divided by the scale
 * (one rounding), limited to 448 and rounded to the nearest E4M3 number, a tie to the even code, the sign kept.
 * Written: codes [v][width] in the same lane order; the scales, float32 [v][width / 128], where the record names the
 * exponents (the same bytes a vector: width / 32); the operands are not written.
 * Launch: grid (ceil(width / 512), vectors), block 256: a wavefront 128 values, a lane two neighbours. */
extern "C" __global__ void __launch_bounds__(LINEAR_ELEMENT_THREADS)
    activation_quantize_128_entry(struct activation_quantize_arguments arguments, unsigned char *arena)
{
    const uint32_t index = 2u * (blockIdx.x * blockDim.x + threadIdx.x);
    if (index >= arguments.width) {
        return; /* the width is a multiple of 128: whole wavefronts leave together */
    }
    const uint64_t vector = blockIdx.y;
    const uint32_t two = *(const uint32_t *)((const uint16_t *)(arena + arguments.values_offset) + vector * arguments.width + index);
    const uint32_t bits[2] = {two & 0xFFFFu, two >> 16};
    float largest = fmaxf(fabsf(bf16_to_float((uint16_t)bits[0])), fabsf(bf16_to_float((uint16_t)bits[1])));
#pragma unroll
    for (uint32_t distance = 32u; distance != 0u; distance >>= 1u) {
        largest = fmaxf(largest, __shfl_xor(largest, (int)distance, WAVE));
    }
    const float scale = __fdiv_rn(fmaxf(largest, 1e-4f), 448.0f);
    unsigned char *codes = arena + arguments.codes_offset + vector * arguments.width;
#pragma unroll
    for (uint32_t i = 0; i < 2u; i++) {
        const float scaled = __fdiv_rn(bf16_to_float((uint16_t)bits[i]), scale);
        const float magnitude = fminf(fabsf(scaled), 448.0f);
        const uint32_t field = __float_as_uint(fmaxf(magnitude, 0.015625f)) >> 23;
        const uint32_t units = (uint32_t)__builtin_rintf(__fmul_rn(magnitude, __uint_as_float((257u - field) << 23)));
        const uint32_t code = (((field - 120u) << 3) + units - 8u) | ((bits[i] >> 8) & 0x80u);
        const uint32_t at = index + i, u = at % 16u;
        codes[quantize_word_of(at / 64u, (at % 64u) / 16u, (u % 8u) / 2u) + 2u * (u % 2u) + u / 8u] = (unsigned char)code;
    }
    if (index % 128u == 0u) {
        ((float *)(arena + arguments.exponents_offset))[vector * (arguments.width / 128u) + index / 128u] = scale;
    }
}
ANEMONE_KERNEL(KERNEL_FILE_ACTIVATION_QUANTIZE, activation_quantize_128_entry, activation_quantize_arguments);
