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
