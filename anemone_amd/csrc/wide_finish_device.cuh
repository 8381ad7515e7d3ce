/*
 * wide_finish_device.cuh -- what a block of the wide routed experts does with its sums, shared by the kernels of the
 * reference's weight formats (kernel_wide_linear.hip) and of gfx950's own (kernel_native_linear.hip): the gate/up
 * launch's hidden step and quantizer from the registers the sums are in, the down launch's stores. A block's columns are
 * `pair_count` sorted pairs from `pairs` on (COLUMN_BLOCKS blocks of 16 at most); chain[t][j]: tile t of the wavefront's
 * strip (gate's STRIP tiles, then up's) by column block j, a lane holding rows 4 (lane / 16) .. + 3 of column lane % 16.
 */
#ifndef WIDE_FINISH_DEVICE_CUH
#define WIDE_FINISH_DEVICE_CUH

#include "linear_device.cuh"
#include "quantize_device.cuh"

#ifndef WIDE_WAVES
#define WIDE_WAVES 4u
#endif

/* window: the block's LDS window, free once the K steps are done (one tile a strip: the two wavefronts of a quantizer
 * block pass each other their halves' largest magnitude through it; every wavefront of the block calls together) */
template <uint32_t STRIP, uint32_t COLUMN_BLOCKS, bool B128>
__device__ static __forceinline__ void wide_gate_up_finish(const struct wide_expert_gate_up_arguments &arguments, unsigned char *arena,
                                                           unsigned char *window, const struct wide_pair *pairs, uint32_t pair_count,
                                                           uint32_t block_strip, uint32_t tile0, uint32_t wave, uint32_t lane,
                                                           float4_t (&chain)[2u * STRIP][COLUMN_BLOCKS])
{
    constexpr uint32_t STRIP_OUTPUTS = STRIP * 16u;
    /* The hidden step, as expert_gate_up_1 rounds it (the one chain is added to +0 first, as S chains are), and the
     * quantizer's step on it, from the registers the sums are in. A lane holds, of a column of every column block, rows
     * 4 (lane / 16) .. + 3 of the strip's tiles. Two tiles a strip: the 32 outputs of one quantizer block are the 8
     * values of each of the 4 lanes of a column. One tile a strip: the block is the strips of the wavefronts 2 p and
     * 2 p + 1 (the matrix holds whole blocks of 32 outputs: both are inside it or neither), which pass each other the
     * largest magnitude of their halves through LDS. Codes are bytes 2 (v % 2) + g / 2 of a word, so the lanes g and
     * g ^ 2 of a column hold the halves of the same two words: one exchange, and each writes one whole word. */
    const uint32_t width = arguments.output_size, first_output = (block_strip * WIDE_WAVES + wave) * STRIP_OUTPUTS;
    const bool strip_is_live = first_output < width; /* else: a strip wholly past the matrix (its tiles were the strip's before it) */
    const float limit = arguments.activation_limit;
    const uint32_t g = lane / 16u, upper = g / 2u;
    /* column block j: the hidden values of the lane's rows of its column, and the largest magnitude of the column's 16
     * STRIP values of this strip (the same in the column's four lanes) */
    const auto hidden_of = [&](uint32_t j, uint32_t (&bits)[STRIP][4]) -> float {
        const uint32_t column = 16u * j + lane % 16u;
        float largest = 0.0f;
        if (column < pair_count && strip_is_live) { /* the same in the four lanes of a column */
            const float weight = pairs[column].route_weight;
#pragma unroll
            for (uint32_t n = 0; n < STRIP; n++) {
#pragma unroll
                for (uint32_t v = 0; v < 4u; v++) {
                    const float gate_sum = __fadd_rn(0.0f, chain[n][j][v]), up_sum = __fadd_rn(0.0f, chain[STRIP + n][j][v]);
                    const float gate = bf16_to_float(float_to_bf16(gate_sum)), up = bf16_to_float(float_to_bf16(up_sum));
                    const float bounded_gate = fminf(gate, limit);
                    const float bounded_up = fminf(fmaxf(up, -limit), limit);
                    const float value = __fmul_rn(__fmul_rn(linear_silu(bounded_gate), bounded_up), weight);
                    bits[n][v] = float_to_bf16(value);
                    largest = fmaxf(largest, fabsf(bf16_to_float((uint16_t)bits[n][v])));
                }
            }
            if constexpr (B128) {
                /* the hidden values themselves, where the record names the hidden operands (bfloat16 [pair][width]
                 * either way): this format's quantizer takes 128 values a scale, in a launch of its own */
                uint16_t *values = (uint16_t *)(arena + arguments.hidden_operands_offset) + (uint64_t)pairs[column].pair_index * width;
#pragma unroll
                for (uint32_t n = 0; n < STRIP; n++) {
                    *(uint2_t *)(values + (tile0 + n) * 16u + 4u * g) = (uint2_t){bits[n][0] | (bits[n][1] << 16), bits[n][2] | (bits[n][3] << 16)};
                }
            }
            largest = fmaxf(largest, __shfl_xor(largest, 16, WAVE));
            largest = fmaxf(largest, __shfl_xor(largest, 32, WAVE));
        }
        return largest;
    };
    /* column block j: the quantizer's step on those values under the block's largest magnitude, and its stores */
    const auto store_of = [&](uint32_t j, const uint32_t (&bits)[STRIP][4], float largest) {
        const uint32_t column = 16u * j + lane % 16u;
        if (column < pair_count) {
            const uint64_t pair = pairs[column].pair_index;
            const uint32_t code_exponent = quantize_exponent_code(largest);
            unsigned char *codes = arena + arguments.hidden_codes_offset + pair * width;
            uint16_t *operands = (uint16_t *)(arena + arguments.hidden_operands_offset) + pair * width;
#pragma unroll
            for (uint32_t n = 0; n < STRIP; n++) {
                uint32_t own, carried[4];
                quantize_codes4(bits[n], code_exponent, own, carried);
                const uint32_t load = (tile0 + n) / 4u, step = (tile0 + n) % 4u, t = 2u * (g % 2u);
                const uint32_t word0 = quantize_word_of(load, step, t), word1 = quantize_word_of(load, step, t + 1u);
                /* word0 is (a0, b0, a1, b1) and word1 (a2, b2, a3, b3) of the codes a of the lower lane and b of the
                 * upper: each takes the other's four and stores one of the words */
                const uint32_t other = (uint32_t)__shfl_xor((int)own, 32, WAVE);
                *(uint32_t *)(codes + (upper != 0u ? word1 : word0)) = __builtin_amdgcn_perm(other, own, upper != 0u ? 0x03070206u : 0x05010400u);
                *(uint32_t *)(operands + word0 + 2u * upper) = quantize_operand_pair(carried[0], carried[1], code_exponent);
                *(uint32_t *)(operands + word1 + 2u * upper) = quantize_operand_pair(carried[2], carried[3], code_exponent);
            }
            if (g == 0u && first_output % 32u == 0u) {
                (arena + arguments.hidden_exponents_offset)[pair * (width / 32u) + first_output / 32u] = (unsigned char)code_exponent;
            }
        }
    };
    if constexpr (STRIP == 2u && !B128) {
        /* a quantizer block is this wavefront's own: a column block at a time, its values in eight registers */
#pragma unroll
        for (uint32_t j = 0; j < COLUMN_BLOCKS; j++) {
            uint32_t bits[STRIP][4];
            const float largest = hidden_of(j, bits);
            if (strip_is_live) {
                store_of(j, bits, largest);
            }
        }
        return;
    }
    uint32_t bits[COLUMN_BLOCKS][STRIP][4];
    float largest[COLUMN_BLOCKS];
#pragma unroll
    for (uint32_t j = 0; j < COLUMN_BLOCKS; j++) {
        largest[j] = hidden_of(j, bits[j]);
    }
    if constexpr (B128) {
        return;
    }
    if constexpr (STRIP == 1u) {
        float *halves = (float *)window; /* [wavefront][column]: the stages are done with */
        __syncthreads();
#pragma unroll
        for (uint32_t j = 0; j < COLUMN_BLOCKS; j++) {
            if (g == 0u) {
                halves[wave * (COLUMN_BLOCKS * 16u) + 16u * j + lane] = largest[j];
            }
        }
        __syncthreads();
#pragma unroll
        for (uint32_t j = 0; j < COLUMN_BLOCKS; j++) {
            largest[j] = fmaxf(largest[j], halves[(wave ^ 1u) * (COLUMN_BLOCKS * 16u) + 16u * j + lane % 16u]);
        }
    }
    if (!strip_is_live) {
        return;
    }
#pragma unroll
    for (uint32_t j = 0; j < COLUMN_BLOCKS; j++) {
        store_of(j, bits[j], largest[j]);
    }
}

template <uint32_t STRIP, uint32_t COLUMN_BLOCKS>
__device__ static __forceinline__ void wide_down_finish(const struct wide_expert_down_arguments &arguments, unsigned char *arena,
                                                        const struct wide_pair *pairs, uint32_t pair_count, uint32_t block_strip,
                                                        uint32_t tile0, uint32_t wave, uint32_t lane, float4_t (&chain)[STRIP][COLUMN_BLOCKS])
{
    constexpr uint32_t STRIP_OUTPUTS = STRIP * 16u;
    const uint32_t first_output = (block_strip * WIDE_WAVES + wave) * STRIP_OUTPUTS;
    if (first_output >= arguments.output_size) {
        return;
    }
#pragma unroll
    for (uint32_t j = 0; j < COLUMN_BLOCKS; j++) {
        const uint32_t column = 16u * j + lane % 16u;
        if (column < pair_count) {
            const uint64_t pair = pairs[column].pair_index;
#pragma unroll
            for (uint32_t n = 0; n < STRIP; n++) {
                if ((tile0 + n) * 16u < first_output) {
                    continue; /* a tile the strip before this one stores */
                }
                uint16_t *out = (uint16_t *)(arena + arguments.output_offset) + pair * arguments.output_size + (tile0 + n) * 16u + 4u * (lane / 16u);
                const float s0 = __fadd_rn(0.0f, chain[n][j][0]), s1 = __fadd_rn(0.0f, chain[n][j][1]);
                const float s2 = __fadd_rn(0.0f, chain[n][j][2]), s3 = __fadd_rn(0.0f, chain[n][j][3]);
                *(uint2_t *)out = (uint2_t){(uint32_t)float_to_bf16(s0) | ((uint32_t)float_to_bf16(s1) << 16),
                                            (uint32_t)float_to_bf16(s2) | ((uint32_t)float_to_bf16(s3) << 16)};
            }
        }
    }
}

#endif
