/*
 * kernel_wide_linear.hip -- the routed experts of the original FP4 / FP8 weights for a prefill-sized step on gfx950:
 * a grouped GEMM over the tiles of at most 64 pairs of one expert that the router's wide select writes. Entry names,
 * records and what is written follow the reference (include/anemone/wide_linear_records.h:80-118,
 * source/kernel_wide_linear.cu): wide_expert_gate_up_<S> writes, for each pair of a tile, what the quantizer writes
 * from the hidden values expert_gate_up_<S> computes (codes, exponents, operands, not the values);
 * wide_expert_down_<S> writes a pair's output at its pair_index. An output's bits depend on its matrix, its pair's
 * input and S alone (the reference's class R): here they are expert_gate_up_<S>'s and expert_down_<S>'s of
 * kernel_expert_linear.hip bit for bit, because a column's sum is the same chain of the same MFMAs in the same order.
 * Built for S = 1 (one chain an output).
 *
 * Work mapping (this build's own). A block is one tile of pairs (64 columns: four MFMA column blocks of 16) by 256
 * outputs: four wavefronts, each a strip of tiles of 16 outputs (64 outputs of 4-bit weights, 32 of one-byte
 * weights; gate AND up of the strip in the gate/up kernel). A stage is one K step (128 inputs): each wavefront's
 * weights and their scales go from memory straight into its part of the stage in LDS; the 64 columns' codes (8 KB)
 * and scale words go there once a block, two column groups a wavefront, and serve all four. Three stages are on
 * their way or in use; one barrier a step. A weight tile's operand is prepared once (four 8-byte LDS reads and
 * sixteen vector instructions for 4-bit weights) and feeds four MFMAs of 128 inputs each.
 */
#include "kernel_registry.h"
#include "linear_device.cuh"
#include "quantize_device.cuh"

#include "wide_device.cuh"

/* grid (ceil(output_size / (4 strips)), tile_count), block 256; a strip is STRIP tiles of gate and STRIP of up */
template <bool BYTES, uint32_t STRIP, uint32_t DEPTH, bool B128 = false>
__device__ static __forceinline__ void wide_expert_gate_up(const struct wide_expert_gate_up_arguments &arguments, unsigned char *arena)
{
    typedef wide_chain<2, BYTES, STRIP, DEPTH, B128> chain_type;
    constexpr uint32_t TILES = chain_type::TILES, STRIP_OUTPUTS = STRIP * 16u;
    static_assert(STRIP == 1u || STRIP == 2u, "a quantizer block of 32 outputs is one strip or two");
    extern __shared__ __attribute__((aligned(16))) unsigned char window[];
    const struct wide_expert_tile tile = ((const struct wide_expert_tile *)(arena + arguments.tiles_offset))[blockIdx.y];
    if (tile.pair_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const struct wide_pair *pairs = (const struct wide_pair *)(arena + arguments.pairs_offset) + tile.first_pair;
    /* columns past the tile's last pair read its first pair's vector; their sums are never stored */
    uint32_t code_vectors[2];
#pragma unroll
    for (uint32_t part = 0; part < 2u; part++) {
        const uint32_t column = 8u * (2u * wave + part) + lane / 8u;
        code_vectors[part] = pairs[column < tile.pair_count ? column : 0u].pair_index / arguments.pairs_per_row;
    }
    const uint32_t scale_column = 16u * wave + lane % 16u;
    const uint32_t exponent_vector = pairs[scale_column < tile.pair_count ? scale_column : 0u].pair_index / arguments.pairs_per_row;
    chain_type chain_of;
    const unsigned char *const matrices[2] = {arena + tile.gate_offset, arena + tile.up_offset};
    const uint32_t window_address = (uint32_t)(uintptr_t)(lds_pointer)window;
    uint32_t tile0 = 0;
    chain_of.place(matrices, arguments.output_size, arguments.input_size, blockIdx.x, arena + arguments.codes_offset,
                   arena + arguments.exponents_offset, code_vectors, exponent_vector, window_address, wave, lane, tile0);
    float4_t chain[TILES][WIDE_COLUMN_BLOCKS];
#pragma unroll
    for (uint32_t t = 0; t < TILES; t++) {
#pragma unroll
        for (uint32_t j = 0; j < WIDE_COLUMN_BLOCKS; j++) {
            chain[t][j] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
    const uint32_t live_blocks = (tile.pair_count + 15u) / 16u;
    chain_of.whole(arguments.input_size / 128u, live_blocks, chain);
    /* The hidden step, as expert_gate_up_1 rounds it (the one chain is added to +0 first, as S chains are), and the
     * quantizer's step on it, from the registers the sums are in. A lane holds, of a column of every column block, rows
     * 4 (lane / 16) .. + 3 of the strip's tiles. Two tiles a strip: the 32 outputs of one quantizer block are the 8
     * values of each of the 4 lanes of a column. One tile a strip: the block is the strips of the wavefronts 2 p and
     * 2 p + 1 (the matrix holds whole blocks of 32 outputs: both are inside it or neither), which pass each other the
     * largest magnitude of their halves through LDS. Codes are bytes 2 (v % 2) + g / 2 of a word, so the lanes g and
     * g ^ 2 of a column hold the halves of the same two words: one exchange, and each writes one whole word. */
    const uint32_t width = arguments.output_size, first_output = (blockIdx.x * WIDE_WAVES + wave) * STRIP_OUTPUTS;
    const bool strip_is_live = first_output < width; /* else: a strip wholly past the matrix (its tiles were the strip's before it) */
    const float limit = arguments.activation_limit;
    const uint32_t g = lane / 16u, upper = g / 2u;
    uint32_t bits[WIDE_COLUMN_BLOCKS][STRIP][4];
    float largest[WIDE_COLUMN_BLOCKS];
#pragma unroll
    for (uint32_t j = 0; j < WIDE_COLUMN_BLOCKS; j++) {
        const uint32_t column = 16u * j + lane % 16u;
        largest[j] = 0.0f;
        if (column < tile.pair_count && strip_is_live) { /* the same in the four lanes of a column */
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
                    bits[j][n][v] = float_to_bf16(value);
                    largest[j] = fmaxf(largest[j], fabsf(bf16_to_float((uint16_t)bits[j][n][v])));
                }
            }
            if constexpr (B128) {
                /* the hidden values themselves, where the record names the hidden operands (bfloat16 [pair][width]
                 * either way): this format's quantizer takes 128 values a scale, in a launch of its own */
                uint16_t *values = (uint16_t *)(arena + arguments.hidden_operands_offset) + (uint64_t)pairs[column].pair_index * width;
#pragma unroll
                for (uint32_t n = 0; n < STRIP; n++) {
                    *(uint2_t *)(values + (tile0 + n) * 16u + 4u * g) = (uint2_t){bits[j][n][0] | (bits[j][n][1] << 16), bits[j][n][2] | (bits[j][n][3] << 16)};
                }
            }
            largest[j] = fmaxf(largest[j], __shfl_xor(largest[j], 16, WAVE));
            largest[j] = fmaxf(largest[j], __shfl_xor(largest[j], 32, WAVE));
        }
    }
    if constexpr (B128) {
        return;
    }
    if constexpr (STRIP == 1u) {
        float *halves = (float *)window; /* [wavefront][column]: the stages are done with */
        __syncthreads();
#pragma unroll
        for (uint32_t j = 0; j < WIDE_COLUMN_BLOCKS; j++) {
            if (g == 0u) {
                halves[wave * WIDE_TILE_PAIRS + 16u * j + lane] = largest[j];
            }
        }
        __syncthreads();
#pragma unroll
        for (uint32_t j = 0; j < WIDE_COLUMN_BLOCKS; j++) {
            largest[j] = fmaxf(largest[j], halves[(wave ^ 1u) * WIDE_TILE_PAIRS + 16u * j + lane % 16u]);
        }
    }
    if (!strip_is_live) {
        return;
    }
#pragma unroll
    for (uint32_t j = 0; j < WIDE_COLUMN_BLOCKS; j++) {
        const uint32_t column = 16u * j + lane % 16u;
        if (column < tile.pair_count) {
            const uint64_t pair = pairs[column].pair_index;
            const uint32_t code_exponent = quantize_exponent_code(largest[j]);
            unsigned char *codes = arena + arguments.hidden_codes_offset + pair * width;
            uint16_t *operands = (uint16_t *)(arena + arguments.hidden_operands_offset) + pair * width;
#pragma unroll
            for (uint32_t n = 0; n < STRIP; n++) {
                uint32_t own, carried[4];
                quantize_codes4(bits[j][n], code_exponent, own, carried);
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
    }
}

template <bool BYTES, bool B128 = false>
__device__ static __forceinline__ void wide_expert_down(const struct wide_expert_down_arguments &arguments, unsigned char *arena)
{
    typedef wide_chain<1, BYTES, (BYTES ? 2u : 4u), 2u, B128> chain_type;
    constexpr uint32_t TILES = chain_type::TILES, STRIP = chain_type::STRIP, STRIP_OUTPUTS = STRIP * 16u;
    extern __shared__ __attribute__((aligned(16))) unsigned char window[];
    const struct wide_expert_tile tile = ((const struct wide_expert_tile *)(arena + arguments.tiles_offset))[blockIdx.y];
    if (tile.pair_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const struct wide_pair *pairs = (const struct wide_pair *)(arena + arguments.pairs_offset) + tile.first_pair;
    uint32_t code_vectors[2]; /* the vectors are the pairs' hidden vectors */
#pragma unroll
    for (uint32_t part = 0; part < 2u; part++) {
        const uint32_t column = 8u * (2u * wave + part) + lane / 8u;
        code_vectors[part] = pairs[column < tile.pair_count ? column : 0u].pair_index;
    }
    const uint32_t scale_column = 16u * wave + lane % 16u;
    const uint32_t exponent_vector = pairs[scale_column < tile.pair_count ? scale_column : 0u].pair_index;
    chain_type chain_of;
    const unsigned char *const matrices[1] = {arena + tile.down_offset};
    uint32_t tile0 = 0;
    chain_of.place(matrices, arguments.output_size, arguments.input_size, blockIdx.x, arena + arguments.codes_offset,
                   arena + arguments.exponents_offset, code_vectors, exponent_vector, (uint32_t)(uintptr_t)(lds_pointer)window, wave, lane, tile0);
    float4_t chain[TILES][WIDE_COLUMN_BLOCKS];
#pragma unroll
    for (uint32_t t = 0; t < TILES; t++) {
#pragma unroll
        for (uint32_t j = 0; j < WIDE_COLUMN_BLOCKS; j++) {
            chain[t][j] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
    chain_of.whole(arguments.input_size / 128u, (tile.pair_count + 15u) / 16u, chain);
    const uint32_t first_output = (blockIdx.x * WIDE_WAVES + wave) * STRIP_OUTPUTS;
    if (first_output >= arguments.output_size) {
        return;
    }
#pragma unroll
    for (uint32_t j = 0; j < WIDE_COLUMN_BLOCKS; j++) {
        const uint32_t column = 16u * j + lane % 16u;
        if (column < tile.pair_count) {
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

/* wide_expert_gate_up_1, wide_expert_down_1: the reference's entries, of WEIGHT_FORMAT_E2M1_SCALED experts; the _e4m3_
 * entries take WEIGHT_FORMAT_E4M3_SCALED experts (no counterpart among the reference's expert kernels). The LDS window
 * is dynamic shared memory (more than the 64 KB a kernel may declare): wide_gate_up_window_bytes and
 * wide_down_window_bytes of anemone_records.h. */
extern "C" __global__ void __launch_bounds__(WIDE_THREADS) wide_expert_gate_up_1(struct wide_expert_gate_up_arguments arguments, unsigned char *arena)
{
    wide_expert_gate_up<false, 2u, 2u>(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_WIDE_LINEAR, wide_expert_gate_up_1, wide_expert_gate_up_arguments);
extern "C" __global__ void __launch_bounds__(WIDE_THREADS) wide_expert_down_1(struct wide_expert_down_arguments arguments, unsigned char *arena)
{
    wide_expert_down<false>(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_WIDE_LINEAR, wide_expert_down_1, wide_expert_down_arguments);
extern "C" __global__ void __launch_bounds__(WIDE_THREADS) wide_expert_gate_up_e4m3_1(struct wide_expert_gate_up_arguments arguments, unsigned char *arena)
{
    wide_expert_gate_up<true, 1u, 2u>(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_WIDE_LINEAR, wide_expert_gate_up_e4m3_1, wide_expert_gate_up_arguments);
extern "C" __global__ void __launch_bounds__(WIDE_THREADS) wide_expert_down_e4m3_1(struct wide_expert_down_arguments arguments, unsigned char *arena)
{
    wide_expert_down<true>(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_WIDE_LINEAR, wide_expert_down_e4m3_1, wide_expert_down_arguments);
/* WEIGHT_FORMAT_E4M3_BLOCK128 experts (float32 scales of 128 x 128 blocks; no counterpart in the reference): the
 * gate/up entry writes the hidden VALUES at hidden_operands_offset and no codes */
extern "C" __global__ void __launch_bounds__(WIDE_THREADS) wide_expert_gate_up_b128_1(struct wide_expert_gate_up_arguments arguments, unsigned char *arena)
{
    wide_expert_gate_up<true, 1u, 2u, true>(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_WIDE_LINEAR, wide_expert_gate_up_b128_1, wide_expert_gate_up_arguments);
extern "C" __global__ void __launch_bounds__(WIDE_THREADS) wide_expert_down_b128_1(struct wide_expert_down_arguments arguments, unsigned char *arena)
{
    wide_expert_down<true, true>(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_WIDE_LINEAR, wide_expert_down_b128_1, wide_expert_down_arguments);

static_assert(wide_chain<2, false, 2u, 2u>::WINDOW_BYTES == WIDE_GATE_UP_WINDOW_BYTES && wide_chain<2, true, 1u, 2u>::WINDOW_BYTES == WIDE_GATE_UP_E4M3_WINDOW_BYTES &&
                  wide_chain<1, false, 4u, 2u>::WINDOW_BYTES == WIDE_DOWN_WINDOW_BYTES && wide_chain<1, true, 2u, 2u>::WINDOW_BYTES == WIDE_DOWN_E4M3_WINDOW_BYTES,
              "the windows the host asks for are the kernels'");
