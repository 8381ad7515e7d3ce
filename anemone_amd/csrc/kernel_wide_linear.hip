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
#include "wide_finish_device.cuh"

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
    wide_gate_up_finish<STRIP, WIDE_COLUMN_BLOCKS, B128>(arguments, arena, window, pairs, tile.pair_count, blockIdx.x, tile0, wave, lane, chain);
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
    wide_down_finish<STRIP, WIDE_COLUMN_BLOCKS>(arguments, arena, pairs, tile.pair_count, blockIdx.x, tile0, wave, lane, chain);
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
