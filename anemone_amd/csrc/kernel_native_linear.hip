/*
 * kernel_native_linear.hip -- the wide routed experts of weights stored in gfx950's own lane order
 * (WEIGHT_FORMAT_E2M1_GFX950, WEIGHT_FORMAT_E4M3_GFX950). The reference's E2M1_SCALED and E4M3_SCALED are by definition
 * the lane order of its cards' matrix instruction (include/anemone/weight_format_seam.h:22-46 there) and its seam says
 * how a backend brings its own: a new format, its kernels, its reference decode among the tests. These are the kernels:
 * what they read, write and sum is what wide_expert_gate_up_1 / wide_expert_down_1 of kernel_wide_linear.hip do for
 * the same matrix in the reference's lay-out, bit for bit (a lane's operand is the same bytes, so every sum is the same
 * chain of the same matrix instructions); only where the bytes lie in memory differs, and with it the work between the
 * load and the matrix instruction: none here.
 *
 * A block takes GROUP consecutive tiles of one expert from the wide select's table (GROUP x 64 columns) by 4 strips of
 * outputs; of an expert's run of tiles the blocks of the tiles at even places do the work of their pair and the others
 * leave at once, so that an expert of up to 128 pairs is read once.
 */
#include "kernel_registry.h"
#include "linear_device.cuh"
#include "quantize_device.cuh"

#include "native_device.cuh"
#include "wide_finish_device.cuh"

/* Which strip of outputs (of the grid's x) and which tile (of its y) a block takes. The card deals blocks to its eight dies
 * in turn by their number x + gx y, so die c holds the blocks whose x % 8 is c, in the order of their rows. Every block of
 * a tile reads the tile's columns, and every block of a strip of an expert's tiles (which follow each other in the table)
 * reads the same weights. The blocks of 32 consecutive rows are re-assigned so that a die holds, of those rows, every
 * strip of four consecutive tiles, the four tiles of a strip next to each other in its order: the tiles' columns come
 * from memory into that die's level-2 cache once, and a strip's weights once for the tiles of an expert among the four
 * (a grid whose x is no multiple of eight, and the rows past the last whole 32, stay as dealt). Measured on one card:
 * E2M1_GFX950 gate/up 1366 -> 1345 us, down 741 -> 727; E4M3_GFX950, whose blocks stream an expert's weights once and
 * pair tiles, 961 -> 1118 and 466 -> 553: BY_DIE is the 4-bit launches' alone. */
#define NATIVE_DIES 8u
#define NATIVE_DIE_TILES 4u
template <bool BY_DIE>
__device__ static __forceinline__ void native_block_of(uint32_t &strip_out, uint32_t &tile_out)
{
    constexpr uint32_t ROWS = NATIVE_DIES * NATIVE_DIE_TILES;
    uint32_t strip = blockIdx.x, tile = blockIdx.y;
    if (BY_DIE && gridDim.x % NATIVE_DIES == 0u && tile < gridDim.y / ROWS * ROWS) {
        const uint32_t place = gridDim.x / NATIVE_DIES * (tile % ROWS) + blockIdx.x / NATIVE_DIES; /* among the die's blocks of these rows */
        strip = place / NATIVE_DIE_TILES;
        tile = tile / ROWS * ROWS + NATIVE_DIE_TILES * (blockIdx.x % NATIVE_DIES) + place % NATIVE_DIE_TILES;
    }
    strip_out = strip;
    tile_out = tile;
}

/* The block's columns: the tile `index` names and, with GROUP 2, the tile behind it where both are the same expert's
 * and this one stands at an even place of the expert's run. Returns false for a block that has nothing to do. `which`
 * picks the offsets the launch reads (gate and up, or down): tiles that agree in them and follow each other in the
 * sorted pairs are one run, whoever's they are. */
template <uint32_t GROUP, bool DOWN>
__device__ static __forceinline__ bool native_columns_of(const struct wide_expert_tile *tiles, uint32_t tile_count, uint32_t index, uint32_t lane,
                                                         struct wide_expert_tile &tile_out, uint32_t &pair_count_out)
{
    const struct wide_expert_tile tile = tiles[index];
    tile_out = tile;
    pair_count_out = tile.pair_count;
    if (tile.pair_count == 0u) {
        return false;
    }
    if constexpr (GROUP == 2u) {
        /* how many tiles of the same run lie before this one: the lanes look at the 64 tiles before it, then further */
        uint32_t before = 0;
        for (uint32_t looked = 0;; looked += WAVE) {
            const uint32_t distance = looked + lane + 1u;
            bool same = false;
            if (distance <= index) {
                const struct wide_expert_tile *other = &tiles[index - distance];
                same = (DOWN ? other->down_offset == tile.down_offset : other->gate_offset == tile.gate_offset && other->up_offset == tile.up_offset) &&
                       other->pair_count == WIDE_TILE_PAIRS && other->first_pair + distance * WIDE_TILE_PAIRS == tile.first_pair;
            }
            const uint64_t mask = __ballot(same);
            const uint32_t run = mask == ~0ull ? WAVE : (uint32_t)__builtin_ctzll(~mask);
            before += run;
            if (run < WAVE) {
                break;
            }
        }
        if (before % 2u != 0u) {
            return false; /* the block of the tile before this one takes both */
        }
        if (tile.pair_count == WIDE_TILE_PAIRS && index + 1u < tile_count) {
            const struct wide_expert_tile next = tiles[index + 1u];
            const bool same = (DOWN ? next.down_offset == tile.down_offset : next.gate_offset == tile.gate_offset && next.up_offset == tile.up_offset) &&
                              next.first_pair == tile.first_pair + WIDE_TILE_PAIRS;
            if (same) {
                pair_count_out += next.pair_count;
            }
        }
    }
    return true;
}

/* the vectors of the columns a wavefront brings: code_vectors[i][part] of column 8 (2 (WAVE_BLOCKS wave + i) + part) +
 * lane / 8, exponent_vector of column 16 WAVE_BLOCKS wave + lane; columns past the last pair read the first pair's */
template <uint32_t WAVE_BLOCKS>
__device__ static __forceinline__ void native_vectors_of(const struct wide_pair *pairs, uint32_t pair_count, uint32_t divisor, uint32_t wave,
                                                         uint32_t lane, uint32_t (&code_vectors)[WAVE_BLOCKS][2], uint32_t &exponent_vector)
{
#pragma unroll
    for (uint32_t i = 0; i < WAVE_BLOCKS; i++) {
#pragma unroll
        for (uint32_t part = 0; part < 2u; part++) {
            const uint32_t column = 8u * (2u * (WAVE_BLOCKS * wave + i) + part) + lane / 8u;
            code_vectors[i][part] = pairs[column < pair_count ? column : 0u].pair_index / divisor;
        }
    }
    const uint32_t scale_column = 16u * WAVE_BLOCKS * wave + lane % (16u * WAVE_BLOCKS);
    exponent_vector = pairs[scale_column < pair_count ? scale_column : 0u].pair_index / divisor;
}

/* grid (ceil(output_size / (4 strips)), tile_count), block 256; a strip is STRIP tiles of gate and STRIP of up */
/* sets of weight registers and stages of columns: 4-bit weights 3 and 2 (156 registers: three wavefronts a SIMD; with a
 * third stage 177, and two wavefronts measured 8 % slower, held to 168 by spills 38 % slower); one-byte weights 3 and 3
 * (150 registers; 4 and 3, at 168, and 6 and 3 measured the same) */
/* float32 block scales: a step's products start from zero and are added times the scales, which takes registers the
 * E8M0 forms leave free. Three sets of weight registers for either product; gate/up two wavefronts a SIMD (901 us a
 * launch of 2048 tokens, against 915 to 940 with four sets, and 1065 with four sets held to 168 registers by spills),
 * down three (459 us, against 484 at two wavefronts and 529 with four sets) */
#define NATIVE_B128_SLOTS 3u
#define NATIVE_B128_GATE_UP_WAVES 2
#define NATIVE_B128_DOWN_WAVES 2
template <bool BYTES, bool B128 = false>
struct native_depths {
    static constexpr uint32_t SLOTS = 3u, DEPTH = BYTES ? NATIVE_E4M3_STAGES : NATIVE_E2M1_STAGES;
};

template <bool BYTES, uint32_t STRIP, uint32_t GROUP, bool B128 = false>
__device__ static __forceinline__ void native_expert_gate_up(const struct wide_expert_gate_up_arguments &arguments, unsigned char *arena)
{
    constexpr uint32_t COLUMN_BLOCKS = 4u * GROUP;
    typedef native_chain<2, BYTES, STRIP, COLUMN_BLOCKS, native_depths<BYTES, B128>::SLOTS, native_depths<BYTES, B128>::DEPTH, B128> chain_type;
    constexpr uint32_t TILES = chain_type::TILES;
    static_assert(STRIP == 1u || STRIP == 2u, "a quantizer block of 32 outputs is one strip or two");
    extern __shared__ __attribute__((aligned(16))) unsigned char window[];
    const uint32_t lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    struct wide_expert_tile tile;
    uint32_t pair_count = 0, block_strip = 0, tile_index = 0;
    native_block_of<!BYTES>(block_strip, tile_index);
    if (!native_columns_of<GROUP, false>((const struct wide_expert_tile *)(arena + arguments.tiles_offset), arguments.tile_count, tile_index, lane, tile, pair_count)) {
        return;
    }
    const struct wide_pair *pairs = (const struct wide_pair *)(arena + arguments.pairs_offset) + tile.first_pair;
    uint32_t code_vectors[chain_type::WAVE_BLOCKS][2], exponent_vector = 0;
    native_vectors_of<chain_type::WAVE_BLOCKS>(pairs, pair_count, arguments.pairs_per_row, wave, lane, code_vectors, exponent_vector);
    chain_type chain_of;
    const unsigned char *const matrices[2] = {arena + tile.gate_offset, arena + tile.up_offset};
    uint32_t tile0 = 0;
    chain_of.place(matrices, arguments.output_size, arguments.input_size, block_strip, arena + arguments.codes_offset,
                   arena + arguments.exponents_offset, code_vectors, exponent_vector, (uint32_t)(uintptr_t)(lds_pointer)window, wave, lane, tile0);
    float4_t chain[TILES][COLUMN_BLOCKS];
#pragma unroll
    for (uint32_t t = 0; t < TILES; t++) {
#pragma unroll
        for (uint32_t j = 0; j < COLUMN_BLOCKS; j++) {
            chain[t][j] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
    chain_of.whole(arguments.input_size / 128u, (pair_count + 15u) / 16u, chain);
    wide_gate_up_finish<STRIP, COLUMN_BLOCKS, B128>(arguments, arena, window, pairs, pair_count, block_strip, tile0, wave, lane, chain);
}

template <bool BYTES, uint32_t GROUP, bool B128 = false>
__device__ static __forceinline__ void native_expert_down(const struct wide_expert_down_arguments &arguments, unsigned char *arena)
{
    constexpr uint32_t COLUMN_BLOCKS = 4u * GROUP;
    typedef native_chain<1, BYTES, (BYTES ? 2u : 4u), COLUMN_BLOCKS, native_depths<BYTES, B128>::SLOTS, native_depths<BYTES, B128>::DEPTH, B128> chain_type;
    constexpr uint32_t TILES = chain_type::TILES, STRIP = chain_type::STRIP;
    extern __shared__ __attribute__((aligned(16))) unsigned char window[];
    const uint32_t lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    struct wide_expert_tile tile;
    uint32_t pair_count = 0, block_strip = 0, tile_index = 0;
    native_block_of<!BYTES>(block_strip, tile_index);
    if (!native_columns_of<GROUP, true>((const struct wide_expert_tile *)(arena + arguments.tiles_offset), arguments.tile_count, tile_index, lane, tile, pair_count)) {
        return;
    }
    const struct wide_pair *pairs = (const struct wide_pair *)(arena + arguments.pairs_offset) + tile.first_pair;
    uint32_t code_vectors[chain_type::WAVE_BLOCKS][2], exponent_vector = 0; /* the vectors are the pairs' hidden vectors */
    native_vectors_of<chain_type::WAVE_BLOCKS>(pairs, pair_count, 1u, wave, lane, code_vectors, exponent_vector);
    chain_type chain_of;
    const unsigned char *const matrices[1] = {arena + tile.down_offset};
    uint32_t tile0 = 0;
    chain_of.place(matrices, arguments.output_size, arguments.input_size, block_strip, arena + arguments.codes_offset,
                   arena + arguments.exponents_offset, code_vectors, exponent_vector, (uint32_t)(uintptr_t)(lds_pointer)window, wave, lane, tile0);
    float4_t chain[TILES][COLUMN_BLOCKS];
#pragma unroll
    for (uint32_t t = 0; t < TILES; t++) {
#pragma unroll
        for (uint32_t j = 0; j < COLUMN_BLOCKS; j++) {
            chain[t][j] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
    chain_of.whole(arguments.input_size / 128u, (pair_count + 15u) / 16u, chain);
    wide_down_finish<STRIP, COLUMN_BLOCKS>(arguments, arena, pairs, pair_count, block_strip, tile0, wave, lane, chain);
}

/* E2M1_GFX950 experts: a block is one tile of pairs by 128 outputs of gate and up (256 of down); E4M3_GFX950 experts: two
 * tiles by 64 (128 of down). The LDS window is dynamic shared memory: NATIVE_WINDOW_BYTES(column blocks, stages). */
#define NATIVE_E2M1_WAVES 3 /* 168 registers */
extern "C" __global__ void __launch_bounds__(NATIVE_THREADS, NATIVE_E2M1_WAVES) native_expert_gate_up_1(struct wide_expert_gate_up_arguments arguments, unsigned char *arena)
{
    native_expert_gate_up<false, 2u, NATIVE_E2M1_COLUMN_BLOCKS / 4u>(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_NATIVE_LINEAR, native_expert_gate_up_1, wide_expert_gate_up_arguments);
extern "C" __global__ void __launch_bounds__(NATIVE_THREADS, NATIVE_E2M1_WAVES) native_expert_down_1(struct wide_expert_down_arguments arguments, unsigned char *arena)
{
    native_expert_down<false, NATIVE_E2M1_COLUMN_BLOCKS / 4u>(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_NATIVE_LINEAR, native_expert_down_1, wide_expert_down_arguments);
#define NATIVE_E4M3_WAVES 3 /* 150 and 152 registers (with four sets of weight registers the down launch took 170 left to itself, and at two wavefronts a SIMD 487 against 461 us) */
extern "C" __global__ void __launch_bounds__(NATIVE_THREADS, NATIVE_E4M3_WAVES) native_expert_gate_up_e4m3_1(struct wide_expert_gate_up_arguments arguments, unsigned char *arena)
{
    native_expert_gate_up<true, 1u, NATIVE_E4M3_COLUMN_BLOCKS / 4u>(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_NATIVE_LINEAR, native_expert_gate_up_e4m3_1, wide_expert_gate_up_arguments);
extern "C" __global__ void __launch_bounds__(NATIVE_THREADS, NATIVE_E4M3_WAVES) native_expert_down_e4m3_1(struct wide_expert_down_arguments arguments, unsigned char *arena)
{
    native_expert_down<true, NATIVE_E4M3_COLUMN_BLOCKS / 4u>(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_NATIVE_LINEAR, native_expert_down_e4m3_1, wide_expert_down_arguments);

/* E4M3_BLOCK128_GFX950 experts (float32 scales of 128 x 128 blocks, columns of 128-value float32 scales): the E4M3_GFX950
 * launches' shape; the gate/up launch leaves the hidden VALUES where the record names the hidden operands, and their
 * quantizer (activation_quantize_128_entry) is a launch of its own */
extern "C" __global__ void __launch_bounds__(NATIVE_THREADS, NATIVE_B128_GATE_UP_WAVES) native_expert_gate_up_b128_1(struct wide_expert_gate_up_arguments arguments, unsigned char *arena)
{
    native_expert_gate_up<true, 1u, NATIVE_E4M3_COLUMN_BLOCKS / 4u, true>(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_NATIVE_LINEAR, native_expert_gate_up_b128_1, wide_expert_gate_up_arguments);
extern "C" __global__ void __launch_bounds__(NATIVE_THREADS, NATIVE_B128_DOWN_WAVES) native_expert_down_b128_1(struct wide_expert_down_arguments arguments, unsigned char *arena)
{
    native_expert_down<true, NATIVE_E4M3_COLUMN_BLOCKS / 4u, true>(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_NATIVE_LINEAR, native_expert_down_b128_1, wide_expert_down_arguments);

static_assert(native_chain<2, false, 2u, NATIVE_E2M1_COLUMN_BLOCKS, 3u, NATIVE_E2M1_STAGES>::WINDOW_BYTES == NATIVE_WINDOW_BYTES(NATIVE_E2M1_COLUMN_BLOCKS, NATIVE_E2M1_STAGES) &&
                  native_chain<1, true, 2u, NATIVE_E4M3_COLUMN_BLOCKS, 4u, NATIVE_E4M3_STAGES>::WINDOW_BYTES == NATIVE_WINDOW_BYTES(NATIVE_E4M3_COLUMN_BLOCKS, NATIVE_E4M3_STAGES),
              "the windows the host asks for are the kernels'");

