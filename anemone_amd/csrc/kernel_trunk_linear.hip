/*
 * kernel_trunk_linear.hip -- the shared expert's linears on gfx950: y = W x of one or two matrices stored as
 * WEIGHT_FORMAT_E4M3_SCALED for rows of quantized vectors, the hidden step alone, and the shared expert's down with
 * the FFN site's join behind it. Entry names, records and rounding points follow the reference
 * (include/anemone/linear_records.h:106-125, 307-356; include/anemone/expert_fused_records.h:42-52;
 * source/kernel_trunk_linear.cu): a product is cut in S slices of whole loads, a slice is one chain over its blocks
 * of 32 inputs in ascending order, the S chains are added from +0 in order and the sum is rounded once to bfloat16.
 * The arithmetic form is the block-scaled one (v_mfma_scale_f32_16x16x128_f8f6f4 with both E8M0 scales inside), the
 * chains those of the routed experts' kernels (strip_device.cuh, wide_device.cuh).
 *   - trunk_linear_quantized_<S>: 1 to LINEAR_MAXIMUM_ROWS rows. A block is one strip of TRUNK_STRIP_OUTPUTS outputs
 *     of one matrix (matrix 1's strips follow matrix 0's), S wavefronts its slices; grid (strips of both, 1).
 *   - trunk_linear_quantized_wide_<S>: any number of rows in groups of LINEAR_MAXIMUM_ROWS; of grid[0] = strips x n,
 *     block b computes strip b / n for the groups b % n, b % n + n, .., one after the other, each exactly as the thin
 *     instance computes a launch of those rows alone: every output has the thin instance's bits, whatever n.
 *   - trunk_linear_quantized_interleaved_1: one slice, for steps of many rows. A block is one tile of
 *     TRUNK_INTERLEAVED_ROWS rows (four MFMA column blocks) by TRUNK_INTERLEAVED_BLOCK_OUTPUTS outputs of one matrix;
 *     grid (blocks of both matrices, tiles of rows). An output's chain is the same MFMAs on the same operands in the
 *     same order as the thin instance's of one slice: the same bits.
 *   - trunk_hidden_entry: bfloat16((g / (1 + exp(-g))) u) of g = min(gate, L), u = clamp(up, +-L), a route weight of 1.
 *   - expert_shared_join_<S>: trunk_linear_quantized_<S> of the shared expert's down and behind it the join
 *     (join_device.cuh) of the strip's outputs, read from where the block keeps them.
 */
#include "kernel_registry.h"
#include "join_device.cuh"
#include "linear_device.cuh"
#include "strip_device.cuh"
#include "wide_device.cuh"

/* which matrix a block of grid[0] works on, and which of its blocks: matrix 1's follow matrix 0's */
__device__ static __forceinline__ void trunk_matrix_of(const struct trunk_linear_quantized_arguments &arguments, uint32_t block,
                                                       uint32_t block_outputs, uint32_t &matrix, uint32_t &index)
{
    const uint32_t first = (arguments.output_size[0] + block_outputs - 1u) / block_outputs;
    matrix = block < first ? 0u : 1u;
    index = block < first ? block : block - first;
}

/* One strip of one matrix for rows first_row .. first_row + row_count - 1 (at most LINEAR_MAXIMUM_ROWS); every thread
 * of the block calls it (barriers inside). copy: where the block keeps the strip's outputs for a step behind the
 * product, [row][TRUNK_STRIP_OUTPUTS] bfloat16, or nullptr. */
template <uint32_t S>
__device__ static __forceinline__ void trunk_strip(const unsigned char *matrix, uint32_t outputs, uint32_t inputs, uint32_t strip,
                                                   const unsigned char *codes, const unsigned char *exponents, uint32_t first_row,
                                                   uint32_t row_count, uint16_t *out, unsigned char *window_bytes, uint16_t *copy)
{
    typedef strip_chain<1, true> chain_type;
    constexpr uint32_t TILES = chain_type::TILES, STRIP = chain_type::STRIP;
    static_assert(STRIP * 16u == TRUNK_STRIP_OUTPUTS && chain_type::WINDOW_BYTES >= TILES * WAVE * 16u, "a strip is 32 outputs; a wavefront's sums fit its idle window");
    const uint32_t lane = threadIdx.x % WAVE, slice = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), column = lane % 16u;
    const bool live = column < row_count;
    uint32_t rows[8]; /* columns without a row read the first row; their sums are never stored */
#pragma unroll
    for (uint32_t c = 0; c < 8u; c++) {
        rows[c] = first_row + (c < row_count ? c : 0u);
    }
    const uint32_t steps = inputs / 128u;
    const uint32_t first = steps * slice / S, last = steps * (slice + 1u) / S;
    chain_type chain_of;
    const unsigned char *const matrices[1] = {matrix};
    unsigned char *window = window_bytes + slice * chain_type::WINDOW_BYTES;
    chain_of.place(matrices, outputs, inputs, strip, first, codes, exponents, rows, (uint32_t)(uintptr_t)(lds_pointer)window, lane);
    float4_t chain[TILES];
#pragma unroll
    for (uint32_t tile = 0; tile < TILES; tile++) {
        chain[tile] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
    }
    chain_of.whole(last - first, chain);
    float4_t *sums = (float4_t *)window;
#pragma unroll
    for (uint32_t tile = 0; tile < TILES; tile++) {
        sums[tile * WAVE + lane] = chain[tile];
    }
    __syncthreads();
    const uint32_t tiles = outputs / 16u;
    const uint32_t tile0 = strip * STRIP + STRIP <= tiles ? strip * STRIP : tiles - STRIP;
    for (uint32_t n = slice; n < STRIP; n += S) {
        if (!live || tile0 + n < strip * STRIP) { /* a tile the strip before this one stores */
            continue;
        }
        float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (uint32_t part = 0; part < S; part++) {
            const float4_t d4 = ((const float4_t *)(window_bytes + part * chain_type::WINDOW_BYTES))[n * WAVE + lane];
#pragma unroll
            for (uint32_t v = 0; v < 4u; v++) {
                sum[v] = __fadd_rn(sum[v], d4[v]);
            }
        }
        const uint2_t four = {(uint32_t)float_to_bf16(sum[0]) | ((uint32_t)float_to_bf16(sum[1]) << 16),
                              (uint32_t)float_to_bf16(sum[2]) | ((uint32_t)float_to_bf16(sum[3]) << 16)};
        *(uint2_t *)(out + (uint64_t)(first_row + column) * outputs + (tile0 + n) * 16u + 4u * (lane / 16u)) = four;
        if (copy != nullptr) {
            *(uint2_t *)(copy + column * TRUNK_STRIP_OUTPUTS + n * 16u + 4u * (lane / 16u)) = four;
        }
    }
}

#define TRUNK_WINDOW(S) __shared__ __attribute__((aligned(16))) unsigned char window[S * strip_chain<1, true>::WINDOW_BYTES]

template <uint32_t S>
__device__ static __forceinline__ void trunk_linear_quantized(const struct trunk_linear_quantized_arguments &arguments, unsigned char *arena)
{
    TRUNK_WINDOW(S);
    uint32_t matrix, strip;
    trunk_matrix_of(arguments, blockIdx.x, TRUNK_STRIP_OUTPUTS, matrix, strip);
    trunk_strip<S>(arena + arguments.weights_offset[matrix], arguments.output_size[matrix], arguments.input_size, strip,
                   arena + arguments.codes_offset, arena + arguments.exponents_offset, 0u, arguments.row_count,
                   (uint16_t *)(arena + arguments.output_offset[matrix]), window, nullptr);
}

template <uint32_t S>
__device__ static __forceinline__ void trunk_linear_quantized_wide(const struct trunk_linear_quantized_arguments &arguments, unsigned char *arena)
{
    TRUNK_WINDOW(S);
    const uint32_t strips = (arguments.output_size[0] + TRUNK_STRIP_OUTPUTS - 1u) / TRUNK_STRIP_OUTPUTS +
                            (arguments.output_size[1] + TRUNK_STRIP_OUTPUTS - 1u) / TRUNK_STRIP_OUTPUTS;
    const uint32_t n = gridDim.x / strips, groups = (arguments.row_count + LINEAR_MAXIMUM_ROWS - 1u) / LINEAR_MAXIMUM_ROWS;
    uint32_t matrix, strip;
    trunk_matrix_of(arguments, blockIdx.x / n, TRUNK_STRIP_OUTPUTS, matrix, strip);
    for (uint32_t group = blockIdx.x % n; group < groups; group += n) {
        const uint32_t first_row = group * LINEAR_MAXIMUM_ROWS;
        const uint32_t rows = arguments.row_count - first_row < LINEAR_MAXIMUM_ROWS ? arguments.row_count - first_row : LINEAR_MAXIMUM_ROWS;
        trunk_strip<S>(arena + arguments.weights_offset[matrix], arguments.output_size[matrix], arguments.input_size, strip,
                       arena + arguments.codes_offset, arena + arguments.exponents_offset, first_row, rows,
                       (uint16_t *)(arena + arguments.output_offset[matrix]), window, nullptr);
        __syncthreads(); /* the windows are read before the next group's loads land in them */
    }
}

/* grid (ceil(output_size[0] / 128) + ceil(output_size[1] / 128), ceil(row_count / 64)), block 256 */
__device__ static __forceinline__ void trunk_linear_quantized_interleaved(const struct trunk_linear_quantized_arguments &arguments, unsigned char *arena)
{
    typedef wide_chain<1, true, 2u, 2u> chain_type;
    constexpr uint32_t TILES = chain_type::TILES, STRIP = chain_type::STRIP, STRIP_OUTPUTS = STRIP * 16u;
    static_assert(chain_type::WINDOW_BYTES == TRUNK_INTERLEAVED_WINDOW_BYTES && WIDE_WAVES * STRIP_OUTPUTS == TRUNK_INTERLEAVED_BLOCK_OUTPUTS &&
                      WIDE_TILE_PAIRS == TRUNK_INTERLEAVED_ROWS, "the window and the block the host asks for are the kernel's");
    extern __shared__ __attribute__((aligned(16))) unsigned char wide_window[];
    uint32_t matrix, block;
    trunk_matrix_of(arguments, blockIdx.x, TRUNK_INTERLEAVED_BLOCK_OUTPUTS, matrix, block);
    const uint32_t outputs = arguments.output_size[matrix];
    const uint32_t lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t first_row = blockIdx.y * TRUNK_INTERLEAVED_ROWS;
    const uint32_t row_count = arguments.row_count - first_row < TRUNK_INTERLEAVED_ROWS ? arguments.row_count - first_row : TRUNK_INTERLEAVED_ROWS;
    /* columns past the tile's last row read its first row's vector; their sums are never stored */
    uint32_t code_vectors[2];
#pragma unroll
    for (uint32_t part = 0; part < 2u; part++) {
        const uint32_t column = 8u * (2u * wave + part) + lane / 8u;
        code_vectors[part] = first_row + (column < row_count ? column : 0u);
    }
    const uint32_t scale_column = 16u * wave + lane % 16u;
    const uint32_t exponent_vector = first_row + (scale_column < row_count ? scale_column : 0u);
    chain_type chain_of;
    const unsigned char *const matrices[1] = {arena + arguments.weights_offset[matrix]};
    uint32_t tile0 = 0;
    chain_of.place(matrices, outputs, arguments.input_size, block, arena + arguments.codes_offset, arena + arguments.exponents_offset,
                   code_vectors, exponent_vector, (uint32_t)(uintptr_t)(lds_pointer)wide_window, wave, lane, tile0);
    float4_t chain[TILES][WIDE_COLUMN_BLOCKS];
#pragma unroll
    for (uint32_t t = 0; t < TILES; t++) {
#pragma unroll
        for (uint32_t j = 0; j < WIDE_COLUMN_BLOCKS; j++) {
            chain[t][j] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
    chain_of.whole(arguments.input_size / 128u, (row_count + 15u) / 16u, chain);
    const uint32_t first_output = (block * WIDE_WAVES + wave) * STRIP_OUTPUTS;
    if (first_output >= outputs) {
        return;
    }
#pragma unroll
    for (uint32_t j = 0; j < WIDE_COLUMN_BLOCKS; j++) {
        const uint32_t column = 16u * j + lane % 16u;
        if (column < row_count) {
#pragma unroll
            for (uint32_t n = 0; n < STRIP; n++) {
                if ((tile0 + n) * 16u < first_output) {
                    continue; /* a tile the strip before this one stores */
                }
                uint16_t *out = (uint16_t *)(arena + arguments.output_offset[matrix]) + (uint64_t)(first_row + column) * outputs + (tile0 + n) * 16u + 4u * (lane / 16u);
                const float s0 = __fadd_rn(0.0f, chain[n][j][0]), s1 = __fadd_rn(0.0f, chain[n][j][1]);
                const float s2 = __fadd_rn(0.0f, chain[n][j][2]), s3 = __fadd_rn(0.0f, chain[n][j][3]);
                *(uint2_t *)out = (uint2_t){(uint32_t)float_to_bf16(s0) | ((uint32_t)float_to_bf16(s1) << 16),
                                            (uint32_t)float_to_bf16(s2) | ((uint32_t)float_to_bf16(s3) << 16)};
            }
        }
    }
}

/* The shared expert's down and the join of its strip: grid (ceil(width / 32), 1), block 64 S. Thread 4 r + h joins
 * values 8 h .. 8 h + 7 of the strip for row r, reading the strip's outputs from the block's copy. */
template <uint32_t S>
__device__ static __forceinline__ void expert_shared_join(const struct expert_shared_join_arguments &arguments, unsigned char *arena)
{
    TRUNK_WINDOW(S);
    __shared__ __attribute__((aligned(16))) uint16_t copy[LINEAR_MAXIMUM_ROWS][TRUNK_STRIP_OUTPUTS];
    const uint32_t width = arguments.reserved_zero == 0u ? 5120u : arguments.reserved_zero, strip = blockIdx.x;
    trunk_strip<S>(arena + arguments.weights_offset, width, arguments.input_size, strip, arena + arguments.codes_offset,
                   arena + arguments.exponents_offset, 0u, arguments.row_count, (uint16_t *)(arena + arguments.output_offset), window, &copy[0][0]);
    __syncthreads();
    const uint32_t row = threadIdx.x / 4u, piece = threadIdx.x % 4u;
    /* a last strip that reaches past the matrix starts earlier: its first outputs are the strip's before it */
    const uint32_t tiles = width / 16u, tile0 = strip * 2u + 2u <= tiles ? strip * 2u : tiles - 2u;
    const uint32_t output = tile0 * 16u + piece * HYPER_VALUES_PER_THREAD;
    if (row >= arguments.row_count || output < strip * TRUNK_STRIP_OUTPUTS) {
        return;
    }
    const uint64_t row_threads = width / HYPER_VALUES_PER_THREAD, thread = output / HYPER_VALUES_PER_THREAD;
    float shared_output[HYPER_VALUES_PER_THREAD];
    join_unpack(*(const uint4_t *)&copy[row][piece * HYPER_VALUES_PER_THREAD], shared_output);
    join_values((const uint4_t *)(arena + arguments.pair_output_offset) + (uint64_t)row * arguments.pairs_per_row * row_threads + thread,
                arguments.pairs_per_row, shared_output, (const float *)(arena + arguments.post_offset) + (uint64_t)row * MODEL_STREAMS,
                (const float *)(arena + arguments.comb_offset) + (uint64_t)row * MODEL_STREAMS * MODEL_STREAMS,
                (uint4_t *)(arena + arguments.streams_offset) + (uint64_t)row * MODEL_STREAMS * row_threads + thread,
                arguments.row_sums_offset == EXPERT_JOIN_NO_ROW_SUMS
                    ? nullptr
                    : (float4_t *)(arena + arguments.row_sums_offset) + ((uint64_t)row * row_threads + thread) * 2u,
                row_threads);
}

#define TRUNK_ENTRIES(S)                                                                                          \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        trunk_linear_quantized_##S(struct trunk_linear_quantized_arguments arguments, unsigned char *arena)       \
    {                                                                                                             \
        trunk_linear_quantized<S>(arguments, arena);                                                              \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_TRUNK_LINEAR, trunk_linear_quantized_##S, trunk_linear_quantized_arguments);       \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        trunk_linear_quantized_wide_##S(struct trunk_linear_quantized_arguments arguments, unsigned char *arena)  \
    {                                                                                                             \
        trunk_linear_quantized_wide<S>(arguments, arena);                                                         \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_TRUNK_LINEAR, trunk_linear_quantized_wide_##S, trunk_linear_quantized_arguments);  \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_shared_join_##S(struct expert_shared_join_arguments arguments, unsigned char *arena)               \
    {                                                                                                             \
        expert_shared_join<S>(arguments, arena);                                                                  \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_TRUNK_LINEAR, expert_shared_join_##S, expert_shared_join_arguments)
TRUNK_ENTRIES(1);
TRUNK_ENTRIES(2);
TRUNK_ENTRIES(4);
TRUNK_ENTRIES(8);

extern "C" __global__ void __launch_bounds__(WIDE_THREADS)
    trunk_linear_quantized_interleaved_1(struct trunk_linear_quantized_arguments arguments, unsigned char *arena)
{
    trunk_linear_quantized_interleaved(arguments, arena);
}
ANEMONE_KERNEL(KERNEL_FILE_TRUNK_LINEAR, trunk_linear_quantized_interleaved_1, trunk_linear_quantized_arguments);

/* grid (ceil(width / (8 block[0])), vectors): a thread takes eight consecutive values where the width is a multiple of
 * eight, else one value at a time */
extern "C" __global__ void trunk_hidden_entry(struct trunk_hidden_arguments arguments, unsigned char *arena)
{
    const uint32_t first = (blockIdx.x * blockDim.x + threadIdx.x) * HYPER_VALUES_PER_THREAD;
    if (first >= arguments.width) {
        return;
    }
    const uint64_t at = (uint64_t)blockIdx.y * arguments.width + first;
    const uint16_t *gate = (const uint16_t *)(arena + arguments.gate_offset) + at, *up = (const uint16_t *)(arena + arguments.up_offset) + at;
    uint16_t *hidden = (uint16_t *)(arena + arguments.hidden_offset) + at;
    const float limit = arguments.activation_limit;
    if (arguments.width % HYPER_VALUES_PER_THREAD == 0u) {
        float g[HYPER_VALUES_PER_THREAD], u[HYPER_VALUES_PER_THREAD], h[HYPER_VALUES_PER_THREAD];
        join_unpack(*(const uint4_t *)gate, g);
        join_unpack(*(const uint4_t *)up, u);
#pragma unroll
        for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
            const float bounded_gate = fminf(g[v], limit), bounded_up = fminf(fmaxf(u[v], -limit), limit);
            h[v] = __fmul_rn(__fmul_rn(det_silu(bounded_gate), bounded_up), 1.0f);
        }
        *(uint4_t *)hidden = join_pack(h);
        return;
    }
    for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD && first + v < arguments.width; v++) {
        const float bounded_gate = fminf(bf16_to_float(gate[v]), limit), bounded_up = fminf(fmaxf(bf16_to_float(up[v]), -limit), limit);
        hidden[v] = float_to_bf16(__fmul_rn(__fmul_rn(det_silu(bounded_gate), bounded_up), 1.0f));
    }
}
ANEMONE_KERNEL(KERNEL_FILE_TRUNK_LINEAR, trunk_hidden_entry, trunk_hidden_arguments);
