/*
 * kernel_expert_linear.hip -- the routed experts of the original FP4 weights on gfx950: gate and up products with the
 * hidden step, the down product, and the row sum. Entry names, records, launch shapes and rounding points follow the
 * reference (source/kernel_expert_linear.cu:157-231, 403-419; include/anemone/linear_records.h:45-99, 231-305):
 *   - weights WEIGHT_FORMAT_E2M1_SCALED exactly as stored (lane order words [tile][load][lane][step], E8M0 scales
 *     [tile][load][g] behind them; include/anemone/weight_format_seam.h:26-34), vectors as the quantizer writes them
 *     (E4M3 codes in lane order, E8M0 exponents per 32);
 *   - a product is cut in S slices of whole loads; a slice is one chain over its blocks of 32 inputs in ascending
 *     order; the S chains are added from +0 in order and the sum is rounded once to bfloat16;
 *   - the hidden step: g = min(gate, L), u = clamp(up, +-L), bf16(((g / (1 + exp(-g))) u) route weight), gate and up
 *     rounded to bfloat16 first.
 * The arithmetic form is the block-scaled one (the reference's native form, include/anemone/linear_records.h:63-66):
 * one v_mfma_scale_f32_16x16x128_f8f6f4 takes 128 inputs = four blocks of 32 with both E8M0 scale codes inside the
 * instruction and adds their terms to the running chain; E2M1 weights by E4M3 vector codes, no conversion.
 *
 * Work mapping (this build's own). What bounds a streaming kernel on this card, besides memory itself, is the number
 * of memory instructions: a compute unit takes one wavefront-wide load every 16 cycles whatever its width, which at
 * full memory speed leaves room for about six a KB of weights, and in practice far fewer. So:
 *   - a block is one strip of tiles (64 outputs of 4-bit weights, 32 of one-byte weights) of one job; a wavefront is one slice of the inputs, for the
 *     gate AND the up matrix (their sums meet in one lane for the hidden step, no exchange);
 *   - a stage is one K step (128 inputs) of all the wavefront's tiles: 1,024 bytes a tile go from memory straight
 *     into the wavefront's LDS window with one 16-byte-a-lane load (no registers in between), the tiles' 64 scale
 *     bytes each with one more load for every four tiles; two or three stages are on their way while one is used;
 *   - the codes of the job's (at most eight) vectors for the step and their scale codes travel the same way, one load
 *     each a stage, and serve every tile of the wavefront; nothing of the loop passes through registers, so the
 *     compiler has no wait of its own to place and the waits are this file's constants;
 *   - lane (o, g) of the MFMA needs output row o of inputs block g, which the stored form spreads over four stored
 *     lanes (t = 0..3) as the even (o < 8) or odd (o >= 8) nibbles of two words each: four 8-byte LDS reads, and two
 *     shifts, a shift and a bit-field insert a register.
 *
 * MFMA operand layout on gfx950, as measured on the card: A (fp4) lane l: row l % 16, element e = 8 v + n (register v,
 * nibble n) is k = 32 (l / 16) + e; B (fp8) lane l: column l % 16, element e = 4 v + b is k = 64 (e / 16) +
 * 16 (l / 16) + e % 16; scale of lane l: row or column l % 16, inputs block l / 16; D lane l: column l % 16, rows
 * 4 (l / 16) + v.
 */
#include "kernel_registry.h"
#include "linear_device.cuh"
#include "quantize_device.cuh"
#include "strip_device.cuh"


/* gate and up: block = S wavefronts (slices of the inputs); grid (ceil(output_size / 64), jobs) */
template <uint32_t S, bool BYTES, bool B128 = false, bool NATIVE = false>
__device__ static __forceinline__ void expert_gate_up(const struct expert_gate_up_arguments &arguments,
                                                      unsigned char *arena, uint16_t *strip_hidden = nullptr)
{
    typedef strip_chain<2, BYTES, B128, NATIVE> chain_type;
    constexpr uint32_t TILES = chain_type::TILES, STRIP = chain_type::STRIP;
    __shared__ __attribute__((aligned(16))) unsigned char window[S][chain_type::WINDOW_BYTES];
    static_assert(chain_type::WINDOW_BYTES >= TILES * WAVE * 16u, "a wavefront's sums fit its idle window");
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + arguments.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x % WAVE, slice = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t column = lane % 16u;
    const bool live = column < job->row_count; /* a job holds at most eight rows */
    const uint32_t pair = live ? job->pair_index[column] : 0u;
    uint32_t rows[8]; /* the vectors' rows; columns without a row read row 0, and are never stored */
#pragma unroll
    for (uint32_t c = 0; c < 8u; c++) {
        rows[c] = c < job->row_count ? job->pair_index[c] / arguments.pairs_per_row : 0u;
    }
    const uint32_t steps = arguments.input_size / 128u;
    const uint32_t first = steps * slice / S, last = steps * (slice + 1u) / S;
    chain_type chain_of;
    const unsigned char *const matrices[2] = {arena + job->gate_offset, arena + job->up_offset};
    chain_of.place(matrices, arguments.output_size, arguments.input_size, blockIdx.x, first, arena + arguments.codes_offset,
                   arena + arguments.exponents_offset, rows, (uint32_t)(uintptr_t)(lds_pointer)&window[slice][0], lane);
    float4_t chain[TILES];
#pragma unroll
    for (uint32_t tile = 0; tile < TILES; tile++) {
        chain[tile] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
    }
    chain_of.whole(last - first, chain);
    /* the S chains meet in the windows, idle now: [slice][tile][lane] float4 */
    float4_t *sums = (float4_t *)&window[slice][0];
#pragma unroll
    for (uint32_t tile = 0; tile < TILES; tile++) {
        sums[tile * WAVE + lane] = chain[tile];
    }
    __syncthreads();
    /* wavefront w finishes the tiles n = w, w + S, ..: the S chains from +0, in order, then the hidden step */
    const uint32_t tiles = arguments.output_size / 16u;
    const uint32_t tile0 = blockIdx.x * STRIP + STRIP <= tiles ? blockIdx.x * STRIP : tiles - STRIP;
    for (uint32_t n = slice; n < STRIP; n += S) {
        if (!live || tile0 + n < blockIdx.x * STRIP) { /* a tile the strip before this one stores */
            continue;
        }
        float gate[4] = {0.0f, 0.0f, 0.0f, 0.0f}, up[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (uint32_t part = 0; part < S; part++) {
            const float4_t g4 = ((const float4_t *)&window[part][0])[n * WAVE + lane];
            const float4_t u4 = ((const float4_t *)&window[part][0])[(STRIP + n) * WAVE + lane];
#pragma unroll
            for (uint32_t v = 0; v < 4u; v++) {
                gate[v] = __fadd_rn(gate[v], g4[v]);
                up[v] = __fadd_rn(up[v], u4[v]);
            }
        }
        const float limit = arguments.activation_limit, weight = job->route_weight[column];
        uint16_t hidden[4];
#pragma unroll
        for (uint32_t v = 0; v < 4u; v++) {
            const float g = bf16_to_float(float_to_bf16(gate[v])), u = bf16_to_float(float_to_bf16(up[v]));
            const float bounded_gate = fminf(g, limit);
            const float bounded_up = fminf(fmaxf(u, -limit), limit);
            const float value = __fmul_rn(__fmul_rn(linear_silu(bounded_gate), bounded_up), weight);
            hidden[v] = float_to_bf16(value);
        }
        uint16_t *out = (uint16_t *)(arena + arguments.hidden_offset) + (uint64_t)pair * arguments.output_size +
                        (tile0 + n) * 16u + 4u * (lane / 16u);
        *(uint2_t *)out = (uint2_t){(uint32_t)hidden[0] | ((uint32_t)hidden[1] << 16), (uint32_t)hidden[2] | ((uint32_t)hidden[3] << 16)};
        if (strip_hidden != nullptr) { /* the producer's copy: [column][the strip's outputs] */
            uint16_t *copy = strip_hidden + column * (STRIP * 16u) + n * 16u + 4u * (lane / 16u);
#pragma unroll
            for (uint32_t v = 0; v < 4u; v++) {
                copy[v] = hidden[v];
            }
        }
    }
}

/* The producer: gate with up, then the quantization of the strip's hidden values, in one launch. A block of the
 * quantization is 32 consecutive outputs and a strip holds whole blocks (64 outputs of 4-bit weights, 32 of one-byte
 * weights), so the second step needs nothing of another block: the hidden values pass through LDS. One more row of
 * blocks (blockIdx.y = the jobs' number) quantizes, from memory, the pairs that stand in no job, as the quantizer's
 * own launch does. Grid (ceil(output_size / strip), jobs + 1). */
template <uint32_t S, bool BYTES>
__device__ static __forceinline__ void expert_gate_up_quantize(const struct expert_gate_up_quantize_arguments &arguments,
                                                               unsigned char *arena)
{
    typedef strip_chain<2, BYTES> chain_type;
    constexpr uint32_t STRIP_OUTPUTS = chain_type::STRIP * 16u;
    __shared__ uint16_t strip_hidden[LINEAR_MAXIMUM_ROWS][STRIP_OUTPUTS];
    __shared__ uint32_t routed[EXPERT_PRODUCER_MOST_PAIRS / 32u];
    const uint32_t tiles = arguments.output_size / 16u;
    const uint32_t tile0 = blockIdx.x * chain_type::STRIP + chain_type::STRIP <= tiles ? blockIdx.x * chain_type::STRIP : tiles - chain_type::STRIP;
    const uint32_t lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t width = arguments.output_size;
    const uint32_t first_output = blockIdx.x * STRIP_OUTPUTS; /* a last strip that reaches past the matrix starts earlier */
    if (blockIdx.y + 1u == gridDim.y) {
        /* the pairs no job holds: a bit a pair from the job table (a job a pair at most), then the quantizer's work */
        const struct expert_job_record *jobs = (const struct expert_job_record *)(arena + arguments.jobs_offset);
        if (threadIdx.x < EXPERT_PRODUCER_MOST_PAIRS / 32u) {
            uint32_t bits = 0;
            for (uint32_t job = 0; job < arguments.pair_count; job++) {
                for (uint32_t column = 0; column < jobs[job].row_count; column++) {
                    const uint32_t pair = jobs[job].pair_index[column];
                    bits |= pair / 32u == threadIdx.x ? 1u << (pair % 32u) : 0u;
                }
            }
            routed[threadIdx.x] = bits;
        }
        __syncthreads();
        for (uint32_t pair = wave; pair < arguments.pair_count; pair += S) {
            if ((routed[pair / 32u] >> (pair % 32u)) & 1u) {
                continue;
            }
            for (uint32_t at = lane; at < STRIP_OUTPUTS; at += WAVE) {
                const uint32_t index = tile0 * 16u + at;
                if (index < first_output) { /* whole blocks of 32 that the strip before this one takes */
                    continue;
                }
                const uint32_t bits = ((const uint16_t *)(arena + arguments.hidden_offset))[(uint64_t)pair * width + index];
                quantize_value(bits, index, arena + arguments.hidden_codes_offset + (uint64_t)pair * width,
                               arena + arguments.hidden_exponents_offset + (uint64_t)pair * (width / 32u),
                               (uint16_t *)(arena + arguments.hidden_operands_offset) + (uint64_t)pair * width);
            }
        }
        return;
    }
    const struct expert_gate_up_arguments plain = {arguments.jobs_offset, arguments.codes_offset, arguments.exponents_offset,
                                                   arguments.operands_offset, arguments.hidden_offset, arguments.output_size,
                                                   arguments.input_size, arguments.pair_count, arguments.pairs_per_row,
                                                   arguments.activation_limit, 0u};
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + arguments.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    expert_gate_up<S, BYTES>(plain, arena, &strip_hidden[0][0]);
    __syncthreads();
    for (uint32_t column = wave; column < job->row_count; column += S) {
        const uint64_t pair = job->pair_index[column];
        for (uint32_t at = lane; at < STRIP_OUTPUTS; at += WAVE) {
            if (tile0 * 16u + at < first_output) {
                continue;
            }
            quantize_value(strip_hidden[column][at], tile0 * 16u + at, arena + arguments.hidden_codes_offset + pair * width,
                           arena + arguments.hidden_exponents_offset + pair * (width / 32u),
                           (uint16_t *)(arena + arguments.hidden_operands_offset) + pair * width);
        }
    }
}

/* down: block = S wavefronts; grid (ceil(output_size / 64), jobs) */
template <uint32_t S, bool BYTES, bool B128 = false, bool NATIVE = false>
__device__ static __forceinline__ void expert_down(const struct expert_down_arguments &arguments, unsigned char *arena)
{
    typedef strip_chain<1, BYTES, B128, NATIVE> chain_type;
    constexpr uint32_t TILES = chain_type::TILES, STRIP = chain_type::STRIP;
    __shared__ __attribute__((aligned(16))) unsigned char window[S][chain_type::WINDOW_BYTES];
    static_assert(chain_type::WINDOW_BYTES >= TILES * WAVE * 16u, "a wavefront's sums fit its idle window");
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + arguments.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x % WAVE, slice = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), column = lane % 16u;
    const bool live = column < job->row_count;
    const uint64_t pair = live ? job->pair_index[column] : 0u;
    uint32_t rows[8]; /* the vectors are the pairs' hidden vectors */
#pragma unroll
    for (uint32_t c = 0; c < 8u; c++) {
        rows[c] = c < job->row_count ? job->pair_index[c] : 0u;
    }
    const uint32_t steps = arguments.input_size / 128u;
    const uint32_t first = steps * slice / S, last = steps * (slice + 1u) / S;
    chain_type chain_of;
    const unsigned char *const matrices[1] = {arena + job->down_offset};
    chain_of.place(matrices, arguments.output_size, arguments.input_size, blockIdx.x, first, arena + arguments.codes_offset,
                   arena + arguments.exponents_offset, rows, (uint32_t)(uintptr_t)(lds_pointer)&window[slice][0], lane);
    float4_t chain[TILES];
#pragma unroll
    for (uint32_t tile = 0; tile < TILES; tile++) {
        chain[tile] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
    }
    chain_of.whole(last - first, chain);
    float4_t *sums = (float4_t *)&window[slice][0];
#pragma unroll
    for (uint32_t tile = 0; tile < TILES; tile++) {
        sums[tile * WAVE + lane] = chain[tile];
    }
    __syncthreads();
    const uint32_t tiles = arguments.output_size / 16u;
    const uint32_t tile0 = blockIdx.x * STRIP + STRIP <= tiles ? blockIdx.x * STRIP : tiles - STRIP;
    for (uint32_t n = slice; n < STRIP; n += S) {
        if (!live || tile0 + n < blockIdx.x * STRIP) {
            continue;
        }
        float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (uint32_t part = 0; part < S; part++) {
            const float4_t d4 = ((const float4_t *)&window[part][0])[n * WAVE + lane];
#pragma unroll
            for (uint32_t v = 0; v < 4u; v++) {
                sum[v] = __fadd_rn(sum[v], d4[v]);
            }
        }
        uint16_t *out = (uint16_t *)(arena + arguments.output_offset) + pair * arguments.output_size + (tile0 + n) * 16u + 4u * (lane / 16u);
        *(uint2_t *)out = (uint2_t){(uint32_t)float_to_bf16(sum[0]) | ((uint32_t)float_to_bf16(sum[1]) << 16),
                                    (uint32_t)float_to_bf16(sum[2]) | ((uint32_t)float_to_bf16(sum[3]) << 16)};
    }
}

/* expert_gate_up_<S>, expert_down_<S>: the reference's entries, of WEIGHT_FORMAT_E2M1_SCALED experts. The _e4m3_
 * entries take WEIGHT_FORMAT_E4M3_SCALED experts (a format the reference stores and lays out but multiplies in its
 * trunk alone: no counterpart among its expert kernels); same records, same rounding points. The _b128_ entries take
 * WEIGHT_FORMAT_E4M3_BLOCK128 experts (E4M3 codes with one float32 scale for every 128 x 128 block, vectors quantized a
 * 128 values with float32 scales, read where the records name the exponents: no counterpart in the reference). The
 * _gfx950_ entries take experts stored in the card's own lane order (WEIGHT_FORMAT_E2M1_GFX950, _E4M3_GFX950,
 * _E4M3_BLOCK128_GFX950: no counterpart in the reference) and give the sums of the same matrices in the reference's lay-out, bit for bit. */
#define EXPERT_ENTRIES(S)                                                                                         \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_gate_up_##S(struct expert_gate_up_arguments arguments, unsigned char *arena)                      \
    {                                                                                                             \
        expert_gate_up<S, false>(arguments, arena);                                                               \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_##S, expert_gate_up_arguments);                      \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_down_##S(struct expert_down_arguments arguments, unsigned char *arena)                            \
    {                                                                                                             \
        expert_down<S, false>(arguments, arena);                                                                  \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_down_##S, expert_down_arguments);                            \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_gate_up_e4m3_##S(struct expert_gate_up_arguments arguments, unsigned char *arena)                 \
    {                                                                                                             \
        expert_gate_up<S, true>(arguments, arena);                                                                \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_e4m3_##S, expert_gate_up_arguments);                 \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_down_e4m3_##S(struct expert_down_arguments arguments, unsigned char *arena)                       \
    {                                                                                                             \
        expert_down<S, true>(arguments, arena);                                                                   \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_down_e4m3_##S, expert_down_arguments);                       \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_gate_up_quantize_##S(struct expert_gate_up_quantize_arguments arguments, unsigned char *arena)    \
    {                                                                                                             \
        expert_gate_up_quantize<S, false>(arguments, arena);                                                      \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_quantize_##S, expert_gate_up_quantize_arguments);    \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_gate_up_quantize_e4m3_##S(struct expert_gate_up_quantize_arguments arguments, unsigned char *arena) \
    {                                                                                                             \
        expert_gate_up_quantize<S, true>(arguments, arena);                                                       \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_quantize_e4m3_##S, expert_gate_up_quantize_arguments);   \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_gate_up_b128_##S(struct expert_gate_up_arguments arguments, unsigned char *arena)                 \
    {                                                                                                             \
        expert_gate_up<S, true, true>(arguments, arena);                                                          \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_b128_##S, expert_gate_up_arguments);                 \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_down_b128_##S(struct expert_down_arguments arguments, unsigned char *arena)                       \
    {                                                                                                             \
        expert_down<S, true, true>(arguments, arena);                                                             \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_down_b128_##S, expert_down_arguments);                       \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_gate_up_gfx950_##S(struct expert_gate_up_arguments arguments, unsigned char *arena)               \
    {                                                                                                             \
        expert_gate_up<S, false, false, true>(arguments, arena);                                                  \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_gfx950_##S, expert_gate_up_arguments);               \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_down_gfx950_##S(struct expert_down_arguments arguments, unsigned char *arena)                     \
    {                                                                                                             \
        expert_down<S, false, false, true>(arguments, arena);                                                     \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_down_gfx950_##S, expert_down_arguments);                     \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_gate_up_e4m3_gfx950_##S(struct expert_gate_up_arguments arguments, unsigned char *arena)          \
    {                                                                                                             \
        expert_gate_up<S, true, false, true>(arguments, arena);                                                   \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_e4m3_gfx950_##S, expert_gate_up_arguments);          \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_down_e4m3_gfx950_##S(struct expert_down_arguments arguments, unsigned char *arena)                \
    {                                                                                                             \
        expert_down<S, true, false, true>(arguments, arena);                                                      \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_down_e4m3_gfx950_##S, expert_down_arguments);                \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_gate_up_b128_gfx950_##S(struct expert_gate_up_arguments arguments, unsigned char *arena)          \
    {                                                                                                             \
        expert_gate_up<S, true, true, true>(arguments, arena);                                                    \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_b128_gfx950_##S, expert_gate_up_arguments);          \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_down_b128_gfx950_##S(struct expert_down_arguments arguments, unsigned char *arena)                \
    {                                                                                                             \
        expert_down<S, true, true, true>(arguments, arena);                                                       \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_down_b128_gfx950_##S, expert_down_arguments)
EXPERT_ENTRIES(1);
EXPERT_ENTRIES(2);
EXPERT_ENTRIES(4);
EXPERT_ENTRIES(8);

/* float32 sum of a row's bfloat16 pair outputs from +0 in ascending slot order; a thread takes
 * EXPERT_ROW_SUM_CHANNELS consecutive outputs (one 16-byte load a slot); grid (ceil(width / (8 x 256)), rows) */
extern "C" __global__ void expert_row_sum_entry(struct expert_row_sum_arguments arguments, unsigned char *arena)
{
    const uint32_t channel = (blockIdx.x * blockDim.x + threadIdx.x) * EXPERT_ROW_SUM_CHANNELS;
    if (channel >= arguments.width) {
        return;
    }
    const uint64_t row = blockIdx.y;
    const uint16_t *pairs = (const uint16_t *)(arena + arguments.pair_output_offset) + row * arguments.pairs_per_row * arguments.width + channel;
    float *out = (float *)(arena + arguments.row_output_offset) + row * arguments.width + channel;
    float sum[EXPERT_ROW_SUM_CHANNELS];
#pragma unroll
    for (uint32_t i = 0; i < EXPERT_ROW_SUM_CHANNELS; i++) {
        sum[i] = 0.0f;
    }
    if (arguments.width % EXPERT_ROW_SUM_CHANNELS == 0u) {
        for (uint32_t slot = 0; slot < arguments.pairs_per_row; slot++) {
            const uint4_t eight = *(const uint4_t *)(pairs + (uint64_t)slot * arguments.width);
            const uint32_t words[4] = {eight.x, eight.y, eight.z, eight.w};
#pragma unroll
            for (uint32_t i = 0; i < EXPERT_ROW_SUM_CHANNELS; i++) {
                sum[i] = __fadd_rn(sum[i], __uint_as_float(i % 2u == 0u ? words[i / 2u] << 16 : words[i / 2u] & 0xFFFF0000u));
            }
        }
        *(float4_t *)out = (float4_t){sum[0], sum[1], sum[2], sum[3]};
        *(float4_t *)(out + 4) = (float4_t){sum[4], sum[5], sum[6], sum[7]};
        return;
    }
    for (uint32_t i = 0; i < EXPERT_ROW_SUM_CHANNELS && channel + i < arguments.width; i++) { /* a width that is no multiple of 8 */
        float one = 0.0f;
        for (uint32_t slot = 0; slot < arguments.pairs_per_row; slot++) {
            one = __fadd_rn(one, bf16_to_float(pairs[(uint64_t)slot * arguments.width + i]));
        }
        out[i] = one;
    }
}
ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_row_sum_entry, expert_row_sum_arguments);
