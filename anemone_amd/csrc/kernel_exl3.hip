/*
 * kernel_exl3.hip -- EXL3 (trellis, codebook mul1) reconstruction and the routed experts' five-launch chain for
 * gfx950. Entry names and records are the reference's (source/kernel_exl3.cu, include/anemone/exl3_records.h);
 * the work mapping is this build's: one wavefront per 128-value transform block, and products by wavefronts that
 * stream strips of eight output tiles through LDS into v_mfma_f32_16x16x32_f16 (exl3_device.cuh).
 *
 * Arithmetic contract (source/kernel_exl3.cu:133-424): operands fp16( H128(bf16 x . fp16 suh) . norm ); products
 * float32 in four contiguous K slices added in slice order from +0; hidden bf16( min(g, L) / (1 + e^-g) . clamp(u) )
 * with g, u = H128(product) . norm . svh; down operand from the unrounded hidden value; pair output
 * H128(down product) . norm . svh . route weight, in place of the down products; row sum in slot order from +0.
 * Inside a slice the MFMA adds 32 products at a time in its own order, which no host reference has bit for bit.
 */
#include "exl3_device.cuh"
#include "kernel_registry.h"

#define PRODUCT_WAVES EXL3_PRODUCT_SLICES
#define PRODUCT_THREADS (PRODUCT_WAVES * WAVE)

extern "C" __global__ void exl3_reconstruct(struct exl3_reconstruct_record record, unsigned char *arena)
{
    const uint64_t element = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (element >= (uint64_t)record.input_size * record.output_size) {
        return;
    }
    const uint32_t input = (uint32_t)(element / record.output_size), output = (uint32_t)(element % record.output_size);
    const uint32_t bits_x2 = exl3_bits_x2(record.bits_per_weight);
    const uint32_t ring_bits = EXL3_TILE_VALUES * bits_x2 / 2u, tile_words = ring_bits / 32u;
    const uint64_t tile = (uint64_t)(input / EXL3_TILE) * (record.output_size / EXL3_TILE) + output / EXL3_TILE;
    const uint32_t *words = (const uint32_t *)(arena + record.matrix_offset) + tile * tile_words;
    const uint32_t i = input % EXL3_TILE, o = output % EXL3_TILE;
    const uint32_t position = 8u * (4u * (o % 8u) + (i % 8u) / 2u) + (i & 1u) + 2u * (i / 8u) + 4u * (o / 8u);
    const uint32_t begin = (exl3_window_end(position, bits_x2) + ring_bits - 16u) % ring_bits;
    const uint32_t word = begin / 32u, shift = begin % 32u;
    uint32_t window = words[word] << shift;
    if (shift != 0u) {
        window |= words[(word + 1u) % tile_words] >> (32u - shift);
    }
    ((uint16_t *)(arena + record.output_offset))[element] = exl3_decode_one(window >> 16);
}
ANEMONE_KERNEL(EXL3_KERNEL_FILE, exl3_reconstruct, exl3_reconstruct_record);

/* the stored width of matrix m (0 gate, 1 up, 2 down) of a job's expert */
__device__ static __forceinline__ uint32_t chain_width(const struct exl3_expert_record &record,
                                                       const unsigned char *arena, uint32_t expert, uint32_t matrix)
{
    if (record.widths_offset == 0u) {
        return record.bits_per_weight;
    }
    return exl3_width_of(((const uint32_t *)(arena + record.widths_offset))[expert], matrix);
}

extern "C" __global__ void exl3_input(struct exl3_expert_record record, unsigned char *arena)
{
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + record.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x, projection = blockIdx.z;
    const uint32_t channel = blockIdx.x * EXL3_TRANSFORM + lane;
    const uint64_t matrix = projection == 0u ? job->gate_offset : job->up_offset;
    const uint32_t bits_x2 = exl3_bits_x2(chain_width(record, arena, job->expert, projection));
    const uint16_t *suh = (const uint16_t *)(arena + matrix + exl3_code_bytes(record.input_size, record.inner_size, bits_x2));
    const float s0 = half_bits_to_float(suh[channel]), s1 = half_bits_to_float(suh[channel + WAVE]);
    const uint16_t *input = (const uint16_t *)(arena + record.input_offset);
    uint16_t *operands = (uint16_t *)(arena + record.operands_offset);
    for (uint32_t column = 0; column < job->row_count; column++) {
        const uint32_t pair = job->pair_index[column];
        const uint64_t row = pair / record.pairs_per_row;
        float v0 = __fmul_rn(bf16_to_float(input[row * record.input_size + channel]), s0);
        float v1 = __fmul_rn(bf16_to_float(input[row * record.input_size + channel + WAVE]), s1);
        wave_hadamard128(v0, v1, lane);
        uint16_t *out = operands + ((uint64_t)projection * record.pair_count + pair) * record.input_size;
        out[channel] = float_to_half_bits(__fmul_rn(v0, EXL3_NORMALIZATION));
        out[channel + WAVE] = float_to_half_bits(__fmul_rn(v1, EXL3_NORMALIZATION));
    }
}
ANEMONE_KERNEL(EXL3_KERNEL_FILE, exl3_input, exl3_expert_record);

/* Products of one job: block = four wavefronts = the four K slices of one strip of STRIP_TILES output tiles (eight; one
 * in the thin instances, which a launch of few jobs takes so that its blocks cover the card: the same slices and the
 * same order of sums, so the same bits). */
template <uint32_t bits_x2, bool down, uint32_t STRIP_TILES>
__device__ static __forceinline__ void chain_product(const struct exl3_expert_record &record, unsigned char *arena,
                                                     const struct expert_job_record *job, uint32_t *staging,
                                                     float *partial)
{
    typedef exl3_width<bits_x2> W;
    const uint32_t projection = blockIdx.z;
    const uint32_t inputs = down ? record.inner_size : record.input_size;
    const uint32_t outputs = down ? record.input_size : record.inner_size;
    const uint32_t lane = threadIdx.x % WAVE, slice = threadIdx.x / WAVE;
    const uint64_t matrix = down ? job->down_offset : projection == 0u ? job->gate_offset : job->up_offset;
    const uint32_t column = lane % 16u;
    const half_t *operand = nullptr;
    if (column < job->row_count) {
        operand = (const half_t *)(arena + record.operands_offset) +
                  ((uint64_t)projection * record.pair_count + job->pair_index[column]) * inputs;
    }
    const uint32_t tiles = inputs / EXL3_TILE;
    float4_t accumulator[STRIP_TILES];
    exl3_wave_product<bits_x2, STRIP_TILES>((const uint32_t *)(arena + matrix), outputs / EXL3_TILE,
                                            blockIdx.x * STRIP_TILES, tiles * slice / PRODUCT_WAVES,
                                            tiles * (slice + 1u) / PRODUCT_WAVES, operand,
                                            staging + slice * (2u * STRIP_TILES * W::tile_words), lane, accumulator);
    /* partial [slice][tile][lane] as float4; slice 0 then adds the four in order from +0 */
    float4_t *mine = (float4_t *)partial + (slice * STRIP_TILES) * WAVE + lane;
#pragma unroll
    for (uint32_t n = 0; n < STRIP_TILES; n++) {
        mine[n * WAVE] = accumulator[n];
    }
    __syncthreads();
    if (slice == 0u && column < job->row_count) {
        float *products = (float *)(arena + record.products_offset) +
                          ((uint64_t)projection * record.pair_count + job->pair_index[column]) * outputs;
#pragma unroll
        for (uint32_t n = 0; n < STRIP_TILES; n++) {
            float4_t sum = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (uint32_t part = 0; part < PRODUCT_WAVES; part++) {
                const float4_t value = ((const float4_t *)partial)[(part * STRIP_TILES + n) * WAVE + lane];
                sum.x = __fadd_rn(sum.x, value.x);
                sum.y = __fadd_rn(sum.y, value.y);
                sum.z = __fadd_rn(sum.z, value.z);
                sum.w = __fadd_rn(sum.w, value.w);
            }
            /* lane: outputs 4 (lane / 16) + 0..3 of tile n of the strip */
            *(float4_t *)(products + (blockIdx.x * STRIP_TILES + n) * EXL3_TILE + 4u * (lane / 16u)) = sum;
        }
    }
}

template <uint32_t fixed_bits_x2, bool down, uint32_t STRIP_TILES>
__device__ static __forceinline__ void chain_product_entry(const struct exl3_expert_record &record,
                                                           unsigned char *arena)
{
    __shared__ __attribute__((aligned(16))) uint32_t staging[PRODUCT_WAVES * 2u * STRIP_TILES * exl3_width<8>::tile_words];
    __shared__ __attribute__((aligned(16))) float partial[PRODUCT_WAVES * STRIP_TILES * WAVE * 4u];
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + record.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    uint32_t bits_x2 = fixed_bits_x2;
    if (fixed_bits_x2 == 0u) {
        bits_x2 = exl3_bits_x2(chain_width(record, arena, job->expert, down ? 2u : blockIdx.z));
    }
    switch (bits_x2) {
    case 4u: chain_product<4u, down, STRIP_TILES>(record, arena, job, staging, partial); break;
    case 5u: chain_product<5u, down, STRIP_TILES>(record, arena, job, staging, partial); break;
    case 6u: chain_product<6u, down, STRIP_TILES>(record, arena, job, staging, partial); break;
    case 8u: chain_product<8u, down, STRIP_TILES>(record, arena, job, staging, partial); break;
    default: break;
    }
}

#define EXL3_PRODUCT_ENTRIES(name, bits_x2)                                                                  \
    extern "C" __global__ void __launch_bounds__(PRODUCT_THREADS)                                            \
        exl3_gate_up_##name(struct exl3_expert_record record, unsigned char *arena)                         \
    {                                                                                                        \
        chain_product_entry<bits_x2, false, EXL3_STRIP_TILES>(record, arena);                                \
    }                                                                                                        \
    ANEMONE_KERNEL(EXL3_KERNEL_FILE, exl3_gate_up_##name, exl3_expert_record);                               \
    extern "C" __global__ void __launch_bounds__(PRODUCT_THREADS)                                            \
        exl3_down_##name(struct exl3_expert_record record, unsigned char *arena)                            \
    {                                                                                                        \
        chain_product_entry<bits_x2, true, EXL3_STRIP_TILES>(record, arena);                                 \
    }                                                                                                        \
    ANEMONE_KERNEL(EXL3_KERNEL_FILE, exl3_down_##name, exl3_expert_record);                                  \
    extern "C" __global__ void __launch_bounds__(PRODUCT_THREADS)                                            \
        exl3_gate_up_##name##_thin(struct exl3_expert_record record, unsigned char *arena)                  \
    {                                                                                                        \
        chain_product_entry<bits_x2, false, EXL3_THIN_STRIP_TILES>(record, arena);                           \
    }                                                                                                        \
    ANEMONE_KERNEL(EXL3_KERNEL_FILE, exl3_gate_up_##name##_thin, exl3_expert_record);                        \
    extern "C" __global__ void __launch_bounds__(PRODUCT_THREADS)                                            \
        exl3_down_##name##_thin(struct exl3_expert_record record, unsigned char *arena)                     \
    {                                                                                                        \
        chain_product_entry<bits_x2, true, EXL3_THIN_STRIP_TILES>(record, arena);                            \
    }                                                                                                        \
    ANEMONE_KERNEL(EXL3_KERNEL_FILE, exl3_down_##name##_thin, exl3_expert_record)
EXL3_PRODUCT_ENTRIES(k2, 4u);
EXL3_PRODUCT_ENTRIES(k2_5, 5u);
EXL3_PRODUCT_ENTRIES(k3, 6u);
EXL3_PRODUCT_ENTRIES(k4, 8u);
EXL3_PRODUCT_ENTRIES(mixed, 0u); /* the width of each matrix from the record's widths table */

extern "C" __global__ void exl3_activate(struct exl3_expert_record record, unsigned char *arena)
{
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + record.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x, channel = blockIdx.x * EXL3_TRANSFORM + lane;
    const uint32_t H = record.input_size, I = record.inner_size;
    const uint16_t *gate_svh = (const uint16_t *)(arena + job->gate_offset +
                                                  exl3_code_bytes(H, I, exl3_bits_x2(chain_width(record, arena, job->expert, 0u)))) + H;
    const uint16_t *up_svh = (const uint16_t *)(arena + job->up_offset +
                                                exl3_code_bytes(H, I, exl3_bits_x2(chain_width(record, arena, job->expert, 1u)))) + H;
    const uint16_t *down_suh = (const uint16_t *)(arena + job->down_offset +
                                                  exl3_code_bytes(I, H, exl3_bits_x2(chain_width(record, arena, job->expert, 2u))));
    const float gs0 = half_bits_to_float(gate_svh[channel]), gs1 = half_bits_to_float(gate_svh[channel + WAVE]);
    const float us0 = half_bits_to_float(up_svh[channel]), us1 = half_bits_to_float(up_svh[channel + WAVE]);
    const float ds0 = half_bits_to_float(down_suh[channel]), ds1 = half_bits_to_float(down_suh[channel + WAVE]);
    const float limit = record.activation_limit;
    const float *products = (const float *)(arena + record.products_offset);
    for (uint32_t column = 0; column < job->row_count; column++) {
        const uint32_t pair = job->pair_index[column];
        float g0 = products[(uint64_t)pair * I + channel], g1 = products[(uint64_t)pair * I + channel + WAVE];
        float u0 = products[((uint64_t)record.pair_count + pair) * I + channel];
        float u1 = products[((uint64_t)record.pair_count + pair) * I + channel + WAVE];
        wave_hadamard128(g0, g1, lane);
        wave_hadamard128(u0, u1, lane);
        float hidden[2];
        const float gate[2] = {__fmul_rn(__fmul_rn(g0, EXL3_NORMALIZATION), gs0), __fmul_rn(__fmul_rn(g1, EXL3_NORMALIZATION), gs1)};
        const float up[2] = {__fmul_rn(__fmul_rn(u0, EXL3_NORMALIZATION), us0), __fmul_rn(__fmul_rn(u1, EXL3_NORMALIZATION), us1)};
#pragma unroll
        for (uint32_t i = 0; i < 2u; i++) {
            const float bounded_gate = fminf(gate[i], limit);
            const float bounded_up = fminf(fmaxf(up[i], -limit), limit);
            hidden[i] = __fmul_rn(det_silu(bounded_gate), bounded_up);
        }
        uint16_t *hidden_out = (uint16_t *)(arena + record.hidden_offset) + (uint64_t)pair * I;
        hidden_out[channel] = float_to_bf16(hidden[0]);
        hidden_out[channel + WAVE] = float_to_bf16(hidden[1]);
        float v0 = __fmul_rn(hidden[0], ds0), v1 = __fmul_rn(hidden[1], ds1);
        wave_hadamard128(v0, v1, lane);
        uint16_t *operand = (uint16_t *)(arena + record.operands_offset) + (uint64_t)pair * I;
        operand[channel] = float_to_half_bits(__fmul_rn(v0, EXL3_NORMALIZATION));
        operand[channel + WAVE] = float_to_half_bits(__fmul_rn(v1, EXL3_NORMALIZATION));
    }
}
ANEMONE_KERNEL(EXL3_KERNEL_FILE, exl3_activate, exl3_expert_record);

extern "C" __global__ void exl3_finish(struct exl3_expert_record record, unsigned char *arena)
{
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + record.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x, channel = blockIdx.x * EXL3_TRANSFORM + lane;
    const uint32_t H = record.input_size, I = record.inner_size;
    const uint16_t *svh = (const uint16_t *)(arena + job->down_offset +
                                             exl3_code_bytes(I, H, exl3_bits_x2(chain_width(record, arena, job->expert, 2u)))) + I;
    const float s0 = half_bits_to_float(svh[channel]), s1 = half_bits_to_float(svh[channel + WAVE]);
    for (uint32_t column = 0; column < job->row_count; column++) {
        const uint32_t pair = job->pair_index[column];
        float *values = (float *)(arena + record.products_offset) + (uint64_t)pair * H;
        float v0 = values[channel], v1 = values[channel + WAVE];
        wave_hadamard128(v0, v1, lane);
        const float weight = job->route_weight[column];
        float *out = (float *)(arena + record.output_offset) + (uint64_t)pair * H;
        out[channel] = __fmul_rn(__fmul_rn(__fmul_rn(v0, EXL3_NORMALIZATION), s0), weight);
        out[channel + WAVE] = __fmul_rn(__fmul_rn(__fmul_rn(v1, EXL3_NORMALIZATION), s1), weight);
    }
}
ANEMONE_KERNEL(EXL3_KERNEL_FILE, exl3_finish, exl3_expert_record);

extern "C" __global__ void exl3_row_sum(struct expert_row_sum_arguments record, unsigned char *arena)
{
    const uint32_t channel = blockIdx.x * blockDim.x + threadIdx.x;
    if (channel >= record.width) {
        return;
    }
    const uint64_t row = blockIdx.y;
    const float *pairs = (const float *)(arena + record.pair_output_offset);
    float sum = 0.0f;
    for (uint32_t slot = 0; slot < record.pairs_per_row; slot++) {
        sum = __fadd_rn(sum, pairs[(row * record.pairs_per_row + slot) * record.width + channel]);
    }
    ((float *)(arena + record.row_output_offset))[row * record.width + channel] = sum;
}
ANEMONE_KERNEL(EXL3_KERNEL_FILE, exl3_row_sum, expert_row_sum_arguments);
