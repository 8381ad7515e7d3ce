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
 * Work mapping (this build's own). A block is one tile of 16 outputs of one job; a wavefront is one slice of one
 * matrix. The 1,024 bytes of a tile's two consecutive loads are one coalesced 16-byte-per-lane read; they pass
 * through a wavefront-private LDS window to reach the MFMA's lanes: lane (o, g) needs output row o of inputs block g,
 * which the stored form spreads over four stored lanes (t = 0..3) as the even (o < 8) or odd (o >= 8) nibbles of two
 * words each. Compaction of eight nibbles into a register is two shifts, two ands and an or. The vector's codes are
 * brought into the same input order with two byte permutes a register.
 *
 * MFMA operand layout on gfx950, as measured on the card: A (fp4) lane l: row l % 16, element e = 8 v + n (register v,
 * nibble n) is k = 32 (l / 16) + e; B (fp8) lane l: column l % 16, element e = 4 v + b is k = 64 (e / 16) +
 * 16 (l / 16) + e % 16; scale of lane l: row or column l % 16, inputs block l / 16; D lane l: column l % 16, rows
 * 4 (l / 16) + v.
 */
#include "exl3_device.cuh" /* det_expf, bf16 helpers, vector types */
#include "kernel_registry.h"

typedef int int8_vector __attribute__((ext_vector_type(8)));

#define TILE_LOAD_BYTES 512u     /* 16 outputs x 64 inputs x 4 bits */
#define STEP_BYTES (2u * TILE_LOAD_BYTES)
#define PREFETCH 4u              /* K steps in flight a wavefront */
#define NIBBLE_MASK 0x0F0F0F0Fu

/* One wavefront: the chain of K steps [first, last) of one tile of one matrix against up to 16 vector columns. */
__device__ static __forceinline__ float4_t
expert_chain(const unsigned char *matrix, uint32_t outputs, uint32_t inputs, uint32_t tile, uint32_t first,
             uint32_t last, const unsigned char *codes, const unsigned char *exponents, bool live, uint32_t *lds,
             uint32_t lane)
{
    const uint32_t loads = inputs / 64u;
    const uint32_t o = lane % 16u, g = lane / 16u, G = o % 8u, parity = o / 8u, ld = g / 2u, q = g % 2u;
    const unsigned char *words = matrix + ((uint64_t)tile * loads + 2u * first) * TILE_LOAD_BYTES + lane * 16u;
    /* scales: uint32 [tile][load][G], byte 2 q + parity */
    const unsigned char *scales = matrix + (uint64_t)outputs * inputs / 2u +
                                  (((uint64_t)tile * loads + 2u * first + ld) * 8u + G) * 4u + 2u * q + parity;
    /* the vector: bytes 64 load + 16 T + 8 q .. + 7 for T = 2 (g % 2), 2 (g % 2) + 1 of both loads of the step */
    const unsigned char *vector = codes + 128u * first + 32u * (g % 2u) + 8u * (g / 2u);
    const unsigned char *vector_scale = exponents + 4u * first + g;
    uint4_t ring[PREFETCH];
    uint32_t scale_ring[PREFETCH];
#pragma unroll
    for (uint32_t i = 0; i < PREFETCH; i++) {
        if (first + i < last) {
            ring[i] = *(const uint4_t *)(words + (uint64_t)i * STEP_BYTES);
            scale_ring[i] = scales[(uint64_t)i * 64u];
        }
    }
    float4_t chain = {0.0f, 0.0f, 0.0f, 0.0f};
    const uint32_t read_at = (512u * ld + 64u * G + 8u * q) / 4u; /* + 4 T words */
    const uint32_t shift = 4u * parity;
    for (uint32_t step = first; step < last; step += PREFETCH) {
#pragma unroll
        for (uint32_t i = 0; i < PREFETCH; i++) {
            if (step + i < last) { /* uniform over the wavefront */
                const uint4_t mine = ring[i];
                const uint32_t scale_a = scale_ring[i];
                if (step + i + PREFETCH < last) {
                    ring[i] = *(const uint4_t *)(words + (uint64_t)(step - first + i + PREFETCH) * STEP_BYTES);
                    scale_ring[i] = scales[(uint64_t)(step - first + i + PREFETCH) * 64u];
                }
                int8_vector b = {0, 0, 0, 0, 0, 0, 0, 0};
                uint32_t scale_b = 127u;
                if (live) {
                    const unsigned char *x = vector + (uint64_t)(step - first + i) * 128u;
#pragma unroll
                    for (uint32_t load = 0; load < 2u; load++) {
#pragma unroll
                        for (uint32_t half = 0; half < 2u; half++) {
                            const uint2_t pair = *(const uint2_t *)(x + 64u * load + 16u * half);
                            b[4u * load + 2u * half] = (int)__builtin_amdgcn_perm(pair.y, pair.x, 0x05010400u);
                            b[4u * load + 2u * half + 1u] = (int)__builtin_amdgcn_perm(pair.y, pair.x, 0x07030602u);
                        }
                    }
                    scale_b = vector_scale[(uint64_t)(step - first + i) * 4u];
                }
                *(uint4_t *)(lds + lane * 4u) = mine;
                __builtin_amdgcn_s_waitcnt(0xc07f);
                __builtin_amdgcn_wave_barrier();
                int8_vector a = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (uint32_t T = 0; T < 4u; T++) {
                    const uint2_t w = *(const uint2_t *)(lds + read_at + 4u * T);
                    a[T] = (int)(((w.x >> shift) & NIBBLE_MASK) | (((w.y >> shift) & NIBBLE_MASK) << 4));
                }
                __builtin_amdgcn_wave_barrier();
                chain = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, chain, 4, 0, 0, (int)scale_a, 0, (int)scale_b);
            }
        }
    }
    return chain;
}

/* gate and up: block = 2 S wavefronts (matrix = wave / S, slice = wave % S); grid (output_size / 16, jobs) */
template <uint32_t S>
__device__ static __forceinline__ void expert_gate_up(const struct expert_gate_up_arguments &arguments,
                                                      unsigned char *arena)
{
    __shared__ __attribute__((aligned(16))) uint32_t exchange[2u * S][256];
    __shared__ __attribute__((aligned(16))) float partial[2u * S][WAVE * 4u];
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + arguments.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, matrix = wave / S, slice = wave % S;
    const uint32_t column = lane % 16u;
    const bool live = column < job->row_count;
    const uint32_t pair = live ? job->pair_index[column] : 0u;
    const uint64_t row = pair / arguments.pairs_per_row;
    const uint32_t steps = arguments.input_size / 128u;
    const float4_t chain = expert_chain(arena + (matrix == 0u ? job->gate_offset : job->up_offset), arguments.output_size,
                                        arguments.input_size, blockIdx.x, steps * slice / S, steps * (slice + 1u) / S,
                                        arena + arguments.codes_offset + row * arguments.input_size,
                                        arena + arguments.exponents_offset + row * (arguments.input_size / 32u), live,
                                        exchange[wave], lane);
    *(float4_t *)&partial[wave][lane * 4u] = chain;
    __syncthreads();
    if (wave == 0u && live) {
        float gate[4] = {0.0f, 0.0f, 0.0f, 0.0f}, up[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (uint32_t part = 0; part < S; part++) { /* the S chains from +0, in order */
#pragma unroll
            for (uint32_t v = 0; v < 4u; v++) {
                gate[v] = __fadd_rn(gate[v], partial[part][lane * 4u + v]);
                up[v] = __fadd_rn(up[v], partial[S + part][lane * 4u + v]);
            }
        }
        const float limit = arguments.activation_limit, weight = job->route_weight[column];
        uint16_t hidden[4];
#pragma unroll
        for (uint32_t v = 0; v < 4u; v++) {
            const float g = bf16_to_float(float_to_bf16(gate[v])), u = bf16_to_float(float_to_bf16(up[v]));
            const float bounded_gate = fminf(g, limit);
            const float bounded_up = fminf(fmaxf(u, -limit), limit);
            const float value = __fmul_rn(__fmul_rn(__fdiv_rn(bounded_gate, __fadd_rn(1.0f, det_expf(-bounded_gate))), bounded_up), weight);
            hidden[v] = float_to_bf16(value);
        }
        uint16_t *out = (uint16_t *)(arena + arguments.hidden_offset) + (uint64_t)pair * arguments.output_size +
                        blockIdx.x * 16u + 4u * (lane / 16u);
        *(uint2_t *)out = (uint2_t){(uint32_t)hidden[0] | ((uint32_t)hidden[1] << 16), (uint32_t)hidden[2] | ((uint32_t)hidden[3] << 16)};
    }
}

/* down: block = S wavefronts; grid (output_size / 16, jobs) */
template <uint32_t S>
__device__ static __forceinline__ void expert_down(const struct expert_down_arguments &arguments, unsigned char *arena)
{
    __shared__ __attribute__((aligned(16))) uint32_t exchange[S][256];
    __shared__ __attribute__((aligned(16))) float partial[S][WAVE * 4u];
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + arguments.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x % WAVE, slice = threadIdx.x / WAVE, column = lane % 16u;
    const bool live = column < job->row_count;
    const uint64_t pair = live ? job->pair_index[column] : 0u;
    const uint32_t steps = arguments.input_size / 128u;
    const float4_t chain = expert_chain(arena + job->down_offset, arguments.output_size, arguments.input_size, blockIdx.x,
                                        steps * slice / S, steps * (slice + 1u) / S,
                                        arena + arguments.codes_offset + pair * arguments.input_size,
                                        arena + arguments.exponents_offset + pair * (arguments.input_size / 32u), live,
                                        exchange[slice], lane);
    *(float4_t *)&partial[slice][lane * 4u] = chain;
    __syncthreads();
    if (slice == 0u && live) {
        float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (uint32_t part = 0; part < S; part++) {
#pragma unroll
            for (uint32_t v = 0; v < 4u; v++) {
                sum[v] = __fadd_rn(sum[v], partial[part][lane * 4u + v]);
            }
        }
        uint16_t *out = (uint16_t *)(arena + arguments.output_offset) + pair * arguments.output_size + blockIdx.x * 16u + 4u * (lane / 16u);
        *(uint2_t *)out = (uint2_t){(uint32_t)float_to_bf16(sum[0]) | ((uint32_t)float_to_bf16(sum[1]) << 16),
                                    (uint32_t)float_to_bf16(sum[2]) | ((uint32_t)float_to_bf16(sum[3]) << 16)};
    }
}

#define EXPERT_ENTRIES(S)                                                                                         \
    extern "C" __global__ void __launch_bounds__(2u * S * WAVE)                                                   \
        expert_gate_up_##S(struct expert_gate_up_arguments arguments, unsigned char *arena)                      \
    {                                                                                                             \
        expert_gate_up<S>(arguments, arena);                                                                      \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_##S, expert_gate_up_arguments);                      \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_down_##S(struct expert_down_arguments arguments, unsigned char *arena)                            \
    {                                                                                                             \
        expert_down<S>(arguments, arena);                                                                         \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_down_##S, expert_down_arguments)
EXPERT_ENTRIES(1);
EXPERT_ENTRIES(2);
EXPERT_ENTRIES(4);
EXPERT_ENTRIES(8);

/* float32 sum of a row's bfloat16 pair outputs from +0 in ascending slot order; grid (ceil(width / 256), rows) */
extern "C" __global__ void expert_row_sum_entry(struct expert_row_sum_arguments arguments, unsigned char *arena)
{
    const uint32_t channel = blockIdx.x * blockDim.x + threadIdx.x;
    if (channel >= arguments.width) {
        return;
    }
    const uint64_t row = blockIdx.y;
    const uint16_t *pairs = (const uint16_t *)(arena + arguments.pair_output_offset);
    float sum = 0.0f;
    for (uint32_t slot = 0; slot < arguments.pairs_per_row; slot++) {
        sum = __fadd_rn(sum, bf16_to_float(pairs[(row * arguments.pairs_per_row + slot) * arguments.width + channel]));
    }
    ((float *)(arena + arguments.row_output_offset))[row * arguments.width + channel] = sum;
}
ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_row_sum_entry, expert_row_sum_arguments);
