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
 * matrix. The 1,024 bytes of a tile's two consecutive loads are one 16-byte-per-lane load from memory straight into
 * a wavefront-private LDS window, whence they reach the MFMA's lanes: lane (o, g) needs output row o of inputs block g,
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
#define DEPTH 8u                 /* K steps in flight a wavefront */
#define STAGE_WORDS (STEP_BYTES / 4u)
#define WINDOW_WORDS (DEPTH * STAGE_WORDS) /* a wavefront's LDS window: DEPTH stages of one step's weights */
#define STAGE_LOADS 7u           /* memory loads a stage issues: scale, four vector pieces, vector scale, weights */
#define NIBBLE_MASK 0x0F0F0F0Fu

typedef const __attribute__((address_space(1))) void *global_pointer;
typedef __attribute__((address_space(3))) void *lds_pointer;

/* 16 bytes a lane from memory straight into LDS: lane L's bytes land at `stage` + 16 L (the base travels in M0).
 * Written as assembly so that the compiler keeps no book on it: it would otherwise guard every LDS read that might
 * alias with a wait for all loads. The waits are this file's own (wait_loads). A fence for the compiler as well, so
 * the stages' loads keep their order, which the waits count on. */
__device__ static __forceinline__ void load_to_lds(const unsigned char *source, uint32_t *stage)
{
    const uint32_t base = (uint32_t)(uintptr_t)(lds_pointer)stage;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(source), "s"(base)
                 : "memory", "m0");
}

/* wait until at most `count` of the wavefront's memory loads are outstanding (they retire in order); also a fence
 * for the compiler: LDS reads of a stage stay behind the wait for the load that fills it */
template <uint32_t count>
__device__ static __forceinline__ void wait_loads()
{
    static_assert(count < 64u, "vmcnt has six bits");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(count) : "memory");
}

/* What a lane keeps through a chain: where its loads start and where it reads its operands in a stage. */
struct chain_lane {
    const unsigned char *words;        /* this lane's 16-byte piece of the chain's first step */
    const unsigned char *scales;       /* its weight scale byte of the first step */
    const unsigned char *vector;       /* its 8-byte pieces of the vector's codes, first step */
    const unsigned char *vector_scale; /* its vector scale byte, first step */
    uint32_t *lds;                     /* the wavefront's window */
    uint32_t read_at[4];               /* word offsets of its pieces T = 0..3 inside a stage */
    uint32_t shift;                    /* 0: the even nibbles (outputs 0..7 of the tile), 4: the odd ones */
};

struct chain_stage { /* what a stage keeps in registers while its weights are on their way into LDS */
    uint2_t vector[4];
    uint32_t scale, vector_scale;
};

__device__ static __forceinline__ void stage_issue(const chain_lane &lane, uint32_t stage, uint32_t at, chain_stage &kept)
{
    kept.scale = lane.scales[(uint64_t)at * 64u];
#pragma unroll
    for (uint32_t part = 0; part < 4u; part++) {
        kept.vector[part] = *(const uint2_t *)(lane.vector + (uint64_t)at * 128u + 64u * (part / 2u) + 16u * (part % 2u));
    }
    kept.vector_scale = lane.vector_scale[(uint64_t)at * 4u];
    load_to_lds(lane.words + (uint64_t)at * STEP_BYTES, lane.lds + stage * STAGE_WORDS); /* the last of STAGE_LOADS */
}

__device__ static __forceinline__ float4_t stage_consume(const chain_lane &lane, uint32_t stage, chain_stage kept, float4_t chain)
{
    /* the stage's registers are first touched here, behind the wait: their uses may not drift to where an earlier
     * wait would have to cover them */
    asm volatile("" : "+v"(kept.scale), "+v"(kept.vector_scale));
    int8_vector b;
#pragma unroll
    for (uint32_t part = 0; part < 4u; part++) {
        uint2_t pair = kept.vector[part];
        asm volatile("" : "+v"(pair.x), "+v"(pair.y));
        b[2u * part] = (int)__builtin_amdgcn_perm(pair.y, pair.x, 0x05010400u);
        b[2u * part + 1u] = (int)__builtin_amdgcn_perm(pair.y, pair.x, 0x07030602u);
    }
    int8_vector a = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (uint32_t T = 0; T < 4u; T++) {
        const uint2_t w = *(const uint2_t *)(lane.lds + stage * STAGE_WORDS + lane.read_at[T]);
        a[T] = (int)(((w.x >> lane.shift) & NIBBLE_MASK) | (((w.y >> lane.shift) & NIBBLE_MASK) << 4));
    }
    /* the stage is read once its values are in registers; only then may it be filled again */
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, chain, 4, 0, 0, (int)kept.scale, 0, (int)kept.vector_scale);
}

/* N steps from `at` on, N known to the compiler (at most 2 DEPTH): straight-line code, so that every wait is a
 * constant: before step s, the stages asked for behind it number min(N, s + DEPTH) - 1 - s. The window must be idle
 * on entry (nothing of this wavefront on its way), and is idle again on return. */
template <uint32_t N>
__device__ static __forceinline__ float4_t chain_run(const chain_lane &lane, uint32_t at, float4_t chain)
{
    static_assert(N >= 1u && N <= 2u * DEPTH, "one or two rounds of the window");
    chain_stage kept[DEPTH];
#pragma unroll
    for (uint32_t s = 0; s < (N < DEPTH ? N : DEPTH); s++) {
        stage_issue(lane, s, at + s, kept[s]);
    }
#pragma unroll
    for (uint32_t s = 0; s < N; s++) {
        constexpr uint32_t none = 0;
        const uint32_t asked = (s + DEPTH < N ? s + DEPTH : N) - 1u - s; /* folds: s is an unrolled constant */
        switch (asked) {
        case 7: wait_loads<STAGE_LOADS * 7u>(); break;
        case 6: wait_loads<STAGE_LOADS * 6u>(); break;
        case 5: wait_loads<STAGE_LOADS * 5u>(); break;
        case 4: wait_loads<STAGE_LOADS * 4u>(); break;
        case 3: wait_loads<STAGE_LOADS * 3u>(); break;
        case 2: wait_loads<STAGE_LOADS * 2u>(); break;
        case 1: wait_loads<STAGE_LOADS * 1u>(); break;
        default: wait_loads<none>(); break;
        }
        chain = stage_consume(lane, s % DEPTH, kept[s % DEPTH], chain);
        if (s + DEPTH < N) {
            stage_issue(lane, s % DEPTH, at + s + DEPTH, kept[s % DEPTH]);
        }
    }
    return chain;
}

/* One wavefront: the chain of K steps [first, last) of one tile of one matrix against up to 16 vector columns.
 *
 * The 1,024 bytes of a step go from memory straight into a stage of the wavefront's LDS window (no registers in
 * between), up to DEPTH stages ahead, so that a wavefront keeps DEPTH KB on their way. Lane L of the load lands at
 * bytes 16 L of the stage, and asks for the 16-byte piece p = L ^ (2 bit4(L) + bit5(L)) of the step: the pieces of
 * one T (p = 32 ld + 4 G + T) then lie in different LDS banks for the readers, and every 16 lanes still read 256
 * contiguous bytes of memory. The vector's codes and both scale codes of a stage are asked for together with its
 * weights and wait in registers: loads retire in order, so anything asked for later than the weights of a far stage
 * would have to wait for them. Columns without a row read the vector of row 0; their sums are never stored. */
__device__ static __forceinline__ float4_t
expert_chain(const unsigned char *matrix, uint32_t outputs, uint32_t inputs, uint32_t tile, uint32_t first,
             uint32_t last, const unsigned char *codes, const unsigned char *exponents, uint32_t *lds, uint32_t lane_index)
{
    static_assert(DEPTH == 8u, "the waits of chain_run are written out for eight stages");
    const uint32_t loads = inputs / 64u;
    const uint32_t o = lane_index % 16u, g = lane_index / 16u, G = o % 8u, parity = o / 8u, ld = g / 2u, q = g % 2u;
    const uint32_t piece = lane_index ^ (2u * ((lane_index >> 4) & 1u) + ((lane_index >> 5) & 1u));
    chain_lane lane;
    lane.words = matrix + ((uint64_t)tile * loads + 2u * first) * TILE_LOAD_BYTES + piece * 16u;
    /* scales: uint32 [tile][load][G], byte 2 q + parity */
    lane.scales = matrix + (uint64_t)outputs * inputs / 2u + (((uint64_t)tile * loads + 2u * first + ld) * 8u + G) * 4u + 2u * q + parity;
    /* the vector: bytes 64 load + 16 T + 8 q .. + 7 for T = 2 (g % 2), 2 (g % 2) + 1 of both loads of the step */
    lane.vector = codes + 128u * first + 32u * (g % 2u) + 8u * (g / 2u);
    lane.vector_scale = exponents + 4u * first + g;
    lane.lds = lds;
    /* where this lane reads its piece T of a stage: slot 32 ld + 4 G + (T ^ (2 (G / 4) + ld)), half q */
#pragma unroll
    for (uint32_t T = 0; T < 4u; T++) {
        lane.read_at[T] = (16u * (32u * ld + 4u * G + (T ^ (2u * (G / 4u) + ld))) + 8u * q) / 4u;
    }
    lane.shift = 4u * parity;
    const uint32_t total = last - first; /* the same in every lane */
    float4_t chain = {0.0f, 0.0f, 0.0f, 0.0f};
    uint32_t at = 0;
    for (; at + 2u * DEPTH <= total; at += 2u * DEPTH) {
        chain = chain_run<2u * DEPTH>(lane, at, chain);
    }
    switch (total - at) {
#define CHAIN_REST(n)                                                                                               \
    case n: chain = chain_run<n>(lane, at, chain); break
        CHAIN_REST(1); CHAIN_REST(2); CHAIN_REST(3); CHAIN_REST(4); CHAIN_REST(5); CHAIN_REST(6); CHAIN_REST(7); CHAIN_REST(8);
        CHAIN_REST(9); CHAIN_REST(10); CHAIN_REST(11); CHAIN_REST(12); CHAIN_REST(13); CHAIN_REST(14); CHAIN_REST(15);
#undef CHAIN_REST
    default: break;
    }
    return chain;
}

/* gate and up: block = 2 S wavefronts (matrix = wave / S, slice = wave % S); grid (output_size / 16, jobs) */
template <uint32_t S>
__device__ static __forceinline__ void expert_gate_up(const struct expert_gate_up_arguments &arguments,
                                                      unsigned char *arena)
{
    __shared__ __attribute__((aligned(16))) uint32_t window[2u * S][WINDOW_WORDS];
    __shared__ __attribute__((aligned(16))) float partial[2u * S][WAVE * 4u];
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + arguments.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t matrix = wave / S, slice = wave % S;
    const uint32_t column = lane % 16u;
    const bool live = column < job->row_count;
    const uint32_t pair = live ? job->pair_index[column] : 0u;
    const uint64_t row = pair / arguments.pairs_per_row;
    const uint32_t steps = arguments.input_size / 128u;
    const float4_t chain = expert_chain(arena + (matrix == 0u ? job->gate_offset : job->up_offset), arguments.output_size,
                                        arguments.input_size, blockIdx.x, steps * slice / S, steps * (slice + 1u) / S,
                                        arena + arguments.codes_offset + row * arguments.input_size,
                                        arena + arguments.exponents_offset + row * (arguments.input_size / 32u),
                                        window[wave], lane);
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
    __shared__ __attribute__((aligned(16))) uint32_t window[S][WINDOW_WORDS];
    __shared__ __attribute__((aligned(16))) float partial[S][WAVE * 4u];
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + arguments.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x % WAVE, slice = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), column = lane % 16u;
    const bool live = column < job->row_count;
    const uint64_t pair = live ? job->pair_index[column] : 0u;
    const uint32_t steps = arguments.input_size / 128u;
    const float4_t chain = expert_chain(arena + job->down_offset, arguments.output_size, arguments.input_size, blockIdx.x,
                                        steps * slice / S, steps * (slice + 1u) / S,
                                        arena + arguments.codes_offset + pair * arguments.input_size,
                                        arena + arguments.exponents_offset + pair * (arguments.input_size / 32u),
                                        window[slice], lane);
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
    extern "C" __global__ void __launch_bounds__(2u * S * WAVE) __attribute__((amdgpu_waves_per_eu(4)))           \
        expert_gate_up_##S(struct expert_gate_up_arguments arguments, unsigned char *arena)                      \
    {                                                                                                             \
        expert_gate_up<S>(arguments, arena);                                                                      \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_##S, expert_gate_up_arguments);                      \
    extern "C" __global__ void __launch_bounds__(S * WAVE) __attribute__((amdgpu_waves_per_eu(4)))                \
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
