/*
 * kernel_site_front.hip -- the fused fronts of a block's sites on gfx950: site_front_<R> (a site's mix project, its mix
 * finish and the quantization of the sublayer's input in one launch) and ffn_front_<R> (the same with the router's scores
 * and its select between the finish and the quantization); input_front_<R> and then coefficient_front_<R>, the site front
 * in two launches (the first stores hidden, codes, exponents and operands; the second the mixes, post, comb and the site's
 * pre, and may run beside later launches up to the site's post). Entry names, record and what is written follow the reference
 * (include/anemone/site_front_records.h:10-37, source/kernel_site_front.cu): every output has the bits of the launches
 * the front stands for, because it runs their code (dense_device.cuh, hyper_device.cuh, router_device.cuh,
 * quantize_device.cuh) on the same operands in the same order.
 *
 * Work mapping (this build's own). Two chains run side by side: streams and carried pre -> a row's input -> its
 * quantization, the router's scores, the select; and streams -> mixes -> post, comb and the site's pre. Blocks of
 * width / 8 threads (a row's block of the mix finish; a quarter of 256 threads of it is the dense product's block) take
 * a ticket each and their part by it:
 *     tickets 0 .. rows - 1           a row: its input, its quantization; publishes rows_ready
 *     then site_front_mix_blocks      SITE_FRONT_MIX_OUTPUTS mixes a quarter, every row; publishes arrived; the last to
 *                                     arrive waits for rows_ready = rows (the rows' blocks have read the pre) and forms
 *                                     every row's post, comb and pre, sixteen threads a row
 *     then site_front_score_blocks    (FFN front) waits for rows_ready = rows; SITE_FRONT_SCORE_OUTPUTS experts a quarter,
 *                                     every row; publishes scored; the last to arrive runs the select
 * A wait is thread 0 polling the counter (agent scope) with a sleep between polls, at most SITE_FRONT_WAIT_POLLS times;
 * a block whose wait runs out counts itself in gave_up, skips its part and leaves: every wave of the grid ends. The
 * last block to leave (departed) clears the counters.
 *
 * The two halves need no tickets and no waits: the input front is a row a block (grid rows); the coefficient front is the
 * mix project's blocks (grid site_front_mix_blocks), the last of which to publish arrived forms post, comb and pre and
 * clears that counter. The stream orders them: the coefficient front writes the pre that the input front read.
 */
#include "kernel_registry.h"
#include "dense_device.cuh"
#include "hyper_device.cuh"
#include "quantize_device.cuh"
#include "router_device.cuh"

#define FRONT_MOST_THREADS (SITE_FRONT_MOST_WIDTH / HYPER_VALUES_PER_THREAD) /* 640: three wavefronts a SIMD at most, 168 registers each */
#define FRONT_MOST_QUARTERS (FRONT_MOST_THREADS / DENSE_THREADS_VALUE)

__device__ static __forceinline__ uint32_t front_add(uint32_t *counter)
{
    return __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* Every thread of the block calls; the old value of the counter, on every thread. RELEASE: what the block's threads stored
 * is visible at agent scope before the counter moves (every thread's stores are through to the block's level 2 cache
 * before the block meets; thread 0 then writes that cache's lines back once for all). ACQUIRE: what the earlier
 * publishers stored is visible to the block's threads behind the call (thread 0 drops the stale lines once for all). */
template <bool RELEASE, bool ACQUIRE>
__device__ static __forceinline__ uint32_t front_publish(uint32_t *counter, uint32_t thread, uint32_t *word)
{
    if (RELEASE) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    }
    __syncthreads();
    if (thread == 0u) {
        if (RELEASE) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        }
        *word = front_add(counter);
        if (ACQUIRE) {
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        }
    }
    __syncthreads();
    if (ACQUIRE) {
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    }
    return *word;
}

/* every thread of the block calls; whether the counter reached `target`. ACQUIRE as above. */
template <bool ACQUIRE>
__device__ static __forceinline__ bool front_wait(uint32_t *counter, uint32_t target, uint32_t thread, uint32_t *word, uint32_t *gave_up)
{
    __syncthreads(); /* the word's readers are through */
    if (thread == 0u) {
        uint32_t polls = 0;
        while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target && polls < SITE_FRONT_WAIT_POLLS) {
            __builtin_amdgcn_s_sleep(2);
            polls++;
        }
        const bool reached = polls < SITE_FRONT_WAIT_POLLS;
        if (!reached) {
            front_add(gave_up);
        }
        if (ACQUIRE) {
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        }
        *word = reached ? 1u : 0u;
    }
    __syncthreads();
    if (ACQUIRE) {
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    }
    return *word != 0u;
}

/* a row's block: the row's input, then its quantization, a thread four values at a time */
__device__ static __forceinline__ void front_row(const struct site_front_arguments &arguments, const struct hyper_finish_arguments &finish,
                                                 unsigned char *arena, uint32_t row, uint32_t thread, uint32_t threads, float *group_sums)
{
    const uint32_t width = threads * HYPER_VALUES_PER_THREAD;
    hyper_row_input_body(finish, arena, row, thread, threads, group_sums);
    __syncthreads(); /* the row is written: this block's threads read it */
    const struct activation_quantize_arguments quantize = {arguments.hidden_offset, arguments.codes_offset, arguments.exponents_offset,
                                                           arguments.operands_offset, width};
    for (uint32_t q = thread; q < width / 4u; q += threads) {
        activation_quantize_body(quantize, arena, q, row);
    }
}

/* block `block` of the mix project's: float32 [24][4 width] by the streams as rows of 4 width values, with the row's scale,
 * SITE_FRONT_MIX_OUTPUTS mixes a quarter of 256 threads, into the scratch's mixes */
template <uint32_t ROWS>
__device__ static __forceinline__ void front_mix_project(const struct site_front_arguments &arguments, unsigned char *arena, uint32_t rows,
                                                         uint32_t block, uint32_t thread, uint32_t threads,
                                                         dense_group_sums<ROWS, SITE_FRONT_MIX_OUTPUTS> *sums)
{
    const uint32_t quarter = thread / DENSE_THREADS_VALUE, quarters = threads / DENSE_THREADS_VALUE;
    const bool in_quarter = quarter < quarters;
    struct dense_linear_arguments dense = {};
    dense.weights_offset = arguments.mix_weights_offset;
    dense.rows_offset = arguments.streams_offset;
    dense.output_offset = arguments.scratch_offset + offsetof(struct site_front_scratch, mixes);
    dense.output_size = MODEL_MIXES;
    dense.input_size = MODEL_STREAMS * threads * HYPER_VALUES_PER_THREAD;
    dense.row_count = rows;
    dense.output_type = DENSE_FLOAT32;
    dense.flags = DENSE_ROW_SCALE;
    dense.output_scale = 1.0f;
    dense.epsilon = MODEL_NORM_EPSILON;
    constexpr uint32_t groups = MODEL_MIXES / SITE_FRONT_MIX_OUTPUTS;
    const uint32_t group = block * quarters + quarter;
    dense_linear_body<DENSE_FLOAT32, ROWS, SITE_FRONT_MIX_OUTPUTS>(dense, arena, (const uint16_t *)(arena + dense.rows_offset),
                                                                   group * SITE_FRONT_MIX_OUTPUTS, 0u, thread % DENSE_THREADS_VALUE,
                                                                   in_quarter && group < groups, sums[in_quarter ? quarter : 0u]);
}

template <uint32_t ROWS, bool FFN>
__device__ static __forceinline__ void site_front(const struct site_front_arguments &arguments, unsigned char *arena)
{
    __shared__ union {
        dense_group_sums<ROWS, SITE_FRONT_MIX_OUTPUTS> mixes[FRONT_MOST_QUARTERS];
        dense_group_sums<ROWS, SITE_FRONT_SCORE_OUTPUTS> scores[FRONT_MOST_QUARTERS];
        float group_sums[32];
        struct router_select_lds select;
    } lds;
    __shared__ uint32_t word;
    const uint32_t thread = threadIdx.x, threads = blockDim.x, width = threads * HYPER_VALUES_PER_THREAD;
    const uint32_t rows = arguments.select.row_count;
    const uint32_t quarter = thread / DENSE_THREADS_VALUE, quarters = threads / DENSE_THREADS_VALUE, quarter_thread = thread % DENSE_THREADS_VALUE;
    const bool in_quarter = quarter < quarters; /* a width that is no multiple of 2,048 leaves the last threads out of the dense products */
    const uint32_t slot = in_quarter ? quarter : 0u;
    struct site_front_scratch *scratch = (struct site_front_scratch *)(arena + arguments.scratch_offset);
    const uint64_t mixes_offset = arguments.scratch_offset + offsetof(struct site_front_scratch, mixes);
    const uint32_t shape = arguments.select.reference_order_and_shape;
    const uint32_t expert_bits = (shape >> 1) & 1023u, experts = expert_bits != 0u ? expert_bits : ROUTER_DEFAULT_EXPERTS;
    const uint32_t mix_blocks = site_front_mix_blocks(width), score_blocks = FFN ? site_front_score_blocks(width, experts) : 0u;
    if (gridDim.x != rows + mix_blocks + score_blocks) {
        return; /* not the grid of this record: no block takes a ticket */
    }
    if (thread == 0u) {
        word = front_add(&scratch->tickets);
    }
    __syncthreads();
    const uint32_t ticket = word;
    const struct hyper_finish_arguments finish = {arguments.streams_offset, arguments.pre_offset, mixes_offset, arguments.scale_offset,
                                                  arguments.base_offset, arguments.post_offset, arguments.comb_offset,
                                                  arguments.norm_weight_offset, arguments.hidden_offset};
    if (ticket < rows) {
        /* a row: its input, then its quantization, a thread four values at a time */
        front_row(arguments, finish, arena, ticket, thread, threads, lds.group_sums);
        front_publish<true, false>(&scratch->rows_ready, thread, &word);
    } else if (ticket < rows + mix_blocks) {
        /* the mix project: float32 [24][4 width] by the streams as rows of 4 width values, with the row's scale */
        front_mix_project<ROWS>(arguments, arena, rows, ticket - rows, thread, threads, lds.mixes);
        if (front_publish<true, true>(&scratch->arrived, thread, &word) == mix_blocks - 1u &&
            front_wait<false>(&scratch->rows_ready, rows, thread, &word, &scratch->gave_up)) {
            /* every mix is stored and every row's block has read the carried pre */
            if (thread < rows * MODEL_STREAMS * MODEL_STREAMS) {
                hyper_coefficients_body(finish, arena, thread / (MODEL_STREAMS * MODEL_STREAMS), thread % (MODEL_STREAMS * MODEL_STREAMS));
            }
        }
    } else if constexpr (FFN) {
        struct router_select_arguments select = {};
        select.step_offset = arguments.select.step_offset;
        select.scores_offset = arguments.select.scores_offset;
        select.bias_offset = arguments.select.bias_offset;
        select.expert_offsets_offset = arguments.select.expert_offsets_offset;
        select.affinities_offset = arguments.select.affinities_offset;
        select.jobs_offset = arguments.select.jobs_offset;
        select.weights_offset = arguments.select.weights_offset;
        select.gate_up_last_offset = arguments.select.gate_up_last_offset;
        select.down_last_offset = arguments.select.down_last_offset;
        select.row_count = rows;
        select.reference_order = shape & 1u;
        select.expert_count = expert_bits;
        select.pick_count = (shape >> 11) & 15u;
        select.affinity_kind = (shape >> 15) & 1u;
        select.route_scale = shape >> 16 != 0u ? half_bits_to_float((uint16_t)(shape >> 16)) : 0.0f;
        /* the router's scores in the dense product's order: bf16 [experts][width] by the rows' inputs, no flag, scale 1 */
        struct dense_linear_arguments dense = {};
        dense.weights_offset = arguments.router_weights_offset;
        dense.rows_offset = arguments.hidden_offset;
        dense.output_offset = select.scores_offset;
        dense.output_size = experts;
        dense.input_size = width;
        dense.row_count = rows;
        dense.output_type = DENSE_FLOAT32;
        dense.output_scale = 1.0f;
        const uint32_t groups = experts / SITE_FRONT_SCORE_OUTPUTS, group = (ticket - rows - mix_blocks) * quarters + quarter;
        if (front_wait<true>(&scratch->rows_ready, rows, thread, &word, &scratch->gave_up)) {
            dense_linear_body<DENSE_BFLOAT16, ROWS, SITE_FRONT_SCORE_OUTPUTS>(dense, arena, (const uint16_t *)(arena + dense.rows_offset),
                                                                              group * SITE_FRONT_SCORE_OUTPUTS, 0u, quarter_thread,
                                                                              in_quarter && group < groups, lds.scores[slot]);
            if (front_publish<true, true>(&scratch->scored, thread, &word) == score_blocks - 1u) {
                router_select_body(select, arena, thread, threads, lds.select);
            }
        }
    }
    /* the last block to leave clears the counters: no block reads them any more */
    if (front_publish<false, false>(&scratch->departed, thread, &word) == gridDim.x - 1u && thread == 0u) {
        scratch->tickets = 0u;
        scratch->arrived = 0u;
        scratch->rows_ready = 0u;
        scratch->scored = 0u;
        scratch->departed = 0u;
    }
}

/* the site front's first half: a row a block */
__device__ static __forceinline__ void input_front(const struct site_front_arguments &arguments, unsigned char *arena)
{
    __shared__ float group_sums[32];
    const uint32_t rows = arguments.select.row_count;
    if (gridDim.x != rows) {
        return;
    }
    const struct hyper_finish_arguments finish = {arguments.streams_offset, arguments.pre_offset,
                                                  arguments.scratch_offset + offsetof(struct site_front_scratch, mixes), arguments.scale_offset,
                                                  arguments.base_offset, arguments.post_offset, arguments.comb_offset,
                                                  arguments.norm_weight_offset, arguments.hidden_offset};
    front_row(arguments, finish, arena, blockIdx.x, threadIdx.x, blockDim.x, group_sums);
}

/* its second half: the mix project's blocks; the last to publish forms every row's post, comb and pre */
template <uint32_t ROWS>
__device__ static __forceinline__ void coefficient_front(const struct site_front_arguments &arguments, unsigned char *arena)
{
    __shared__ dense_group_sums<ROWS, SITE_FRONT_MIX_OUTPUTS> sums[FRONT_MOST_QUARTERS];
    __shared__ uint32_t word;
    const uint32_t thread = threadIdx.x, threads = blockDim.x, rows = arguments.select.row_count;
    const uint32_t mix_blocks = site_front_mix_blocks(threads * HYPER_VALUES_PER_THREAD);
    struct site_front_scratch *scratch = (struct site_front_scratch *)(arena + arguments.scratch_offset);
    if (gridDim.x != mix_blocks) {
        return;
    }
    front_mix_project<ROWS>(arguments, arena, rows, blockIdx.x, thread, threads, sums);
    if (front_publish<true, true>(&scratch->arrived, thread, &word) == mix_blocks - 1u) {
        const struct hyper_finish_arguments finish = {arguments.streams_offset, arguments.pre_offset,
                                                      arguments.scratch_offset + offsetof(struct site_front_scratch, mixes), arguments.scale_offset,
                                                      arguments.base_offset, arguments.post_offset, arguments.comb_offset,
                                                      arguments.norm_weight_offset, arguments.hidden_offset};
        if (thread < rows * MODEL_STREAMS * MODEL_STREAMS) {
            hyper_coefficients_body(finish, arena, thread / (MODEL_STREAMS * MODEL_STREAMS), thread % (MODEL_STREAMS * MODEL_STREAMS));
        }
        if (thread == 0u) {
            scratch->arrived = 0u; /* every block has added to it */
        }
    }
}

#define FRONT_STAMP(name, rows, ffn)                                                                                           \
    extern "C" __global__ void __launch_bounds__(FRONT_MOST_THREADS) name##_##rows(struct site_front_arguments arguments, \
                                                                                            unsigned char *arena)              \
    {                                                                                                                          \
        site_front<rows, ffn>(arguments, arena);                                                                               \
    }                                                                                                                          \
    ANEMONE_KERNEL(KERNEL_FILE_SITE_FRONT, name##_##rows, site_front_arguments);
FRONT_STAMP(site_front, 1, false)
FRONT_STAMP(site_front, 8, false)
FRONT_STAMP(ffn_front, 1, true)
FRONT_STAMP(ffn_front, 8, true)

#define HALF_STAMP(name, rows, call)                                                                                           \
    extern "C" __global__ void __launch_bounds__(FRONT_MOST_THREADS) name##_##rows(struct site_front_arguments arguments, \
                                                                                            unsigned char *arena)              \
    {                                                                                                                          \
        call(arguments, arena);                                                                                                \
    }                                                                                                                          \
    ANEMONE_KERNEL(KERNEL_FILE_SITE_FRONT, name##_##rows, site_front_arguments);
HALF_STAMP(input_front, 1, input_front)
HALF_STAMP(input_front, 8, input_front)
HALF_STAMP(coefficient_front, 1, coefficient_front<1>)
HALF_STAMP(coefficient_front, 8, coefficient_front<8>)
