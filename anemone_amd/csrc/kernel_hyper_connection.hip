/*
 * kernel_hyper_connection.hip -- the FFN site's post and join on gfx950: what follows the routed experts of a layer.
 * Entry names, records and arithmetic follow the reference (source/kernel_hyper_connection.cu:204-226, 249-271;
 * source/kernel_hyper_connection.cuh:62-85; source/kernel_expert_join.cuh:35-57;
 * include/anemone/hyper_connection_records.h:27-29; include/anemone/expert_fused_records.h:31-41):
 *   - hyper_post_entry: stream k of a row becomes bfloat16(post_k y_d + ((((0 + c_0k X_0d) + c_1k X_1d) + c_2k X_2d) +
 *     c_3k X_3d)) of the four streams X as they were before any is written, in place; with is_combined 1, y_d is first
 *     bfloat16(s_d + y_d) of the routed experts' float32 sums s;
 *   - expert_join: expert_row_sum_entry (the float32 sum of a row's pair outputs from +0 in ascending slot order,
 *     stored where the record names an array for it) and behind it that post with the combine, in one launch.
 *   - hyper_mix_finish: the step ahead of the sublayer (below, with its own comment).
 * Every product and sum is rounded on its own (no fused multiply-add); a bfloat16 is rounded to nearest with a tie to
 * even, a not-a-number to 0x7FC0.
 *
 * Work mapping: a thread takes HYPER_VALUES_PER_THREAD = 8 consecutive values of one row (one 16-byte load of each
 * array); grid (width / (8 block[0]), rows). The streams' width is what the grid covers: the reference fixes it at its
 * model's 5,120 (it checks blockDim.x gridDim.x against that); here any multiple of 8 block[0]. Every load of a thread
 * is asked for before the first is used: the kernel moves (pairs_per_row + 9) x 2 bytes a value and computes little.
 */
#include "kernel_registry.h"
#include "join_device.cuh"

extern "C" __global__ void __launch_bounds__(HYPER_PIECE_THREADS) hyper_post_entry(struct hyper_post_arguments arguments, unsigned char *arena)
{
    const uint64_t row = blockIdx.y, row_threads = (uint64_t)gridDim.x * blockDim.x, thread = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const float *post = (const float *)(arena + arguments.post_offset) + row * MODEL_STREAMS;
    const float *comb = (const float *)(arena + arguments.comb_offset) + row * MODEL_STREAMS * MODEL_STREAMS;
    uint4_t *streams = (uint4_t *)(arena + arguments.streams_offset) + row * MODEL_STREAMS * row_threads + thread;
    float output[HYPER_VALUES_PER_THREAD];
    join_unpack(((const uint4_t *)(arena + arguments.output_offset))[row * row_threads + thread], output);
    if (arguments.is_combined != 0u) {
        const float4_t *sums = (const float4_t *)(arena + arguments.sums_offset) + (row * row_threads + thread) * 2u;
        const float4_t low = sums[0], high = sums[1];
#pragma unroll
        for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
            output[v] = bf16_to_float(float_to_bf16(__fadd_rn(v < 4u ? low[v % 4u] : high[v % 4u], output[v])));
        }
    }
    join_post_values(output, post, comb, streams, row_threads);
}
ANEMONE_KERNEL(KERNEL_FILE_HYPER_CONNECTION, hyper_post_entry, hyper_post_arguments);

extern "C" __global__ void __launch_bounds__(HYPER_PIECE_THREADS) expert_join(struct expert_join_arguments arguments, unsigned char *arena)
{
    const uint64_t row = blockIdx.y, row_threads = (uint64_t)gridDim.x * blockDim.x, thread = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    float shared_output[HYPER_VALUES_PER_THREAD];
    join_unpack(((const uint4_t *)(arena + arguments.shared_output_offset))[row * row_threads + thread], shared_output);
    join_values((const uint4_t *)(arena + arguments.pair_output_offset) + row * arguments.pairs_per_row * row_threads + thread,
                arguments.pairs_per_row, shared_output, (const float *)(arena + arguments.post_offset) + row * MODEL_STREAMS,
                (const float *)(arena + arguments.comb_offset) + row * MODEL_STREAMS * MODEL_STREAMS,
                (uint4_t *)(arena + arguments.streams_offset) + row * MODEL_STREAMS * row_threads + thread,
                arguments.row_sums_offset == EXPERT_JOIN_NO_ROW_SUMS
                    ? nullptr
                    : (float4_t *)(arena + arguments.row_sums_offset) + (row * row_threads + thread) * 2u,
                row_threads);
}
ANEMONE_KERNEL(KERNEL_FILE_HYPER_CONNECTION, expert_join, expert_join_arguments);

/* ---- the mix finish: what stands between a site's mix project and its sublayer ----
 * include/anemone/hyper_connection_records.h:10-22 and source/kernel_hyper_connection.cu:40-125,
 * source/kernel_hyper_connection.cuh of the reference. A row's block: the collapse of the four streams with the CARRIED
 * pre p, h_d = bfloat16((((0 + p_0 X_0d) + p_1 X_1d) + p_2 X_2d) + p_3 X_3d); q, the sum of the h_d h_d in a fixed tree
 * (a thread its eight from +0, a group of 32 threads by exchanges at distance 16 down to 1, one group the groups' sums
 * with zeros behind them); hidden_d = bfloat16(w_d (h_d r(q (1 / width) + 1e-20))), r the float32 nearest the reciprocal
 * square root (the reference takes its card's rsqrtf); and Sinkhorn of the row's 24 mixes, which writes post and comb and
 * replaces the carried pre with the site's once every thread has read it (behind the block's barrier). e^x is det_expf
 * (the reference takes its card's expf), every division IEEE, a line's four values added (x_0 + x_2) + (x_1 + x_3). */
__device__ static __forceinline__ float hyper_group_sum(float value)
{
#pragma unroll
    for (uint32_t distance = 16u; distance != 0u; distance /= 2u) {
        value = __fadd_rn(value, __shfl_xor(value, (int)distance, 32));
    }
    return value;
}

__device__ static __forceinline__ float hyper_sigmoid(float value)
{
    return __fdiv_rn(1.0f, __fadd_rn(1.0f, det_expf(-value)));
}

/* the value of lane `source` of the first sixteen (every one of them calls) */
__device__ static __forceinline__ float hyper_lane(float value, uint32_t source)
{
    return __shfl(value, (int)source, 16);
}

/* element e = 4 row + column of comb on lane e of sixteen: divided by its row's or its column's sum */
__device__ static __forceinline__ float hyper_divide(float value, uint32_t element, bool rows, float sum_epsilon, float quotient_epsilon)
{
    const uint32_t first = rows ? element / MODEL_STREAMS * MODEL_STREAMS : element % MODEL_STREAMS, stride = rows ? 1u : MODEL_STREAMS;
    const float x0 = hyper_lane(value, first), x1 = hyper_lane(value, first + stride), x2 = hyper_lane(value, first + 2u * stride),
                x3 = hyper_lane(value, first + 3u * stride);
    const float sum = __fadd_rn(__fadd_rn(x0, x2), __fadd_rn(x1, x3));
    return __fadd_rn(__fdiv_rn(value, __fadd_rn(sum, sum_epsilon)), quotient_epsilon);
}

extern "C" __global__ void __launch_bounds__(HYPER_FINISH_MOST_THREADS) hyper_mix_finish(struct hyper_finish_arguments arguments, unsigned char *arena)
{
    __shared__ float group_sums[32];
    const uint64_t row = blockIdx.y, row_threads = blockDim.x;
    const uint32_t thread = threadIdx.x, lane = thread % 32u;
    float *carried = (float *)(arena + arguments.pre_offset) + row * MODEL_STREAMS;
    const float4_t pre = *(const float4_t *)carried;
    const uint4_t *streams = (const uint4_t *)(arena + arguments.streams_offset) + row * MODEL_STREAMS * row_threads + thread;
    uint4_t loads[MODEL_STREAMS];
#pragma unroll
    for (uint32_t stream = 0; stream < MODEL_STREAMS; stream++) {
        loads[stream] = streams[stream * row_threads];
    }
    const uint4_t weight_load = ((const uint4_t *)(arena + arguments.weight_offset))[thread];
    if (thread < 32u) {
        group_sums[thread] = 0.0f; /* zeros behind the row's groups */
    }
    float hidden[HYPER_VALUES_PER_THREAD], square_sum = 0.0f;
#pragma unroll
    for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
        hidden[v] = 0.0f;
    }
#pragma unroll
    for (uint32_t stream = 0; stream < MODEL_STREAMS; stream++) {
        float values[HYPER_VALUES_PER_THREAD];
        join_unpack(loads[stream], values);
#pragma unroll
        for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
            hidden[v] = __fadd_rn(hidden[v], __fmul_rn(pre[stream], values[v]));
        }
    }
#pragma unroll
    for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
        hidden[v] = bf16_to_float(float_to_bf16(hidden[v]));
        square_sum = __fadd_rn(square_sum, __fmul_rn(hidden[v], hidden[v]));
    }
    square_sum = hyper_group_sum(square_sum);
    __syncthreads(); /* the zeros are written */
    if (lane == 0u) {
        group_sums[thread / 32u] = square_sum;
    }
    __syncthreads(); /* and every thread has read the carried pre */
    const float operand = __fadd_rn(__fmul_rn(hyper_group_sum(group_sums[lane]), __fdiv_rn(1.0f, (float)(row_threads * HYPER_VALUES_PER_THREAD))),
                                    MODEL_NORM_EPSILON);
    const float factor = (float)(1.0 / __dsqrt_rn((double)operand));
    float weights[HYPER_VALUES_PER_THREAD];
    join_unpack(weight_load, weights);
#pragma unroll
    for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
        hidden[v] = __fmul_rn(weights[v], __fmul_rn(hidden[v], factor));
    }
    ((uint4_t *)(arena + arguments.hidden_offset))[row * row_threads + thread] = join_pack(hidden);
    if (thread >= MODEL_STREAMS * MODEL_STREAMS) {
        return;
    }
    /* Sinkhorn on the first sixteen threads: thread e holds comb's element e = 4 row + column */
    const float *mixes = (const float *)(arena + arguments.mixes_offset) + row * MODEL_MIXES;
    const float *scale = (const float *)(arena + arguments.scale_offset), *base = (const float *)(arena + arguments.base_offset);
    const uint32_t element = thread, first_of_row = element / MODEL_STREAMS * MODEL_STREAMS;
    float comb = __fmaf_rn(mixes[2u * MODEL_STREAMS + element], scale[2], base[2u * MODEL_STREAMS + element]);
    float largest = -__builtin_huge_valf();
#pragma unroll
    for (uint32_t column = 0; column < MODEL_STREAMS; column++) {
        const float other = hyper_lane(comb, first_of_row + column);
        largest = other > largest ? other : largest;
    }
    comb = det_expf(__fsub_rn(comb, largest));
    comb = hyper_divide(comb, element, true, 0.0f, MODEL_HYPER_EPSILON);
    comb = hyper_divide(comb, element, false, MODEL_HYPER_EPSILON, 0.0f);
    for (uint32_t round = 1; round < MODEL_SINKHORN_ITERATIONS; round++) {
        comb = hyper_divide(comb, element, true, MODEL_HYPER_EPSILON, 0.0f);
        comb = hyper_divide(comb, element, false, MODEL_HYPER_EPSILON, 0.0f);
    }
    ((float *)(arena + arguments.comb_offset))[row * MODEL_STREAMS * MODEL_STREAMS + element] = comb;
    if (thread < MODEL_STREAMS) {
        ((float *)(arena + arguments.post_offset))[row * MODEL_STREAMS + thread] =
            __fmul_rn(2.0f, hyper_sigmoid(__fmaf_rn(mixes[MODEL_STREAMS + thread], scale[1], base[MODEL_STREAMS + thread])));
        carried[thread] = __fadd_rn(hyper_sigmoid(__fmaf_rn(mixes[thread], scale[0], base[thread])), MODEL_HYPER_EPSILON);
    }
}
ANEMONE_KERNEL(KERNEL_FILE_HYPER_CONNECTION, hyper_mix_finish, hyper_finish_arguments);
