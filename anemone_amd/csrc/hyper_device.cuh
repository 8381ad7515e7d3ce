/*
 * hyper_device.cuh -- a site's mix finish as device code (see kernel_hyper_connection.hip for its definition), shared by
 * hyper_mix_finish and the fused site fronts.
 */
#ifndef HYPER_DEVICE_CUH
#define HYPER_DEVICE_CUH

#include "join_device.cuh"

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

/* The sublayer's input of row `row` (the collapse of its streams by the carried pre, and its norm) by the `row_threads` =
 * width / 8 threads `thread` 0 .. of a block (every one of them calls: barriers inside); group_sums: 32 floats of LDS. */
__device__ static __forceinline__ void hyper_row_input_body(const struct hyper_finish_arguments &arguments, unsigned char *arena, uint64_t row,
                                                             uint32_t thread, uint64_t row_threads, float *group_sums)
{
    const uint32_t lane = thread % 32u;
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
}

/* Row `row`'s post, comb and pre from its mixes, by sixteen threads `thread` 0 .. 15 that are sixteen lanes in a row of one
 * wavefront, after every reader of the carried pre: Sinkhorn, thread e holding comb's element e = 4 row + column */
__device__ static __forceinline__ void hyper_coefficients_body(const struct hyper_finish_arguments &arguments, unsigned char *arena, uint64_t row,
                                                               uint32_t thread)
{
    float *carried = (float *)(arena + arguments.pre_offset) + row * MODEL_STREAMS;
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

/* both, as hyper_mix_finish runs them: the row's block */
__device__ static __forceinline__ void hyper_mix_finish_body(const struct hyper_finish_arguments &arguments, unsigned char *arena, uint64_t row,
                                                             uint32_t thread, uint64_t row_threads, float *group_sums)
{
    hyper_row_input_body(arguments, arena, row, thread, row_threads, group_sums);
    if (thread < MODEL_STREAMS * MODEL_STREAMS) {
        hyper_coefficients_body(arguments, arena, row, thread);
    }
}

#endif
