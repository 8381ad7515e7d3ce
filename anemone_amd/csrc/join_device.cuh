/*
 * join_device.cuh -- the join of the FFN site for eight consecutive values of one row, which the post, the join
 * (kernel_hyper_connection.hip) and the shared join (kernel_trunk_linear.hip) share. The arithmetic of the reference's
 * source/kernel_hyper_connection.cuh:42-85 and source/kernel_expert_join.cuh:35-57, value by value, in their order:
 * every product and sum rounded on its own.
 */
#ifndef JOIN_DEVICE_CUH
#define JOIN_DEVICE_CUH

#include "exl3_device.cuh" /* bf16 helpers, vector types */

#include "anemone_records.h"

/* the eight bfloat16 values of a 16-byte load as float32, and eight float32 values rounded to bfloat16 as one */
__device__ static __forceinline__ void join_unpack(uint4_t load, float (&values)[HYPER_VALUES_PER_THREAD])
{
#pragma unroll
    for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
        const uint32_t word = load[v / 2u];
        values[v] = __uint_as_float(v % 2u == 0u ? word << 16 : word & 0xFFFF0000u);
    }
}

__device__ static __forceinline__ uint4_t join_pack(const float (&values)[HYPER_VALUES_PER_THREAD])
{
    uint4_t load;
#pragma unroll
    for (uint32_t word = 0; word < 4u; word++) {
        load[word] = (uint32_t)float_to_bf16(values[2u * word]) | ((uint32_t)float_to_bf16(values[2u * word + 1u]) << 16);
    }
    return load;
}

/* The post of a thread's eight values of a row: output y as the post takes it (with the combine, the routed sums added
 * and rounded); post and comb the row's; streams the thread's load of stream 0, the streams `stride` loads apart, read
 * and written in place. */
__device__ static __forceinline__ void join_post_values(const float (&output)[HYPER_VALUES_PER_THREAD], const float *post, const float *comb,
                                                        uint4_t *streams, uint64_t stride)
{
    uint4_t loads[MODEL_STREAMS];
#pragma unroll
    for (uint32_t stream = 0; stream < MODEL_STREAMS; stream++) {
        loads[stream] = streams[stream * stride];
    }
    const float4_t post_of = *(const float4_t *)post;
    float4_t comb_of[MODEL_STREAMS]; /* [source][target] */
#pragma unroll
    for (uint32_t source = 0; source < MODEL_STREAMS; source++) {
        comb_of[source] = ((const float4_t *)comb)[source];
    }
    float values[MODEL_STREAMS][HYPER_VALUES_PER_THREAD];
#pragma unroll
    for (uint32_t stream = 0; stream < MODEL_STREAMS; stream++) {
        join_unpack(loads[stream], values[stream]);
    }
#pragma unroll
    for (uint32_t target = 0; target < MODEL_STREAMS; target++) {
        float mixed[HYPER_VALUES_PER_THREAD];
#pragma unroll
        for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
            float sum = 0.0f;
#pragma unroll
            for (uint32_t source = 0; source < MODEL_STREAMS; source++) {
                sum = __fadd_rn(sum, __fmul_rn(comb_of[source][target], values[source][v]));
            }
            mixed[v] = __fadd_rn(__fmul_rn(post_of[target], output[v]), sum);
        }
        streams[target * stride] = join_pack(mixed);
    }
}

#define JOIN_SLOTS_IN_FLIGHT 8u

/* The join of eight values of a row: pairs their load of the row's first pair output, a slot `stride` loads on;
 * shared_output the shared expert's output there; row_sums where their float32 sums go, or nullptr. */
__device__ static __forceinline__ void join_values(const uint4_t *pairs, uint32_t pairs_per_row, const float (&shared_output)[HYPER_VALUES_PER_THREAD],
                                                   const float *post, const float *comb, uint4_t *streams, float4_t *row_sums, uint64_t stride)
{
    float routed[HYPER_VALUES_PER_THREAD], output[HYPER_VALUES_PER_THREAD];
#pragma unroll
    for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
        routed[v] = 0.0f;
    }
    /* eight slots at a time, their loads all asked for before the first is added: one trip to memory for the eight, the
     * additions in slot order as before */
    uint32_t slot = 0;
    for (; slot + JOIN_SLOTS_IN_FLIGHT <= pairs_per_row; slot += JOIN_SLOTS_IN_FLIGHT) {
        uint4_t loaded[JOIN_SLOTS_IN_FLIGHT];
#pragma unroll
        for (uint32_t s = 0; s < JOIN_SLOTS_IN_FLIGHT; s++) {
            loaded[s] = pairs[(uint64_t)(slot + s) * stride];
        }
#pragma unroll
        for (uint32_t s = 0; s < JOIN_SLOTS_IN_FLIGHT; s++) {
            float pair[HYPER_VALUES_PER_THREAD];
            join_unpack(loaded[s], pair);
#pragma unroll
            for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
                routed[v] = __fadd_rn(routed[v], pair[v]);
            }
        }
    }
    for (; slot < pairs_per_row; slot++) {
        float pair[HYPER_VALUES_PER_THREAD];
        join_unpack(pairs[(uint64_t)slot * stride], pair);
#pragma unroll
        for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
            routed[v] = __fadd_rn(routed[v], pair[v]);
        }
    }
    if (row_sums != nullptr) {
        row_sums[0] = (float4_t){routed[0], routed[1], routed[2], routed[3]};
        row_sums[1] = (float4_t){routed[4], routed[5], routed[6], routed[7]};
    }
#pragma unroll
    for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
        output[v] = bf16_to_float(float_to_bf16(__fadd_rn(routed[v], shared_output[v])));
    }
    join_post_values(output, post, comb, streams, stride);
}

#endif
