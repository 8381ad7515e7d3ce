/*
 * orc_site.c -- see orc_site.h. TEST INFRASTRUCTURE: never the product path.
 */
#include "orc_site.h"

#include <math.h>
#include <stddef.h>
#include <string.h>

#include "orc_common.h"
#include "orc_exl3.h" /* orc_expf */

#define DENSE_THREADS 256u
#define DENSE_CHUNK 8u
#define GROUP_LANES 32u
#define DENSE_GROUPS (DENSE_THREADS / GROUP_LANES)
#define STREAMS 4u
#define HYPER_EPSILON 1e-6f
#define NORM_EPSILON 1e-20f
#define SINKHORN_ROUNDS 20u
#define THREAD_VALUES 8u

float orc_reciprocal_root(float operand)
{
    return (float)(1.0 / sqrt((double)operand));
}

/* lane 0's value after every lane l adds lane l ^ d's at d = 16, 8, 4, 2, 1 (include/anemone/dense_linear_records.h:13) */
static float group_sum(float lanes[GROUP_LANES])
{
    for (uint32_t distance = GROUP_LANES / 2u; distance != 0u; distance /= 2u) {
        float next[GROUP_LANES];
        for (uint32_t lane = 0; lane < GROUP_LANES; lane++) {
            next[lane] = lanes[lane] + lanes[lane ^ distance];
        }
        memcpy(lanes, next, sizeof(next));
    }
    return lanes[0];
}

static float weight_value(uint32_t weight_type, const void *weights, uint64_t index)
{
    return weight_type == ORC_DENSE_FLOAT32 ? ((const float *)weights)[index] : orc_bf16_to_float(((const uint16_t *)weights)[index]);
}

/* the block's tree over the threads' chains (source/kernel_dense_linear.cu:133-164 of the reference) */
static float block_sum(const float chains[DENSE_THREADS])
{
    float sum = 0.0f;
    for (uint32_t group = 0; group < DENSE_GROUPS; group++) {
        float lanes[GROUP_LANES];
        memcpy(lanes, chains + group * GROUP_LANES, sizeof(lanes));
        sum = sum + group_sum(lanes);
    }
    return sum;
}

int orc_dense_linear(uint32_t weight_type, const void *weights, uint32_t output_size, uint32_t input_size, uint32_t flags,
                     float epsilon, float output_scale, uint32_t output_type, const uint16_t *rows, uint32_t row_count,
                     void *output)
{
    if (weight_type > ORC_DENSE_FLOAT32 || output_type > ORC_DENSE_FLOAT32 || (flags & ~ORC_DENSE_ROW_SCALE) != 0u ||
        input_size == 0u || input_size % DENSE_CHUNK != 0u || output_size == 0u) {
        return -1;
    }
    const uint32_t chunks = input_size / DENSE_CHUNK;
    for (uint32_t row = 0; row < row_count; row++) {
        const uint16_t *values = rows + (uint64_t)row * input_size;
        float factor = 1.0f;
        if ((flags & ORC_DENSE_ROW_SCALE) != 0u) {
            float squares[DENSE_THREADS];
            for (uint32_t thread = 0; thread < DENSE_THREADS; thread++) {
                float chain = 0.0f;
                for (uint32_t chunk = thread; chunk < chunks; chunk += DENSE_THREADS) {
                    for (uint32_t i = 0; i < DENSE_CHUNK; i++) {
                        const float value = orc_bf16_to_float(values[chunk * DENSE_CHUNK + i]);
                        chain = fmaf(value, value, chain);
                    }
                }
                squares[thread] = chain;
            }
            factor = orc_reciprocal_root(block_sum(squares) * (1.0f / (float)input_size) + epsilon);
        }
        for (uint32_t out = 0; out < output_size; out++) {
            float chains[DENSE_THREADS];
            for (uint32_t thread = 0; thread < DENSE_THREADS; thread++) {
                float chain = 0.0f;
                for (uint32_t chunk = thread; chunk < chunks; chunk += DENSE_THREADS) {
                    for (uint32_t i = 0; i < DENSE_CHUNK; i++) {
                        const uint32_t k = chunk * DENSE_CHUNK + i;
                        chain = fmaf(weight_value(weight_type, weights, (uint64_t)out * input_size + k), orc_bf16_to_float(values[k]), chain);
                    }
                }
                chains[thread] = chain;
            }
            float sum = block_sum(chains);
            if ((flags & ORC_DENSE_ROW_SCALE) != 0u) {
                sum = sum * factor;
            }
            const uint64_t index = (uint64_t)row * output_size + out;
            if (output_type == ORC_DENSE_FLOAT32) {
                ((float *)output)[index] = sum * output_scale;
            } else {
                ((uint16_t *)output)[index] = orc_bf16_from_float(orc_bf16_to_float(orc_bf16_from_float(sum)) * output_scale);
            }
        }
    }
    return 0;
}

static float sigmoid(float value)
{
    return 1.0f / (1.0f + orc_expf(-value));
}

/* (x_0 + x_2) + (x_1 + x_3) of four values `stride` apart (include/anemone/hyper_connection_records.h:12) */
static float line_sum(const float *values, uint32_t stride)
{
    return (values[0] + values[2u * stride]) + (values[stride] + values[3u * stride]);
}

static void divide_by_sums(float *comb, int rows, float sum_epsilon, float quotient_epsilon)
{
    float sums[STREAMS];
    for (uint32_t line = 0; line < STREAMS; line++) {
        sums[line] = rows ? line_sum(comb + line * STREAMS, 1u) : line_sum(comb + line, STREAMS);
    }
    for (uint32_t element = 0; element < STREAMS * STREAMS; element++) {
        comb[element] = comb[element] / (sums[rows ? element / STREAMS : element % STREAMS] + sum_epsilon) + quotient_epsilon;
    }
}

void orc_hyper_sinkhorn(const float *mixes, const float *scale, const float *base, float *pre_out, float *post_out, float *comb_out)
{
    float comb[STREAMS * STREAMS];
    for (uint32_t stream = 0; stream < STREAMS; stream++) {
        pre_out[stream] = sigmoid(fmaf(mixes[stream], scale[0], base[stream])) + HYPER_EPSILON;
        post_out[stream] = 2.0f * sigmoid(fmaf(mixes[STREAMS + stream], scale[1], base[STREAMS + stream]));
    }
    for (uint32_t row = 0; row < STREAMS; row++) {
        float largest = -INFINITY;
        for (uint32_t column = 0; column < STREAMS; column++) {
            const uint32_t element = row * STREAMS + column;
            comb[element] = fmaf(mixes[2u * STREAMS + element], scale[2], base[2u * STREAMS + element]);
            largest = comb[element] > largest ? comb[element] : largest;
        }
        for (uint32_t column = 0; column < STREAMS; column++) {
            comb[row * STREAMS + column] = orc_expf(comb[row * STREAMS + column] - largest);
        }
    }
    divide_by_sums(comb, 1, 0.0f, HYPER_EPSILON);
    divide_by_sums(comb, 0, HYPER_EPSILON, 0.0f);
    for (uint32_t round = 1; round < SINKHORN_ROUNDS; round++) {
        divide_by_sums(comb, 1, HYPER_EPSILON, 0.0f);
        divide_by_sums(comb, 0, HYPER_EPSILON, 0.0f);
    }
    memcpy(comb_out, comb, sizeof(comb));
}

void orc_hyper_collapse(const uint16_t *streams, const float *pre, uint32_t width, uint16_t *collapsed_out)
{
    for (uint32_t d = 0; d < width; d++) {
        float sum = 0.0f;
        for (uint32_t stream = 0; stream < STREAMS; stream++) {
            sum = sum + pre[stream] * orc_bf16_to_float(streams[(uint64_t)stream * width + d]);
        }
        collapsed_out[d] = orc_bf16_from_float(sum);
    }
}

float orc_hyper_norm_operand(const uint16_t *collapsed, uint32_t width)
{
    float group_sums[GROUP_LANES] = {0.0f}; /* zeros behind the row's groups */
    const uint32_t groups = width / THREAD_VALUES / GROUP_LANES;
    for (uint32_t group = 0; group < groups; group++) {
        float lanes[GROUP_LANES];
        for (uint32_t lane = 0; lane < GROUP_LANES; lane++) {
            const uint64_t first = ((uint64_t)group * GROUP_LANES + lane) * THREAD_VALUES;
            float sum = 0.0f;
            for (uint32_t v = 0; v < THREAD_VALUES; v++) {
                const float value = orc_bf16_to_float(collapsed[first + v]);
                sum = sum + value * value;
            }
            lanes[lane] = sum;
        }
        group_sums[group] = group_sum(lanes);
    }
    return group_sum(group_sums) * (1.0f / (float)width) + NORM_EPSILON;
}

void orc_hyper_norm_with(const uint16_t *collapsed, const uint16_t *weight, float factor, uint32_t width, uint16_t *normed_out)
{
    for (uint32_t d = 0; d < width; d++) {
        const float scaled = orc_bf16_to_float(collapsed[d]) * factor;
        normed_out[d] = orc_bf16_from_float(orc_bf16_to_float(weight[d]) * scaled);
    }
}

void orc_hyper_mix_finish(const uint16_t *streams, float *carried_pre, const float *mixes, const float *scale, const float *base,
                          const uint16_t *norm_weight, uint32_t width, float *post_out, float *comb_out, uint16_t *hidden_out)
{
    uint16_t collapsed[8192];
    float site_pre[STREAMS];
    orc_hyper_sinkhorn(mixes, scale, base, site_pre, post_out, comb_out);
    orc_hyper_collapse(streams, carried_pre, width, collapsed);
    orc_hyper_norm_with(collapsed, norm_weight, orc_reciprocal_root(orc_hyper_norm_operand(collapsed, width)), width, hidden_out);
    memcpy(carried_pre, site_pre, sizeof(site_pre));
}
