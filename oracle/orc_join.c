/* orc_join.c -- see orc_join.h. TEST INFRASTRUCTURE, never the product path. */
#include "orc_join.h"

#include <stdlib.h>

#include "orc_common.h"
#include "orc_linear.h"

void orc_hyper_post(const uint16_t *streams, const float *post, const float *comb, const uint16_t *output,
                    const float *routed_sums, uint32_t width, uint16_t *streams_out)
{
    for (uint32_t d = 0; d < width; d++) {
        float y = orc_bf16_to_float(output[d]);
        if (routed_sums != NULL) {
            const float joined = routed_sums[d] + y;
            y = orc_bf16_to_float(orc_bf16_from_float(joined));
        }
        float before[ORC_STREAMS];
        for (uint32_t j = 0; j < ORC_STREAMS; j++) {
            before[j] = orc_bf16_to_float(streams[(uint64_t)j * width + d]);
        }
        for (uint32_t k = 0; k < ORC_STREAMS; k++) {
            float mixed = 0.0f;
            for (uint32_t j = 0; j < ORC_STREAMS; j++) {
                const float product = comb[j * ORC_STREAMS + k] * before[j];
                mixed = mixed + product;
            }
            const float scaled = post[k] * y;
            const float value = scaled + mixed;
            streams_out[(uint64_t)k * width + d] = orc_bf16_from_float(value);
        }
    }
}

void orc_expert_join(const uint16_t *pair_output, const uint16_t *shared_output, uint16_t *streams, const float *post,
                     const float *comb, float *row_sums_out, uint32_t rows, uint32_t pairs_per_row, uint32_t width)
{
    float *sums = malloc((size_t)width * sizeof(float));
    for (uint32_t row = 0; row < rows; row++) {
        for (uint32_t d = 0; d < width; d++) {
            sums[d] = orc_row_sum_bf16(pair_output + (uint64_t)row * pairs_per_row * width, pairs_per_row, width, d);
            if (row_sums_out != NULL) {
                row_sums_out[(uint64_t)row * width + d] = sums[d];
            }
        }
        uint16_t *mine = streams + (uint64_t)row * ORC_STREAMS * width;
        orc_hyper_post(mine, post + (uint64_t)row * ORC_STREAMS, comb + (uint64_t)row * ORC_STREAMS * ORC_STREAMS,
                       shared_output + (uint64_t)row * width, sums, width, mine);
    }
    free(sums);
}

void orc_trunk_hidden(const uint16_t *gate, const uint16_t *up, float limit, uint32_t count, uint16_t *hidden_out)
{
    for (uint32_t i = 0; i < count; i++) {
        hidden_out[i] = orc_hidden_bits(orc_bf16_to_float(gate[i]), orc_bf16_to_float(up[i]), limit, 1.0f);
    }
}
