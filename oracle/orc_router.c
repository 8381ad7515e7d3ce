/*
 * orc_router.c -- CPU oracle of the router. Contract and citations: orc_router.h.
 * TEST INFRASTRUCTURE, never the product path. Build with -ffp-contract=off.
 */
#include "orc_router.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "orc_common.h"
#include "orc_exl3.h" /* orc_expf */

_Static_assert(sizeof(struct orc_job) == 96, "job table entry");
_Static_assert(sizeof(struct orc_wide_tile) == 32, "wide tile");

#define PROJECTION_CHAINS 32u
#define SOFTPLUS_THRESHOLD 20.0f
#define WEIGHT_EPSILON 1e-20f

float orc_log1pf(float y)
{
    /* u = fl(1 + y) and its rounding error c; log(u) by the atanh series on m in (sqrt(1/2), sqrt(2)]; + c / u */
    const float u = 1.0f + y;
    const float c = y - (u - 1.0f);
    float m = u, e = 0.0f;
    if (u > 1.41421354f) {
        m = u * 0.5f;
        e = 1.0f;
    }
    const float f = m - 1.0f;
    const float s = f / (2.0f + f);
    const float z = s * s;
    float r = fmaf(z, 0.222222224f, 0.285714298f);
    r = fmaf(r, z, 0.400000006f);
    r = fmaf(r, z, 0.666666687f);
    r = r * z;
    const float hfsq = 0.5f * f * f;
    const float log_m = f - (hfsq - s * (hfsq + r));
    const float low = fmaf(e, 9.05800061e-06f, c / u);   /* ln2 = 0.693138123 + 9.05800061e-06 */
    return fmaf(e, 0.693138123f, log_m + low);
}

float orc_router_affinity(float score, int kind)
{
    if (kind == ORC_AFFINITY_SIGMOID) {
        return 1.0f / (1.0f + orc_expf(-score));
    }
    if (score != score) {
        return score;
    }
    if (score > SOFTPLUS_THRESHOLD) {
        return sqrtf(score);
    }
    const float positive = score > 0.0f ? score : 0.0f;
    const float softplus = positive + orc_log1pf(orc_expf(-fabsf(score)));
    return sqrtf(softplus);
}

void orc_router_projection(const uint16_t *x_bf16, const uint16_t *w_bf16, uint32_t rows, uint32_t hidden,
                           uint32_t experts, float *scores_out)
{
    for (uint32_t row = 0; row < rows; row++) {
        for (uint32_t expert = 0; expert < experts; expert++) {
            float chain[PROJECTION_CHAINS];
            for (uint32_t c = 0; c < PROJECTION_CHAINS; c++) {
                float sum = 0.0f;
                for (uint32_t k = c; k < hidden; k += PROJECTION_CHAINS) {
                    sum = fmaf(orc_bf16_to_float(w_bf16[(uint64_t)expert * hidden + k]),
                               orc_bf16_to_float(x_bf16[(uint64_t)row * hidden + k]), sum);
                }
                chain[c] = 0.0f + sum;
            }
            for (uint32_t distance = PROJECTION_CHAINS / 2u; distance != 0u; distance /= 2u) {
                for (uint32_t c = 0; c < distance; c++) {
                    chain[c] = chain[c] + chain[c + distance];
                }
            }
            scores_out[(uint64_t)row * experts + expert] = 0.0f + chain[0];
        }
    }
}

/* the order of the top-k as one integer: a larger key comes first */
static uint64_t key_of(float biased, uint32_t expert)
{
    const uint32_t bits = orc_f32_bits(biased);
    uint32_t ordered;
    if (biased != biased) {
        ordered = 0xFFFFFFFFu;
    } else if (bits & 0x80000000u) {
        ordered = ~bits;
    } else {
        ordered = bits | 0x80000000u;
    }
    return ((uint64_t)ordered << 32) | (uint32_t)~expert;
}

void orc_router_select(const float *affinities, const float *bias, uint32_t experts, uint32_t picks,
                       int reference_order, float route_scale, uint32_t *experts_out, float *weights_out)
{
    uint64_t *keys = malloc(experts * sizeof *keys);
    uint32_t *chosen = malloc(picks * sizeof *chosen); /* in the order of the top-k */
    for (uint32_t expert = 0; expert < experts; expert++) {
        keys[expert] = key_of(affinities[expert] + bias[expert], expert);
    }
    for (uint32_t pick = 0; pick < picks; pick++) {
        uint64_t best = 0;
        uint32_t best_expert = 0;
        for (uint32_t expert = 0; expert < experts; expert++) {
            if (keys[expert] > best) {
                best = keys[expert];
                best_expert = expert;
            }
        }
        keys[best_expert] = 0; /* below every key: an ordered float is at least 0x007FFFFF */
        chosen[pick] = best_expert;
    }
    for (uint32_t pick = 0; pick < picks; pick++) {
        uint32_t slot = 0;
        for (uint32_t other = 0; other < picks; other++) {
            slot += chosen[other] < chosen[pick] ? 1u : 0u;
        }
        experts_out[slot] = chosen[pick];
    }
    float sum = 0.0f;
    for (uint32_t slot = 0; slot < picks; slot++) {
        sum = sum + affinities[experts_out[slot]];
    }
    if (reference_order && picks == 6u) {
        const float *a = affinities;
        sum = ((a[chosen[0]] + a[chosen[4]]) + a[chosen[2]]) + ((a[chosen[1]] + a[chosen[5]]) + a[chosen[3]]);
    }
    const float denominator = sum + WEIGHT_EPSILON;
    for (uint32_t slot = 0; slot < picks; slot++) {
        weights_out[slot] = affinities[experts_out[slot]] / denominator * route_scale;
    }
    free(keys);
    free(chosen);
}

void orc_router_jobs(const uint32_t *experts, const float *weights, uint32_t picks, uint32_t live_rows,
                     uint32_t row_count, uint32_t expert_count, const uint64_t *expert_offsets,
                     struct orc_job *jobs_out)
{
    const uint32_t capacity = row_count * picks;
    uint32_t used = 0;
    memset(jobs_out, 0, (size_t)capacity * sizeof *jobs_out);
    for (uint32_t expert = 0; expert < expert_count && used < capacity; expert++) {
        struct orc_job *job = &jobs_out[used];
        for (uint32_t pair = 0; pair < live_rows * picks && job->row_count < ORC_JOB_ROWS; pair++) {
            if (experts[pair] == expert) {
                job->pair_index[job->row_count] = pair;
                job->route_weight[job->row_count] = weights[pair];
                job->row_count++;
            }
        }
        if (job->row_count != 0u) {
            job->gate_offset = expert_offsets[expert * 3u + 0u];
            job->up_offset = expert_offsets[expert * 3u + 1u];
            job->down_offset = expert_offsets[expert * 3u + 2u];
            job->expert = expert;
            used++;
        }
    }
}

uint32_t orc_router_wide_tile_count(uint32_t row_count, uint32_t picks, uint32_t expert_count)
{
    return (row_count * picks + ORC_TILE_PAIRS - 1u) / ORC_TILE_PAIRS + expert_count;
}

uint32_t orc_router_wide_job_count(uint32_t row_count, uint32_t picks, uint32_t expert_count)
{
    const uint32_t pairs = row_count * picks;
    const uint32_t bound = (pairs + (ORC_JOB_ROWS - 1u) * expert_count) / ORC_JOB_ROWS;
    return pairs < bound ? pairs : bound;
}

void orc_router_wide_sort(const uint32_t *experts, const float *weights, uint32_t picks, uint32_t live_rows,
                          uint32_t row_count, uint32_t expert_count, const uint64_t *expert_offsets,
                          struct orc_wide_pair *pairs_out, struct orc_wide_run *runs_out,
                          struct orc_wide_tile *tiles_out)
{
    uint32_t placed = 0, tile = 0;
    memset(tiles_out, 0, (size_t)orc_router_wide_tile_count(row_count, picks, expert_count) * sizeof *tiles_out);
    for (uint32_t expert = 0; expert < expert_count; expert++) {
        runs_out[expert].first_pair = placed;
        for (uint32_t pair = 0; pair < live_rows * picks; pair++) { /* rows ascending, then slots */
            if (experts[pair] == expert) {
                pairs_out[placed].pair_index = pair;
                pairs_out[placed].route_weight = weights[pair];
                placed++;
            }
        }
        runs_out[expert].pair_count = placed - runs_out[expert].first_pair;
        for (uint32_t taken = 0; taken < runs_out[expert].pair_count; taken += ORC_TILE_PAIRS, tile++) {
            const uint32_t left = runs_out[expert].pair_count - taken;
            tiles_out[tile].gate_offset = expert_offsets[expert * 3u + 0u];
            tiles_out[tile].up_offset = expert_offsets[expert * 3u + 1u];
            tiles_out[tile].down_offset = expert_offsets[expert * 3u + 2u];
            tiles_out[tile].first_pair = runs_out[expert].first_pair + taken;
            tiles_out[tile].pair_count = left < ORC_TILE_PAIRS ? left : ORC_TILE_PAIRS;
        }
    }
}

void orc_router_wide_jobs(const uint32_t *experts, const float *weights, uint32_t picks, uint32_t live_rows,
                          uint32_t row_count, uint32_t expert_count, const uint64_t *expert_offsets,
                          struct orc_job *jobs_out)
{
    uint32_t first_job = 0;
    memset(jobs_out, 0, (size_t)orc_router_wide_job_count(row_count, picks, expert_count) * sizeof *jobs_out);
    for (uint32_t expert = 0; expert < expert_count; expert++) {
        uint32_t taken = 0;
        for (uint32_t pair = 0; pair < live_rows * picks; pair++) {
            if (experts[pair] != expert) {
                continue;
            }
            struct orc_job *job = &jobs_out[first_job + taken / ORC_JOB_ROWS];
            job->gate_offset = expert_offsets[expert * 3u + 0u];
            job->up_offset = expert_offsets[expert * 3u + 1u];
            job->down_offset = expert_offsets[expert * 3u + 2u];
            job->expert = expert;
            job->pair_index[job->row_count] = pair;
            job->route_weight[job->row_count] = weights[pair];
            job->row_count++;
            taken++;
        }
        first_job += (taken + ORC_JOB_ROWS - 1u) / ORC_JOB_ROWS;
    }
}

/* the steps a card runs as router_projection and router_select_entry, all rows of a step */
void orc_router_route(const uint16_t *x_bf16, const uint16_t *w_bf16, const float *bias, uint32_t rows, uint32_t hidden,
                      uint32_t experts, uint32_t picks, int affinity_kind, int reference_order, float route_scale,
                      float *affinities_out, uint32_t *experts_out, float *weights_out)
{
    float *scores = malloc((size_t)rows * experts * sizeof *scores);
    orc_router_projection(x_bf16, w_bf16, rows, hidden, experts, scores);
    for (size_t index = 0; index < (size_t)rows * experts; index++) {
        scores[index] = orc_router_affinity(scores[index], affinity_kind);
    }
    for (uint32_t row = 0; row < rows; row++) {
        orc_router_select(scores + (size_t)row * experts, bias, experts, picks, reference_order, route_scale,
                          experts_out + (size_t)row * picks, weights_out + (size_t)row * picks);
    }
    if (affinities_out != NULL) {
        memcpy(affinities_out, scores, (size_t)rows * experts * sizeof *scores);
    }
    free(scores);
}
