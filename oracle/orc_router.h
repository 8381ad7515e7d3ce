/*
 * orc_router.h -- CPU oracle of the router: projection, affinity, top-k choice, job table, wide (prefill) sort.
 *
 * TEST INFRASTRUCTURE: checker of tests/, of the smoke run and of the benchmark's CPU baseline. Never the
 * product path.
 *
 * Restated from (paths relative to the reference tree):
 *   projection order            source/kernel_official_router_projection.cu:33-57 (32 strided fma chains, then a
 *                               halving fold 16, 8, 4, 2, 1)
 *   affinity sqrt(softplus)     include/anemone/router_records.h:8-14; source/kernel_router.cu:53-62
 *   key order of the top-k      source/kernel_router.cuh:35-44 (NaN above every number, -0 below +0, the lower
 *                               expert first among equals); tests/router_reference.c:139-151
 *   slots, weights              source/kernel_router.cuh:48-117; include/anemone/router_records.h:14-21
 *   job table                   include/anemone/linear_records.h:231-253; source/kernel_router.cuh:127-202
 *   wide sort, tiles, jobs      include/anemone/router_records.h:33-47; tests/router_reference.c:270-345
 *
 * The expert count E, the picks per row P, the route scale and the affinity kind are parameters here (the
 * reference fixes 384 / 6 / 1.5 / sqrt-softplus at compile time). Affinity kind 1 (sigmoid) has no counterpart
 * in the reference: closed form only.
 *
 * exp, log1p are fixed sequences of binary32 operations (orc_expf of orc_exl3.h, orc_log1pf here) so that a card
 * running the same sequence produces the same affinity bits and therefore the same expert ids; each is pinned
 * against libm within 2 ulp, and the affinity against the reference's 25-digit values within its own 4-ulp bar
 * (tests/router_reference.h:52).
 */
#ifndef ORC_ROUTER_H
#define ORC_ROUTER_H

#include <stdint.h>

#define ORC_AFFINITY_SQRT_SOFTPLUS 0
#define ORC_AFFINITY_SIGMOID 1
#define ORC_JOB_ROWS 8u
#define ORC_TILE_PAIRS 64u

struct orc_job { /* 96 bytes: include/anemone/linear_records.h:245-253 */
    uint64_t gate_offset, up_offset, down_offset;
    uint32_t row_count, expert;
    uint32_t pair_index[ORC_JOB_ROWS];
    float route_weight[ORC_JOB_ROWS];
};
struct orc_wide_pair { /* 8 bytes */
    uint32_t pair_index;
    float route_weight;
};
struct orc_wide_run { /* 8 bytes */
    uint32_t first_pair, pair_count;
};
struct orc_wide_tile { /* 32 bytes */
    uint64_t gate_offset, up_offset, down_offset;
    uint32_t first_pair, pair_count;
};

float orc_log1pf(float y); /* 0 <= y <= 1 */
float orc_router_affinity(float score, int kind);

/* scores [rows][experts] = W x: x bf16 [rows][hidden], W bf16 [experts][hidden] */
void orc_router_projection(const uint16_t *x_bf16, const uint16_t *w_bf16, uint32_t rows, uint32_t hidden,
                           uint32_t experts, float *scores_out);

/* one row: experts_out / weights_out [picks] by slot (ascending expert) */
void orc_router_select(const float *affinities, const float *bias, uint32_t experts, uint32_t picks,
                       int reference_order, float route_scale, uint32_t *experts_out, float *weights_out);

/* every row of a step in one call: projection, affinities (affinities_out [rows][experts], may be NULL) and the select
 * of each row; experts_out / weights_out [rows][picks] */
void orc_router_route(const uint16_t *x_bf16, const uint16_t *w_bf16, const float *bias, uint32_t rows, uint32_t hidden,
                      uint32_t experts, uint32_t picks, int affinity_kind, int reference_order, float route_scale,
                      float *affinities_out, uint32_t *experts_out, float *weights_out);

/* the thin job table: row_count * picks entries, every byte written */
void orc_router_jobs(const uint32_t *experts, const float *weights, uint32_t picks, uint32_t live_rows,
                     uint32_t row_count, uint32_t expert_count, const uint64_t *expert_offsets,
                     struct orc_job *jobs_out);

uint32_t orc_router_wide_tile_count(uint32_t row_count, uint32_t picks, uint32_t expert_count);
uint32_t orc_router_wide_job_count(uint32_t row_count, uint32_t picks, uint32_t expert_count);
/* pairs_out: live_rows * picks entries; runs_out: expert_count; tiles_out: every tile of row_count */
void orc_router_wide_sort(const uint32_t *experts, const float *weights, uint32_t picks, uint32_t live_rows,
                          uint32_t row_count, uint32_t expert_count, const uint64_t *expert_offsets,
                          struct orc_wide_pair *pairs_out, struct orc_wide_run *runs_out,
                          struct orc_wide_tile *tiles_out);
void orc_router_wide_jobs(const uint32_t *experts, const float *weights, uint32_t picks, uint32_t live_rows,
                          uint32_t row_count, uint32_t expert_count, const uint64_t *expert_offsets,
                          struct orc_job *jobs_out);

#endif
