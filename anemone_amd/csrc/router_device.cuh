/*
 * router_device.cuh -- the router's select as device code: the affinity, a row's top-k choice with its route weights, and
 * the whole select of a thin step (affinities, choices, job table) by one block, shared by router_select_entry and the
 * fused FFN front. Definitions: include/anemone/router_records.h:8-31, source/kernel_router.cuh of the reference.
 */
#ifndef ROUTER_DEVICE_CUH
#define ROUTER_DEVICE_CUH

#include "exl3_device.cuh" /* det_expf, bf16_to_float */

#define SELECT_THREADS (LINEAR_MAXIMUM_ROWS * WAVE) /* a wavefront for each row */
#define JOB_WORDS (sizeof(struct expert_job_record) / 4u)

__device__ static __forceinline__ float det_log1pf(float y) /* 0 <= y <= 1 */
{
    const float u = __fadd_rn(1.0f, y);
    const float c = __fsub_rn(y, __fsub_rn(u, 1.0f));
    float m = u, e = 0.0f;
    if (u > 1.41421354f) {
        m = __fmul_rn(u, 0.5f);
        e = 1.0f;
    }
    const float f = __fsub_rn(m, 1.0f);
    const float s = __fdiv_rn(f, __fadd_rn(2.0f, f));
    const float z = __fmul_rn(s, s);
    float r = __fmaf_rn(z, 0.222222224f, 0.285714298f);
    r = __fmaf_rn(r, z, 0.400000006f);
    r = __fmaf_rn(r, z, 0.666666687f);
    r = __fmul_rn(r, z);
    const float hfsq = __fmul_rn(__fmul_rn(0.5f, f), f);
    const float log_m = __fsub_rn(f, __fsub_rn(hfsq, __fmul_rn(s, __fadd_rn(hfsq, r))));
    const float low = __fmaf_rn(e, 9.05800061e-06f, __fdiv_rn(c, u));
    return __fmaf_rn(e, 0.693138123f, __fadd_rn(log_m, low));
}

__device__ static __forceinline__ float router_affinity(float score, uint32_t kind)
{
    if (kind == ROUTER_AFFINITY_SIGMOID) {
        return __fdiv_rn(1.0f, __fadd_rn(1.0f, det_expf(-score)));
    }
    if (score != score) {
        return score;
    }
    if (score > 20.0f) {
        return sqrtf(score); /* correctly rounded: the compiler default for float32 sqrt and divide */
    }
    const float positive = score > 0.0f ? score : 0.0f;
    return sqrtf(__fadd_rn(positive, det_log1pf(det_expf(-fabsf(score)))));
}

__device__ static __forceinline__ uint64_t router_key(float biased, uint32_t expert)
{
    const uint32_t bits = __float_as_uint(biased);
    const uint32_t ordered = biased != biased ? 0xFFFFFFFFu : (bits & 0x80000000u) != 0u ? ~bits : bits | 0x80000000u;
    return ((uint64_t)ordered << 32) | (uint32_t)~expert;
}

/* The largest 64-bit key of a wavefront, in every lane: a data-parallel-primitive scan (shift by 1, 2, 4, 8 inside
 * rows of 16 lanes, then the row broadcasts), no LDS round trip; lane 63 holds the maximum. */
template <int control, int row_mask>
__device__ static __forceinline__ uint64_t dpp_max_step(uint64_t value)
{
    const uint32_t low = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)value, control, row_mask, 0xF, false);
    const uint32_t high = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(value >> 32), control, row_mask, 0xF, false);
    const uint64_t other = ((uint64_t)high << 32) | low; /* lanes without a source keep 0, below every key */
    return other > value ? other : value;
}

__device__ static __forceinline__ uint64_t wave_max_u64(uint64_t value)
{
    value = dpp_max_step<0x111, 0xF>(value); /* row_shr:1 */
    value = dpp_max_step<0x112, 0xF>(value); /* row_shr:2 */
    value = dpp_max_step<0x114, 0xF>(value); /* row_shr:4 */
    value = dpp_max_step<0x118, 0xF>(value); /* row_shr:8: lane 15 of a row holds the row's maximum */
    value = dpp_max_step<0x142, 0xA>(value); /* row_bcast:15 into rows 1 and 3 */
    value = dpp_max_step<0x143, 0xC>(value); /* row_bcast:31 into rows 2 and 3 */
    const uint32_t low = __builtin_amdgcn_readlane((int)(uint32_t)value, 63);
    const uint32_t high = __builtin_amdgcn_readlane((int)(uint32_t)(value >> 32), 63);
    return ((uint64_t)high << 32) | low;
}

/* One row by one wavefront: its picks by slot and their weights, written by lane 0. */
/* bias: the lane's values of the experts lane, lane + 64, ... (asked for before the affinities are there) */
__device__ static void router_row(const float *affinities, const float (&bias)[ROUTER_MOST_EXPERTS / WAVE], uint32_t lane, uint32_t experts,
                                  uint32_t picks, uint32_t reference_order, float route_scale, uint32_t *chosen,
                                  float *weights)
{
    uint64_t keys[ROUTER_MOST_EXPERTS / WAVE];
    uint32_t picked_experts[ROUTER_MOST_PICKS];
    float picked[ROUTER_MOST_PICKS];
    const uint32_t places = experts / WAVE;
#pragma unroll
    for (uint32_t place = 0; place < ROUTER_MOST_EXPERTS / WAVE; place++) {
        const uint32_t expert = lane + place * WAVE;
        keys[place] = place < places ? router_key(__fadd_rn(affinities[expert], bias[place]), expert) : 0ull;
    }
#pragma unroll
    for (uint32_t pick = 0; pick < ROUTER_MOST_PICKS; pick++) {
        if (pick < picks) {
            uint64_t best = 0ull; /* below every key: an ordered float32 is at least 0x007FFFFF */
#pragma unroll
            for (uint32_t place = 0; place < ROUTER_MOST_EXPERTS / WAVE; place++) {
                best = keys[place] > best ? keys[place] : best;
            }
            best = wave_max_u64(best);
#pragma unroll
            for (uint32_t place = 0; place < ROUTER_MOST_EXPERTS / WAVE; place++) {
                keys[place] = keys[place] == best ? 0ull : keys[place];
            }
            picked_experts[pick] = ~(uint32_t)best;
            picked[pick] = affinities[picked_experts[pick]];
        } else {
            picked_experts[pick] = 0xFFFFFFFFu;
            picked[pick] = 0.0f;
        }
    }
    float by_slot[ROUTER_MOST_PICKS];
    uint32_t expert_by_slot[ROUTER_MOST_PICKS];
#pragma unroll
    for (uint32_t slot = 0; slot < ROUTER_MOST_PICKS; slot++) {
        by_slot[slot] = 0.0f;
        expert_by_slot[slot] = 0u;
    }
#pragma unroll
    for (uint32_t pick = 0; pick < ROUTER_MOST_PICKS; pick++) {
        uint32_t slot = 0;
#pragma unroll
        for (uint32_t other = 0; other < ROUTER_MOST_PICKS; other++) {
            slot += picked_experts[other] < picked_experts[pick] ? 1u : 0u;
        }
#pragma unroll
        for (uint32_t target = 0; target < ROUTER_MOST_PICKS; target++) {
            if (pick < picks && target == slot) {
                by_slot[target] = picked[pick];
                expert_by_slot[target] = picked_experts[pick];
            }
        }
    }
    float sum = 0.0f;
#pragma unroll
    for (uint32_t slot = 0; slot < ROUTER_MOST_PICKS; slot++) {
        if (slot < picks) {
            sum = __fadd_rn(sum, by_slot[slot]);
        }
    }
    if (reference_order != 0u && picks == 6u) {
        sum = __fadd_rn(__fadd_rn(__fadd_rn(picked[0], picked[4]), picked[2]),
                        __fadd_rn(__fadd_rn(picked[1], picked[5]), picked[3]));
    }
    const float denominator = __fadd_rn(sum, 1e-20f);
    if (lane == 0u) {
#pragma unroll
        for (uint32_t slot = 0; slot < ROUTER_MOST_PICKS; slot++) {
            if (slot < picks) {
                chosen[slot] = expert_by_slot[slot];
                weights[slot] = __fmul_rn(__fdiv_rn(by_slot[slot], denominator), route_scale);
            }
        }
    }
}

/* what the select keeps in LDS */
struct router_select_lds {
    float affinities[LINEAR_MAXIMUM_ROWS * ROUTER_MOST_EXPERTS];
    float pair_weights[LINEAR_MAXIMUM_ROWS * ROUTER_MOST_PICKS];
    uint32_t pair_experts[LINEAR_MAXIMUM_ROWS * ROUTER_MOST_PICKS];
    uint32_t pair_is_first[LINEAR_MAXIMUM_ROWS * ROUTER_MOST_PICKS];
};

/* The select of a step of at most LINEAR_MAXIMUM_ROWS rows by one block of `threads` threads (whole wavefronts, at least
 * one; every thread of the block calls: barriers inside). */
__device__ static __forceinline__ void router_select_body(const struct router_select_arguments &arguments, unsigned char *arena,
                                                          uint32_t thread, uint32_t threads, struct router_select_lds &lds)
{
    float *affinities = lds.affinities, *pair_weights = lds.pair_weights;
    uint32_t *pair_experts = lds.pair_experts, *pair_is_first = lds.pair_is_first;
    const uint32_t experts = arguments.expert_count != 0u ? arguments.expert_count : ROUTER_DEFAULT_EXPERTS;
    const uint32_t picks = arguments.pick_count != 0u ? arguments.pick_count : ROUTER_DEFAULT_PICKS;
    const float scale = arguments.route_scale != 0.0f ? arguments.route_scale : ROUTER_DEFAULT_SCALE;
    const uint32_t step_rows = ((const struct step_block *)(arena + arguments.step_offset))->row_count;
    const uint32_t live_rows = step_rows < arguments.row_count ? step_rows : arguments.row_count;
    const uint32_t wave = thread / WAVE, lane = thread % WAVE;
    const uint32_t pair = thread, pair_count = live_rows * picks;
    /* the lane's bias values, asked for now: they arrive while the affinities are formed */
    float bias_of[ROUTER_MOST_EXPERTS / WAVE];
#pragma unroll
    for (uint32_t place = 0; place < ROUTER_MOST_EXPERTS / WAVE; place++) {
        bias_of[place] = lane + place * WAVE < experts ? ((const float *)(arena + arguments.bias_offset))[lane + place * WAVE] : 0.0f;
    }
    for (uint32_t index = thread; index < live_rows * experts; index += threads) {
        const float a = router_affinity(((const float *)(arena + arguments.scores_offset))[index], arguments.affinity_kind);
        affinities[index] = a;
        ((float *)(arena + arguments.affinities_offset))[index] = a;
    }
    __syncthreads();
    for (uint32_t row = wave; row < live_rows; row += threads / WAVE) { /* a wavefront a row (every row at once with eight wavefronts) */
        router_row(affinities + row * experts, bias_of, lane, experts, picks,
                   arguments.reference_order, scale, pair_experts + row * picks, pair_weights + row * picks);
    }
    __syncthreads();
    /* The job table: at most 64 pairs, one a lane of the first wavefront. A pair's column is the number of earlier
     * pairs of its expert, its job the number of distinct experts below its own, a job's rows the pairs of its expert:
     * counted over the other lanes' experts read lane by lane (no LDS round trip a step). */
    static_assert(LINEAR_MAXIMUM_ROWS * ROUTER_MOST_PICKS <= WAVE, "a step's pairs fit one wavefront");
    const bool mine = pair < pair_count;
    uint32_t used_jobs = 0, job = 0, rows = 0, column = 0;
    const uint32_t expert = mine ? pair_experts[pair] : 0xFFFFFFFFu; /* no expert: equal to none that is picked */
    if (wave == 0u) {
#pragma unroll
        for (uint32_t other = 0; other < WAVE; other++) {
            const uint32_t theirs = (uint32_t)__builtin_amdgcn_readlane((int)expert, (int)other);
            const bool same = theirs == expert;
            rows += same ? 1u : 0u;
            column += same && other < lane ? 1u : 0u;
        }
        const uint64_t firsts = __builtin_amdgcn_ballot_w64(mine && column == 0u); /* the first pair of every picked expert */
        used_jobs = (uint32_t)__builtin_popcountll(firsts);
#pragma unroll
        for (uint32_t other = 0; other < WAVE; other++) {
            const uint32_t theirs = (uint32_t)__builtin_amdgcn_readlane((int)expert, (int)other);
            job += ((firsts >> other) & 1u) != 0u && theirs < expert ? 1u : 0u;
        }
        if (lane == 0u) {
            pair_is_first[0] = used_jobs; /* for the wavefronts that clear the table's unused jobs */
        }
    }
    __syncthreads();
    used_jobs = pair_is_first[0];
    struct expert_job_record *jobs = (struct expert_job_record *)(arena + arguments.jobs_offset);
    if (mine) {
        jobs[job].pair_index[column] = pair;
        jobs[job].route_weight[column] = pair_weights[pair];
    }
    if (mine && column == 0u) {
        const uint64_t *offsets = (const uint64_t *)(arena + arguments.expert_offsets_offset) + (uint64_t)expert * MODEL_EXPERT_MATRICES;
        jobs[job].gate_offset = offsets[0];
        jobs[job].up_offset = offsets[1];
        jobs[job].down_offset = offsets[2];
        jobs[job].row_count = rows;
        jobs[job].expert = expert;
        for (uint32_t unused = rows; unused < LINEAR_MAXIMUM_ROWS; unused++) {
            jobs[job].pair_index[unused] = 0u;
            jobs[job].route_weight[unused] = 0.0f;
        }
    }
    uint32_t *empty_words = (uint32_t *)(jobs + used_jobs);
    const uint32_t empty_count = (arguments.row_count * picks - used_jobs) * JOB_WORDS;
    for (uint32_t word = thread; word < empty_count; word += threads) {
        empty_words[word] = 0u;
    }
}

#endif
