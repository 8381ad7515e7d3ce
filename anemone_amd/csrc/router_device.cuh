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

/* 1 / (1 + e^(-score)): the bits of __fdiv_rn(1.0f, __fadd_rn(1.0f, det_expf(-score))) for every float32 score, without
 * det_expf's three tests (see det_silu: the sequence's argument held inside [-104, 89.5] gives the same sums with 1); a
 * not-a-number, which the clamp would lose, is passed through by a select. The library's arithmetic_selfcheck kernel
 * compares the two over all 2^32 scores. */
__device__ static __forceinline__ float det_sigmoid(float score)
{
    const float x = __builtin_amdgcn_fmed3f(-score, -104.0f, 89.5f);
    const float value = __fdiv_rn(1.0f, __fadd_rn(1.0f, det_exp_sequence(x)));
    return score != score ? score : value;
}

__device__ static __forceinline__ float router_affinity(float score, uint32_t kind)
{
    if (kind == ROUTER_AFFINITY_SIGMOID) {
        return det_sigmoid(score);
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

/* A biased affinity as an unsigned word that orders as the select orders values: a not-a-number above everything, then
 * the numbers from +infinity down to -infinity, which is 0x007FFFFF: 0 is below every key. Among equal keys the select
 * takes the lowest expert (include/anemone/router_records.h:12-16 of the reference). */
__device__ static __forceinline__ uint32_t router_key(float biased)
{
    const uint32_t bits = __float_as_uint(biased);
    return biased != biased ? 0xFFFFFFFFu : (bits & 0x80000000u) != 0u ? ~bits : bits | 0x80000000u;
}

/* The largest (smallest) word of a wavefront, in every lane: a data-parallel-primitive scan (shift by 1, 2, 4, 8 inside
 * rows of 16 lanes, then the row broadcasts), no LDS round trip; lane 63 holds the result. A lane without a source takes
 * the operation's neutral word. */
template <bool LARGEST, int control, int row_mask>
__device__ static __forceinline__ uint32_t dpp_extreme_step(uint32_t value)
{
    const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(LARGEST ? 0 : -1, (int)value, control, row_mask, 0xF, false);
    return LARGEST ? (other > value ? other : value) : (other < value ? other : value);
}

template <bool LARGEST>
__device__ static __forceinline__ uint32_t wave_extreme_u32(uint32_t value)
{
    value = dpp_extreme_step<LARGEST, 0x111, 0xF>(value); /* row_shr:1 */
    value = dpp_extreme_step<LARGEST, 0x112, 0xF>(value); /* row_shr:2 */
    value = dpp_extreme_step<LARGEST, 0x114, 0xF>(value); /* row_shr:4 */
    value = dpp_extreme_step<LARGEST, 0x118, 0xF>(value); /* row_shr:8: lane 15 of a row holds the row's */
    value = dpp_extreme_step<LARGEST, 0x142, 0xA>(value); /* row_bcast:15 into rows 1 and 3 */
    value = dpp_extreme_step<LARGEST, 0x143, 0xC>(value); /* row_bcast:31 into rows 2 and 3 */
    return (uint32_t)__builtin_amdgcn_readlane((int)value, 63);
}

#define ROUTER_PLACES (ROUTER_MOST_EXPERTS / WAVE) /* experts a lane holds at most: lane, lane + 64, ... */

/* One row by one wavefront. keys: the lane's experts' keys (PLACES of them: the row's experts are 64 PLACES or fewer; 0
 * past them); affinities: the row's, in LDS, written by this wavefront. Lane p < picks ends with pick p: its expert, its
 * slot (the picks in ascending expert order) and its route weight. The work of a pick is two scans of the wavefront (the
 * largest key; the lowest expert that holds it) and a dozen vector instructions; the slots and the sum in slot order are
 * formed by the picks' lanes side by side: a wavefront runs one instruction at a time, so the row's time is its
 * instruction count. */
template <uint32_t PLACES>
__device__ static __forceinline__ void router_row(const float *affinities, uint32_t (&keys)[PLACES], uint32_t lane, uint32_t picks,
                                                  uint32_t reference_order, float route_scale, uint32_t &expert_out, uint32_t &slot_out,
                                                  float &weight_out)
{
    uint32_t expert = 0xFFFFFFFFu; /* no pick: above every expert */
    float value = 0.0f;
    for (uint32_t pick = 0; pick < picks; pick++) {
        uint32_t best = 0u;
#pragma unroll
        for (uint32_t place = 0; place < PLACES; place++) {
            best = keys[place] > best ? keys[place] : best;
        }
        best = wave_extreme_u32<true>(best);
        uint32_t candidate = 0xFFFFFFFFu; /* the lane's lowest expert that holds it */
#pragma unroll
        for (uint32_t place = PLACES; place-- > 0u;) {
            candidate = keys[place] == best ? lane + place * WAVE : candidate;
        }
        const uint32_t winner = wave_extreme_u32<false>(candidate);
#pragma unroll
        for (uint32_t place = 0; place < PLACES; place++) {
            keys[place] = lane + place * WAVE == winner ? 0u : keys[place];
        }
        const float taken = affinities[winner]; /* the same address in every lane */
        expert = lane == pick ? winner : expert;
        value = lane == pick ? taken : value;
    }
    uint32_t slot = 0;
    for (uint32_t other = 0; other < picks; other++) {
        slot += (uint32_t)__builtin_amdgcn_readlane((int)expert, (int)other) < expert ? 1u : 0u;
    }
    float sum = 0.0f;
    if (reference_order != 0u && picks == 6u) {
        const float p0 = __shfl(value, 0), p1 = __shfl(value, 1), p2 = __shfl(value, 2), p3 = __shfl(value, 3), p4 = __shfl(value, 4),
                    p5 = __shfl(value, 5);
        sum = __fadd_rn(__fadd_rn(__fadd_rn(p0, p4), p2), __fadd_rn(__fadd_rn(p1, p5), p3));
    } else {
        for (uint32_t at = 0; at < picks; at++) { /* in slot order from +0 */
            const uint64_t holder = __builtin_amdgcn_ballot_w64(lane < picks && slot == at);
            sum = __fadd_rn(sum, __shfl(value, (int)__builtin_ctzll(holder)));
        }
    }
    expert_out = expert;
    slot_out = slot;
    weight_out = __fmul_rn(__fdiv_rn(value, __fadd_rn(sum, 1e-20f)), route_scale);
}

/* a row from its scores on: the affinities (LDS and memory), the keys, the picks */
template <uint32_t PLACES>
__device__ static __forceinline__ void router_row_of_scores(const float (&scores)[ROUTER_PLACES], const float (&bias)[ROUTER_PLACES],
                                                            float *affinities, float *affinities_out, uint32_t lane, uint32_t affinity_kind,
                                                            uint32_t picks, uint32_t reference_order, float route_scale, uint32_t &expert_out,
                                                            uint32_t &slot_out, float &weight_out)
{
    uint32_t keys[PLACES];
#pragma unroll
    for (uint32_t place = 0; place < PLACES; place++) {
        const float a = router_affinity(scores[place], affinity_kind);
        affinities[lane + place * WAVE] = a;
        affinities_out[lane + place * WAVE] = a;
        keys[place] = router_key(__fadd_rn(a, bias[place]));
    }
    router_row<PLACES>(affinities, keys, lane, picks, reference_order, route_scale, expert_out, slot_out, weight_out);
}

/* experts: a multiple of 64 up to ROUTER_MOST_EXPERTS; lanes hold 4 or 8 places (the instance of 4 runs half the vector
 * instructions a pick) */
__device__ static __forceinline__ void router_row_any(const float (&scores)[ROUTER_PLACES], const float (&bias)[ROUTER_PLACES], uint32_t experts,
                                                      float *affinities, float *affinities_out, uint32_t lane, uint32_t affinity_kind,
                                                      uint32_t picks, uint32_t reference_order, float route_scale, uint32_t &expert_out,
                                                      uint32_t &slot_out, float &weight_out)
{
    static_assert(ROUTER_PLACES == 8u, "two instances: up to 256 experts, up to 512");
    if (experts == 4u * WAVE) {
        router_row_of_scores<4u>(scores, bias, affinities, affinities_out, lane, affinity_kind, picks, reference_order, route_scale, expert_out,
                                 slot_out, weight_out);
        return;
    }
    /* any other count: the places past the row's experts hold key 0 and are never taken */
    uint32_t keys[ROUTER_PLACES];
#pragma unroll
    for (uint32_t place = 0; place < ROUTER_PLACES; place++) {
        keys[place] = 0u;
        if (place * WAVE < experts) {
            const float a = router_affinity(scores[place], affinity_kind);
            affinities[lane + place * WAVE] = a;
            affinities_out[lane + place * WAVE] = a;
            keys[place] = router_key(__fadd_rn(a, bias[place]));
        }
    }
    router_row<ROUTER_PLACES>(affinities, keys, lane, picks, reference_order, route_scale, expert_out, slot_out, weight_out);
}

/* what the select keeps in LDS */
struct router_select_lds {
    float affinities[LINEAR_MAXIMUM_ROWS * ROUTER_MOST_EXPERTS];
    float pair_weights[LINEAR_MAXIMUM_ROWS * ROUTER_MOST_PICKS];
    uint32_t pair_experts[LINEAR_MAXIMUM_ROWS * ROUTER_MOST_PICKS];
    uint32_t rows_of[ROUTER_MOST_EXPERTS];     /* bit r: row r picked the expert */
    uint32_t picked_words[ROUTER_MOST_EXPERTS / 32u]; /* bit e % 32 of word e / 32: some row picked expert e */
};

/* The select of a step of at most LINEAR_MAXIMUM_ROWS rows by one block of `threads` threads (whole wavefronts, at least
 * one; every thread of the block calls: one barrier inside). A wavefront takes a row from its scores to its picks; the
 * job table then needs of a pair only its expert's rows (a word of bits that the rows' wavefronts set in LDS: integer
 * or, the same whatever the order) and the picked experts below its own (a bit an expert). */
__device__ static __forceinline__ void router_select_body(const struct router_select_arguments &arguments, unsigned char *arena,
                                                          uint32_t thread, uint32_t threads, struct router_select_lds &lds)
{
    const uint32_t experts = arguments.expert_count != 0u ? arguments.expert_count : ROUTER_DEFAULT_EXPERTS;
    const uint32_t picks = arguments.pick_count != 0u ? arguments.pick_count : ROUTER_DEFAULT_PICKS;
    const float scale = arguments.route_scale != 0.0f ? arguments.route_scale : ROUTER_DEFAULT_SCALE;
    const uint32_t wave = thread / WAVE, lane = thread % WAVE, waves = threads / WAVE, places = experts / WAVE;
    const float *all_scores = (const float *)(arena + arguments.scores_offset);
    /* asked for together: the step's rows, the lane's bias values, and the scores of the wavefront's first row (inside the
     * scores' array whether the row is live or not) */
    const uint32_t step_rows = ((const struct step_block *)(arena + arguments.step_offset))->row_count;
    float bias_of[ROUTER_PLACES], scores[ROUTER_PLACES];
    const uint32_t first_row = wave < arguments.row_count ? wave : 0u;
#pragma unroll
    for (uint32_t place = 0; place < ROUTER_PLACES; place++) {
        bias_of[place] = place < places ? ((const float *)(arena + arguments.bias_offset))[lane + place * WAVE] : 0.0f;
        scores[place] = place < places ? all_scores[first_row * experts + lane + place * WAVE] : 0.0f;
    }
    for (uint32_t expert = thread; expert < ROUTER_MOST_EXPERTS; expert += threads) {
        lds.rows_of[expert] = 0u;
    }
    if (thread < ROUTER_MOST_EXPERTS / 32u) {
        lds.picked_words[thread] = 0u;
    }
    __syncthreads(); /* the zeros are there before any row sets a bit */
    const uint32_t live_rows = step_rows < arguments.row_count ? step_rows : arguments.row_count;
    for (uint32_t row = wave; row < live_rows; row += waves) { /* a wavefront a row (every row at once with eight wavefronts) */
        if (row != wave) {
#pragma unroll
            for (uint32_t place = 0; place < ROUTER_PLACES; place++) {
                scores[place] = place < places ? all_scores[row * experts + lane + place * WAVE] : 0.0f;
            }
        }
        uint32_t my_expert, my_slot;
        float my_weight;
        router_row_any(scores, bias_of, experts, lds.affinities + row * experts, (float *)(arena + arguments.affinities_offset) + row * experts, lane,
                       arguments.affinity_kind, picks, arguments.reference_order, scale, my_expert, my_slot, my_weight);
        if (lane < picks) { /* lane p holds pick p */
            lds.pair_experts[row * picks + my_slot] = my_expert;
            lds.pair_weights[row * picks + my_slot] = my_weight;
            __hip_atomic_fetch_or(&lds.rows_of[my_expert], 1u << row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            __hip_atomic_fetch_or(&lds.picked_words[my_expert / 32u], 1u << (my_expert % 32u), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    }
    __syncthreads();
    /* The job table: at most 64 pairs, one a lane of the first wavefront. A pair's column is the number of lower rows
     * that picked its expert, its job the number of picked experts below its own, a job's rows the rows that picked its
     * expert. */
    static_assert(LINEAR_MAXIMUM_ROWS * ROUTER_MOST_PICKS <= WAVE, "a step's pairs fit one wavefront");
    const uint32_t pair = thread, pair_count = live_rows * picks;
    const bool mine = pair < pair_count;
    const uint32_t expert = mine ? lds.pair_experts[pair] : 0u;
    uint32_t used_jobs = 0, job = 0;
    for (uint32_t word = 0; word < experts / 32u; word++) {
        const uint32_t bits = lds.picked_words[word]; /* the same address in every lane */
        used_jobs += (uint32_t)__builtin_popcount(bits);
        const uint32_t below = word < expert / 32u ? 0xFFFFFFFFu : word == expert / 32u ? (1u << (expert % 32u)) - 1u : 0u;
        job += (uint32_t)__builtin_popcount(bits & below);
    }
    struct expert_job_record *jobs = (struct expert_job_record *)(arena + arguments.jobs_offset);
    if (mine) {
        const uint32_t row = pair / picks, holders = lds.rows_of[expert];
        const uint32_t rows = (uint32_t)__builtin_popcount(holders), column = (uint32_t)__builtin_popcount(holders & ((1u << row) - 1u));
        jobs[job].pair_index[column] = pair;
        jobs[job].route_weight[column] = lds.pair_weights[pair];
        if (column == 0u) {
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
    }
    uint32_t *empty_words = (uint32_t *)(jobs + used_jobs);
    const uint32_t empty_count = (arguments.row_count * picks - used_jobs) * JOB_WORDS;
    for (uint32_t word = thread; word < empty_count; word += threads) {
        empty_words[word] = 0u;
    }
}

#endif
