/*
 * sort_device.cuh -- what the sorts of pairs by expert share (the router's wide select and the prefill form of the
 * EXL3 experts): a block's picked experts into LDS, its picks counted an expert, every pick's place, and a block-wide
 * exclusive prefix sum. The only atomic operations are integer additions in LDS that count (the same sums in any order);
 * a pick's place among its expert's is formed from the lanes' ballots, in row order.
 */
#ifndef SORT_DEVICE_CUH
#define SORT_DEVICE_CUH

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "anemone_records.h"

/* the picked experts of the live rows of block `block` of ROUTER_SORT_ROWS rows, into LDS; returns their number */
__device__ static __forceinline__ uint32_t sort_block_picks(const struct router_pick *all_picks, uint32_t picks_per_row,
                                                            uint32_t block, uint32_t live_rows, uint32_t *experts_out)
{
    const uint32_t first_row = block * ROUTER_SORT_ROWS;
    const uint32_t rows = live_rows <= first_row ? 0u : live_rows - first_row < ROUTER_SORT_ROWS ? live_rows - first_row : ROUTER_SORT_ROWS;
    const struct router_pick *picks = all_picks + (uint64_t)first_row * picks_per_row;
    for (uint32_t index = threadIdx.x; index < rows * picks_per_row; index += blockDim.x) {
        experts_out[index] = picks[index].expert;
    }
    return rows * picks_per_row;
}

#define SORT_WAVE 64u
#define SORT_MOST_WAVES 8u /* of a block of the sorts: 512 threads */

/* The block's picks of every expert: histogram[expert] in LDS. Integer additions in LDS: the same sums whatever their
 * order. The whole block calls it (barriers inside); block_experts is complete before the call. */
__device__ static __forceinline__ void sort_count_picks(const uint32_t *block_experts, uint32_t pairs, uint32_t experts, uint32_t *histogram)
{
    for (uint32_t expert = threadIdx.x; expert < experts; expert += blockDim.x) {
        histogram[expert] = 0u;
    }
    __syncthreads();
    for (uint32_t index = threadIdx.x; index < pairs; index += blockDim.x) {
        __hip_atomic_fetch_add(&histogram[block_experts[index]], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __syncthreads();
}

/* The lanes of the wavefront that hold the same word as this lane, among the lanes where `live` (a lane that is not live
 * gets 0): one ballot a bit of the words, `bits` of them. */
__device__ static __forceinline__ uint64_t sort_equal_lanes(uint32_t word, bool live, uint32_t bits)
{
    uint64_t equal = __builtin_amdgcn_ballot_w64(live);
    for (uint32_t bit = 0; bit < bits; bit++) {
        const bool set = ((word >> bit) & 1u) != 0u;
        const uint64_t holders = __builtin_amdgcn_ballot_w64(live && set);
        equal &= set ? holders : ~holders;
    }
    return live ? equal : 0ull;
}

/* Every pick's place, in LDS: place_of[index] = first[expert] + the picks of the same expert before it in the block.
 * Wavefront w of the block's `waves` takes the picks [w share, (w + 1) share) in order, 64 at a time: a pick's place is
 * its expert's cursor plus the lanes below it that hold the same expert (ballots over the expert's bits: no lane waits
 * for another's answer), and the first of them moves the cursor on. A wavefront's cursors begin behind the picks of the
 * wavefronts before it, which a histogram a wavefront (LDS, integer additions) and a walk over the wavefronts by a thread
 * an expert give. first: LDS, experts words (kept); cursors: LDS, SORT_MOST_WAVES x experts words. The whole block
 * calls it (barriers inside). */
__device__ static __forceinline__ void sort_place_picks(const uint32_t *block_experts, uint32_t pairs, uint32_t experts, const uint32_t *first,
                                                        uint32_t *cursors, uint32_t *place_of)
{
    const uint32_t lane = threadIdx.x % SORT_WAVE, wave = threadIdx.x / SORT_WAVE, waves = blockDim.x / SORT_WAVE;
    const uint32_t share = ((pairs + waves - 1u) / waves + SORT_WAVE - 1u) / SORT_WAVE * SORT_WAVE; /* whole groups of 64 a wavefront */
    const uint32_t begin = wave * share < pairs ? wave * share : pairs, end = begin + share < pairs ? begin + share : pairs;
    for (uint32_t at = threadIdx.x; at < waves * experts; at += blockDim.x) {
        cursors[at] = 0u;
    }
    __syncthreads();
    for (uint32_t index = begin + lane; index < end; index += SORT_WAVE) {
        __hip_atomic_fetch_add(&cursors[wave * experts + block_experts[index]], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __syncthreads();
    for (uint32_t expert = threadIdx.x; expert < experts; expert += blockDim.x) {
        uint32_t place = first[expert];
        for (uint32_t other = 0; other < waves; other++) {
            const uint32_t count = cursors[other * experts + expert];
            cursors[other * experts + expert] = place;
            place += count;
        }
    }
    __syncthreads();
    uint32_t bits = 0;
    while ((1u << bits) < experts) {
        bits++;
    }
    uint32_t *mine = cursors + wave * experts;
    for (uint32_t base = begin; base < end; base += SORT_WAVE) {
        const uint32_t index = base + lane;
        const bool live = index < end;
        const uint32_t expert = live ? block_experts[index] : 0u;
        const uint64_t equal = sort_equal_lanes(expert, live, bits);
        const uint32_t below = __builtin_amdgcn_mbcnt_hi((uint32_t)(equal >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)equal, 0u));
        if (live) {
            const uint32_t cursor = mine[expert]; /* every lane of an expert reads it before the first of them writes it: LDS serves
                                                    a wavefront's instructions in their order */
            place_of[index] = cursor + below;
            if (below == 0u) {
                mine[expert] = cursor + (uint32_t)__builtin_popcountll(equal);
            }
        }
    }
    __syncthreads();
}

/* exclusive prefix sums of values[0 .. count) in LDS, count <= ROUTER_MOST_EXPERTS, by the whole block; total returned */
__device__ static __forceinline__ uint32_t block_exclusive_scan(uint32_t *values, uint32_t count, uint32_t *scratch)
{
    /* count is small (at most 512): Hillis-Steele over two buffers */
    uint32_t *from = values, *to = scratch;
    for (uint32_t step = 1; step < count; step *= 2u) {
        for (uint32_t i = threadIdx.x; i < count; i += blockDim.x) {
            to[i] = from[i] + (i >= step ? from[i - step] : 0u);
        }
        __syncthreads();
        uint32_t *swap = from;
        from = to;
        to = swap;
    }
    const uint32_t total = count == 0u ? 0u : from[count - 1u];
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < count; i += blockDim.x) {
        to[i] = i == 0u ? 0u : from[i - 1u];
    }
    __syncthreads();
    if (to != values) {
        for (uint32_t i = threadIdx.x; i < count; i += blockDim.x) {
            values[i] = to[i];
        }
        __syncthreads();
    }
    return total;
}

#endif
