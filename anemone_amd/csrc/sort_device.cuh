/*
 * sort_device.cuh -- what the sorts of pairs by expert share (the router's wide select and the prefill form of the
 * EXL3 experts): a block's picked experts into LDS, and a block-wide exclusive prefix sum. No atomic operation
 * anywhere: a thread owns an expert and walks the block's picks in row order.
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

/* Every pick of a block in order, 32 at a time (eight 16-byte LDS reads in flight, so that a walk waits for LDS once
 * in 32 picks), then eight at a time, then one: visit(index, expert). block_experts is 16-byte aligned. */
template <typename Visit>
__device__ static __forceinline__ void sort_walk_picks(const uint32_t *block_experts, uint32_t pairs, Visit visit)
{
    typedef __attribute__((ext_vector_type(4))) uint32_t four_words;
    uint32_t index = 0;
    for (; index + 32u <= pairs; index += 32u) {
        four_words words[8];
#pragma unroll
        for (uint32_t i = 0; i < 8u; i++) {
            words[i] = *(const four_words *)(block_experts + index + 4u * i);
        }
#pragma unroll
        for (uint32_t i = 0; i < 8u; i++) {
            visit(index + 4u * i, words[i].x);
            visit(index + 4u * i + 1u, words[i].y);
            visit(index + 4u * i + 2u, words[i].z);
            visit(index + 4u * i + 3u, words[i].w);
        }
    }
    for (; index + 8u <= pairs; index += 8u) {
        const four_words low = *(const four_words *)(block_experts + index), high = *(const four_words *)(block_experts + index + 4u);
        visit(index, low.x);
        visit(index + 1u, low.y);
        visit(index + 2u, low.z);
        visit(index + 3u, low.w);
        visit(index + 4u, high.x);
        visit(index + 5u, high.y);
        visit(index + 6u, high.z);
        visit(index + 7u, high.w);
    }
    for (; index < pairs; index++) {
        visit(index, block_experts[index]);
    }
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
