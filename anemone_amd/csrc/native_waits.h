/* native_waits.h -- the wait counts of the kernels that issue their loads by hand (native_device.cuh), as plain integer
 * functions so that a host program can print them and a test can hold them against a model of the issue order
 * (tests/test_native_wait_counts.py compiles this header with g++).
 *
 * A wavefront's loads complete in the order they were issued, and `s_waitcnt vmcnt(N)` returns once at most N are
 * outstanding. The order in which a chain of `total` K steps issues them: the columns of steps 0 .. DEPTH - 2, the
 * weights of steps 0 .. SLOTS - 2, then, in every step j, the columns of step j + DEPTH - 1 and the weights of step
 * j + SLOTS - 1 where the chain has such steps (WEIGHTS_FIRST: the weights ahead of the columns; else behind them). A
 * step's columns are VECTOR_LOADS loads of a wavefront, its weights WEIGHT_LOADS. loads_behind(step, total) is how many
 * loads may still be outstanding at the top of `step` for its own columns and weights to have landed: the loads of later
 * steps that were asked for behind the later of the two. */
#ifndef ANEMONE_NATIVE_WAITS_H
#define ANEMONE_NATIVE_WAITS_H

#include <stdint.h>

#ifdef __HIPCC__
#define NATIVE_WAITS_FUNCTION __host__ __device__ static __forceinline__
#else
#define NATIVE_WAITS_FUNCTION static inline
#endif

template <uint32_t SLOTS, uint32_t DEPTH, bool WEIGHTS_FIRST, uint32_t VECTOR_LOADS, uint32_t WEIGHT_LOADS>
struct native_waits {
    static_assert(SLOTS >= DEPTH && DEPTH >= 2u && SLOTS + DEPTH < 64u, "the weights are asked for at least as far ahead as the columns");
    static_assert((DEPTH - 1u) * VECTOR_LOADS + (SLOTS - 1u) * WEIGHT_LOADS < 64u, "vmcnt has six bits");

    /* a place in the order of issue for the columns and for the weights of step k: what the prologue asks for lies below
     * 64, what step j asks for between 64 (1 + j) and 64 (2 + j) */
    NATIVE_WAITS_FUNCTION uint32_t when_columns(uint32_t k)
    {
        return k < DEPTH - 1u ? k : 64u * (1u + k - (DEPTH - 1u)) + (WEIGHTS_FIRST ? 1u : 0u);
    }

    NATIVE_WAITS_FUNCTION uint32_t when_weights(uint32_t k)
    {
        return k < SLOTS - 1u ? DEPTH - 1u + k : 64u * (1u + k - (SLOTS - 1u)) + (WEIGHTS_FIRST ? 0u : 1u);
    }

    NATIVE_WAITS_FUNCTION uint32_t loads_behind(uint32_t step, uint32_t total)
    {
        const uint32_t mine = when_columns(step) > when_weights(step) ? when_columns(step) : when_weights(step);
        const uint32_t now = 64u * (1u + step); /* what steps before this one asked for lies below this */
        uint32_t count = 0;
#ifdef __HIPCC__
#pragma unroll
#endif
        for (uint32_t ahead = 1; ahead < SLOTS; ahead++) {
            const uint32_t k = step + ahead;
            if (k < total) {
                count += when_columns(k) > mine && when_columns(k) < now ? VECTOR_LOADS : 0u;
                count += when_weights(k) > mine && when_weights(k) < now ? WEIGHT_LOADS : 0u;
            }
        }
        return count;
    }
};

#endif
