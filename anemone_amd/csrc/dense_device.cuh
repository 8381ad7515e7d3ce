/*
 * dense_device.cuh -- the dense product of a step's rows as device code (see kernel_dense_linear.hip for its definition),
 * shared by the dense_linear_* kernels and the fused site fronts.
 */
#ifndef DENSE_DEVICE_CUH
#define DENSE_DEVICE_CUH

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "exl3_device.cuh"

#define DENSE_GROUP_LANES 32u
#define DENSE_GROUPS (DENSE_THREADS_VALUE / DENSE_GROUP_LANES)
#define DENSE_DIES 8u

/* the float32 nearest 1 / sqrt(operand): both steps are correctly rounded in double, whose 53 places decide a tie */
__device__ static __forceinline__ float dense_reciprocal_root(float operand)
{
    return (float)(1.0 / __dsqrt_rn((double)operand));
}

/* what a block of DENSE_THREADS_VALUE threads keeps in LDS */
template <uint32_t ROWS, uint32_t OUTPUTS> struct dense_group_sums {
    float sums[DENSE_GROUPS][OUTPUTS + 1u][ROWS];
};

/* OUTPUTS outputs from first_output on by ROWS rows from first_row on, by the DENSE_THREADS_VALUE threads `thread` 0 ..
 * (every one of them calls, and the others of the block reach the same barrier: `active` false computes and stores
 * nothing that is read). `rows` names row 0 of the rows (memory or LDS). */
template <uint32_t TYPE, uint32_t ROWS, uint32_t OUTPUTS>
__device__ static __forceinline__ void dense_linear_body(const struct dense_linear_arguments &arguments, unsigned char *arena, const uint16_t *rows,
                                                         uint32_t first_output, uint32_t first_row, uint32_t thread, bool active,
                                                         dense_group_sums<ROWS, OUTPUTS> &lds)
{
    float (&group_sums)[DENSE_GROUPS][OUTPUTS + 1u][ROWS] = lds.sums;
    const uint32_t inputs = arguments.input_size, chunks = active ? inputs / DENSE_CHUNK_INPUTS : 0u;
    const bool scaled = (arguments.flags & DENSE_ROW_SCALE) != 0u;
    float chain[OUTPUTS][ROWS], squares[ROWS];
#pragma unroll
    for (uint32_t r = 0; r < ROWS; r++) {
        squares[r] = 0.0f;
#pragma unroll
        for (uint32_t o = 0; o < OUTPUTS; o++) {
            chain[o][r] = 0.0f;
        }
    }
#pragma unroll(ROWS == 1u ? 4 : 1)
    for (uint32_t chunk = thread; chunk < chunks; chunk += DENSE_THREADS_VALUE) {
        /* every row's chunk is asked for before any is used: a chunk costs one trip to memory, not one a row */
        uint4_t packed[ROWS];
#pragma unroll
        for (uint32_t r = 0; r < ROWS; r++) {
            /* a column from row_count on reads row 0 and is stored nowhere */
            const uint32_t row = first_row + r < arguments.row_count ? first_row + r : 0u;
            packed[r] = *(const uint4_t *)(rows + (uint64_t)row * inputs + chunk * DENSE_CHUNK_INPUTS);
        }
        /* and every output's weights before the first chain runs */
        float weights[OUTPUTS][DENSE_CHUNK_INPUTS];
#pragma unroll
        for (uint32_t o = 0; o < OUTPUTS; o++) {
            const uint64_t at = (uint64_t)(first_output + o) * inputs + chunk * DENSE_CHUNK_INPUTS;
            if constexpr (TYPE == DENSE_FLOAT32) {
                const float4_t low = *(const float4_t *)((const float *)(arena + arguments.weights_offset) + at);
                const float4_t high = *(const float4_t *)((const float *)(arena + arguments.weights_offset) + at + 4u);
#pragma unroll
                for (uint32_t i = 0; i < 4u; i++) {
                    weights[o][i] = low[i];
                    weights[o][4u + i] = high[i];
                }
            } else {
                unpack_bf16x8(*(const uint4_t *)((const uint16_t *)(arena + arguments.weights_offset) + at), weights[o]);
            }
        }
        float values[ROWS][DENSE_CHUNK_INPUTS];
#pragma unroll
        for (uint32_t r = 0; r < ROWS; r++) {
            unpack_bf16x8(packed[r], values[r]);
        }
        if (scaled) {
#pragma unroll
            for (uint32_t r = 0; r < ROWS; r++) {
#pragma unroll
                for (uint32_t i = 0; i < DENSE_CHUNK_INPUTS; i++) {
                    squares[r] = __fmaf_rn(values[r][i], values[r][i], squares[r]);
                }
            }
        }
#pragma unroll
        for (uint32_t o = 0; o < OUTPUTS; o++) {
#pragma unroll
            for (uint32_t r = 0; r < ROWS; r++) {
#pragma unroll
                for (uint32_t i = 0; i < DENSE_CHUNK_INPUTS; i++) {
                    chain[o][r] = __fmaf_rn(weights[o][i], values[r][i], chain[o][r]);
                }
            }
        }
    }
    const uint32_t group = thread / DENSE_GROUP_LANES, lane = thread % DENSE_GROUP_LANES;
    /* the exchanges of one distance for every chain before the next distance: each chain's additions are the
     * definition's, and the exchanges of different chains are in flight together */
#pragma unroll
    for (uint32_t distance = DENSE_GROUP_LANES / 2u; distance != 0u; distance /= 2u) {
#pragma unroll
        for (uint32_t r = 0; r < ROWS; r++) {
#pragma unroll
            for (uint32_t o = 0; o < OUTPUTS; o++) {
                chain[o][r] = __fadd_rn(chain[o][r], __shfl_xor(chain[o][r], (int)distance, (int)DENSE_GROUP_LANES));
            }
            if (scaled) {
                squares[r] = __fadd_rn(squares[r], __shfl_xor(squares[r], (int)distance, (int)DENSE_GROUP_LANES));
            }
        }
    }
    if (lane == 0u && active) {
#pragma unroll
        for (uint32_t r = 0; r < ROWS; r++) {
#pragma unroll
            for (uint32_t o = 0; o < OUTPUTS; o++) {
                group_sums[group][o][r] = chain[o][r];
            }
            if (scaled) {
                group_sums[group][OUTPUTS][r] = squares[r];
            }
        }
    }
    __syncthreads();
    const uint32_t o = thread / ROWS, r = thread % ROWS;
    if (!active || thread >= OUTPUTS * ROWS || first_row + r >= arguments.row_count) {
        return;
    }
    float sum = 0.0f, square_sum = 0.0f;
#pragma unroll
    for (uint32_t g = 0; g < DENSE_GROUPS; g++) {
        sum = __fadd_rn(sum, group_sums[g][o][r]);
        if (scaled) {
            square_sum = __fadd_rn(square_sum, group_sums[g][OUTPUTS][r]);
        }
    }
    if (scaled) {
        const float operand = __fadd_rn(__fmul_rn(square_sum, __fdiv_rn(1.0f, (float)inputs)), arguments.epsilon);
        sum = __fmul_rn(sum, dense_reciprocal_root(operand));
    }
    const uint64_t index = (uint64_t)(first_row + r) * arguments.output_size + first_output + o;
    if (arguments.output_type == DENSE_FLOAT32) {
        ((float *)(arena + arguments.output_offset))[index] = __fmul_rn(sum, arguments.output_scale);
    } else {
        ((uint16_t *)(arena + arguments.output_offset))[index] = float_to_bf16(__fmul_rn(bf16_to_float(float_to_bf16(sum)), arguments.output_scale));
    }
}

#endif
