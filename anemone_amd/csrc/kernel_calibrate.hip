/*
 * kernel_calibrate.hip -- a plain copy inside the arena, of a known size: the yardstick the memory-traffic counters
 * of a profile are scaled by (a counter's reading for this kernel against the bytes it is known to move). No
 * counterpart in the reference; not on the routed-expert path.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernel_registry.h"

struct arena_copy_arguments {
    uint64_t source_offset;
    uint64_t destination_offset;
    uint64_t byte_count; /* a multiple of 16 */
};
static_assert(sizeof(struct arena_copy_arguments) == 24, "arena_copy_arguments ABI");

typedef uint32_t copy_word __attribute__((ext_vector_type(4)));

extern "C" __global__ void arena_copy(struct arena_copy_arguments arguments, unsigned char *arena)
{
    const copy_word *source = (const copy_word *)(arena + arguments.source_offset);
    copy_word *destination = (copy_word *)(arena + arguments.destination_offset);
    const uint64_t words = arguments.byte_count / 16u;
    for (uint64_t word = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; word < words; word += (uint64_t)gridDim.x * blockDim.x) {
        destination[word] = source[word];
    }
}
ANEMONE_KERNEL("kernel_calibrate", arena_copy, arena_copy_arguments);

/* issue_rate -- the second yardstick: how often a SIMD issues one vector instruction of the kinds the EXL3 codebook is
 * made of, and how a matrix instruction and vector instructions of one wavefront share the issue. A block is one
 * wavefront; `kind` names the instruction, eight independent chains a lane, `iterations` trips of eight each; kinds 8
 * to 10 are trips of four v_mfma_f32_16x16x32_f16 alone, of eight vector instructions alone, and of the four matrix
 * instructions with two of the vector instructions behind each; kind 11 is trips of eight v_mfma_f32_16x16x1_4b_f32 (the
 * router's many-row projection: one fused multiply-add a sum of four 16 x 16 blocks), each on sums of its own; kinds 12
 * to 15 are trips of ten v_mfma_f32_32x32x16_f16 (the EXL3 prefill GEMM's), each on sums of its own, with 0, 7, 14 and 30 of
 * the codebook's vector instructions behind each: how far a wavefront's decoding runs beside its matrix instructions. The
 * host times the launch; what is written is only there to keep the chains alive. */
struct issue_rate_arguments {
    uint64_t output_offset; /* written: uint32 [grid x 64] */
    uint32_t kind;
    uint32_t iterations;
};
static_assert(sizeof(struct issue_rate_arguments) == 16, "issue_rate_arguments ABI");

typedef _Float16 rate_half8 __attribute__((ext_vector_type(8)));
typedef float rate_float4 __attribute__((ext_vector_type(4)));
typedef float rate_float16 __attribute__((ext_vector_type(16)));

/* kind 11: `iterations` trips of eight v_mfma_f32_16x16x1_4b_f32, eight sets of sums */
__device__ static __forceinline__ float issue_rate_blocks(uint32_t iterations, float left, float right)
{
    rate_float16 sums[8];
    for (uint32_t q = 0; q < 8u; q++) {
        for (uint32_t v = 0; v < 16u; v++) {
            sums[q][v] = 0.0f;
        }
    }
    for (uint32_t trip = 0; trip < iterations; trip++) {
#pragma unroll
        for (uint32_t q = 0; q < 8u; q++) {
            asm volatile("v_mfma_f32_16x16x1_4b_f32 %0, %1, %2, %0" : "+v"(sums[q]) : "v"(left), "v"(right));
        }
    }
    float kept = 0.0f;
    for (uint32_t q = 0; q < 8u; q++) {
        for (uint32_t v = 0; v < 16u; v++) {
            kept += sums[q][v];
        }
    }
    return kept;
}

/* kinds 12 to 15: `iterations` trips of ten v_mfma_f32_32x32x16_f16 with BEHIND vector instructions behind each */
template <uint32_t BEHIND>
__device__ static __forceinline__ float issue_rate_beside(uint32_t iterations, uint32_t (&a)[8], rate_half8 left, rate_half8 right)
{
    rate_float16 sums[10];
    for (uint32_t q = 0; q < 10u; q++) {
        for (uint32_t v = 0; v < 16u; v++) {
            sums[q][v] = 0.0f;
        }
    }
    const uint32_t multiplier = 0x83DCD12Du;
    for (uint32_t trip = 0; trip < iterations; trip++) {
#pragma unroll
        for (uint32_t q = 0; q < 10u; q++) {
            asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(sums[q]) : "v"(left), "v"(right));
#pragma unroll
            for (uint32_t n = 0; n < BEHIND; n++) {
                if (n % 3u == 0u) asm volatile("v_mul_lo_u32 %0, %0, %1" : "+v"(a[n % 8u]) : "s"(multiplier));
                if (n % 3u == 1u) asm volatile("v_bfe_u32 %0, %0, 3, 16" : "+v"(a[n % 8u]));
                if (n % 3u == 2u) asm volatile("v_sad_u8 %0, %0, 0, %0" : "+v"(a[n % 8u]));
            }
        }
    }
    float kept = 0.0f;
    for (uint32_t q = 0; q < 10u; q++) {
        for (uint32_t v = 0; v < 16u; v++) {
            kept += sums[q][v];
        }
    }
    return kept;
}

template <uint32_t KIND>
__device__ static __forceinline__ void issue_rate_loop(uint32_t iterations, uint32_t (&a)[8], rate_float4 (&sums)[4], rate_half8 left, rate_half8 right)
{
    const uint32_t multiplier = 0x83DCD12Du;
    for (uint32_t trip = 0; trip < iterations; trip++) {
#pragma unroll
        for (uint32_t i = 0; i < 8u; i++) {
            if constexpr (KIND == 0u) asm volatile("v_mul_lo_u32 %0, %0, %1" : "+v"(a[i]) : "s"(multiplier));
            if constexpr (KIND == 1u) asm volatile("v_sad_u8 %0, %0, 0, %0" : "+v"(a[i]));
            if constexpr (KIND == 2u) asm volatile("v_bfe_u32 %0, %0, 3, 16" : "+v"(a[i]));
            if constexpr (KIND == 3u) asm volatile("v_and_b32 %0, 0xffff, %0" : "+v"(a[i]));
            if constexpr (KIND == 4u) asm volatile("v_pk_fma_f16 %0, %0, %1, %0" : "+v"(a[i]) : "s"(multiplier));
            if constexpr (KIND == 5u) asm volatile("v_alignbit_b32 %0, %0, %0, 16" : "+v"(a[i]));
            if constexpr (KIND == 6u) asm volatile("v_lshrrev_b32 %0, 3, %0" : "+v"(a[i]));
            if constexpr (KIND == 7u) asm volatile("v_perm_b32 %0, %0, %0, %1" : "+v"(a[i]) : "s"(multiplier));
            if constexpr (KIND >= 8u) {
                if (KIND != 9u && i % 2u == 0u) { /* four matrix instructions a trip, each its own sums */
                    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(sums[i / 2u]) : "v"(left), "v"(right));
                }
                if (KIND != 8u) {
                    if (i % 2u == 0u) {
                        asm volatile("v_mul_lo_u32 %0, %0, %1" : "+v"(a[i]) : "s"(multiplier));
                    } else {
                        asm volatile("v_sad_u8 %0, %0, 0, %0" : "+v"(a[i]));
                    }
                }
            }
        }
    }
}

extern "C" __global__ void __launch_bounds__(64) issue_rate(struct issue_rate_arguments arguments, unsigned char *arena)
{
    uint32_t a[8];
    for (uint32_t i = 0; i < 8u; i++) {
        a[i] = threadIdx.x * 2654435761u + i;
    }
    rate_half8 left, right;
    for (uint32_t i = 0; i < 8u; i++) {
        left[i] = (_Float16)(float)(threadIdx.x % 7u + i);
        right[i] = (_Float16)(float)i;
    }
    rate_float4 sums[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
    if (arguments.kind == 11u) { /* the same in every lane */
        const float kept = issue_rate_blocks(arguments.iterations, (float)(threadIdx.x % 7u) * 0.001f, 1.0f + (float)threadIdx.x * 0.002f);
        ((uint32_t *)(arena + arguments.output_offset))[blockIdx.x * 64u + threadIdx.x] = (uint32_t)kept;
        return;
    }
    if (arguments.kind >= 12u) { /* the same in every lane */
        float kept = 0.0f;
        switch (arguments.kind) {
        case 12u: kept = issue_rate_beside<0u>(arguments.iterations, a, left, right); break;
        case 13u: kept = issue_rate_beside<7u>(arguments.iterations, a, left, right); break;
        case 14u: kept = issue_rate_beside<14u>(arguments.iterations, a, left, right); break;
        default: kept = issue_rate_beside<30u>(arguments.iterations, a, left, right); break;
        }
        uint32_t word = (uint32_t)kept;
        for (uint32_t i = 0; i < 8u; i++) {
            word ^= a[i];
        }
        ((uint32_t *)(arena + arguments.output_offset))[blockIdx.x * 64u + threadIdx.x] = word;
        return;
    }
    switch (arguments.kind) {
    case 0u: issue_rate_loop<0u>(arguments.iterations, a, sums, left, right); break;
    case 1u: issue_rate_loop<1u>(arguments.iterations, a, sums, left, right); break;
    case 2u: issue_rate_loop<2u>(arguments.iterations, a, sums, left, right); break;
    case 3u: issue_rate_loop<3u>(arguments.iterations, a, sums, left, right); break;
    case 4u: issue_rate_loop<4u>(arguments.iterations, a, sums, left, right); break;
    case 5u: issue_rate_loop<5u>(arguments.iterations, a, sums, left, right); break;
    case 6u: issue_rate_loop<6u>(arguments.iterations, a, sums, left, right); break;
    case 7u: issue_rate_loop<7u>(arguments.iterations, a, sums, left, right); break;
    case 8u: issue_rate_loop<8u>(arguments.iterations, a, sums, left, right); break;
    case 9u: issue_rate_loop<9u>(arguments.iterations, a, sums, left, right); break;
    default: issue_rate_loop<10u>(arguments.iterations, a, sums, left, right); break;
    }
    uint32_t kept = 0;
    for (uint32_t i = 0; i < 8u; i++) {
        kept ^= a[i];
    }
    for (uint32_t i = 0; i < 4u; i++) {
        kept ^= (uint32_t)(sums[i][0] + sums[i][1] + sums[i][2] + sums[i][3]);
    }
    ((uint32_t *)(arena + arguments.output_offset))[blockIdx.x * 64u + threadIdx.x] = kept;
}
ANEMONE_KERNEL("kernel_calibrate", issue_rate, issue_rate_arguments);
