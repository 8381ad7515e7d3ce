/*
 * exl3_device.cuh -- device code shared by the EXL3 kernels of gfx950: the mul1 codebook in registers, the
 * 128-point Hadamard transform of one wavefront, the deterministic exponential, and the wavefront product routine
 * that streams trellis tiles through LDS into MFMA.
 *
 * Definitions followed (reference tree): codebook source/kernel_exl3.cu:58-65; tile placement
 * tools/measure/trellis_reference.h:10-11; window end include/anemone/exl3_records.h:111-119; transform order
 * source/kernel_exl3.cu:104-124. The lane mapping below is this build's own (wave64, v_mfma_f32_16x16x32_f16).
 *
 * Lane mapping of one MFMA step. A step multiplies 16 outputs by 32 inputs (two stacked 16 x 16 tiles, tau = 0, 1)
 * with up to 16 operand columns. Lane l owns output row o = l % 16 and input group g = l / 16; it takes from tile
 * tau = g / 2 the two runs of four consecutive ring symbols that belong to row o and to chunks t = 2 q, 2 q + 1,
 * q = g % 2: ring positions 8 (4 (o % 8) + t) + 4 (o / 8) + j, j = 0..3, which are the tile's inputs
 * 2 t + j % 2 + 8 (j / 2). So every symbol of both tiles is decoded by exactly one lane and never moves between
 * lanes. Ordered as (run 0: j = 0, 1), (run 1: j = 0, 1), (run 0: j = 2, 3), (run 1: j = 2, 3) the lane's eight
 * weights are the inputs 16 tau + 4 q + {0, 1, 2, 3, 8, 9, 10, 11}: two runs of four consecutive inputs, which the
 * operand side loads as two 8-byte words.
 */
#ifndef EXL3_DEVICE_CUH
#define EXL3_DEVICE_CUH

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "anemone_records.h"

typedef _Float16 half_t;
typedef half_t half2_t __attribute__((ext_vector_type(2)));
typedef half_t half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

#define WAVE 64u

__device__ static __forceinline__ float bf16_to_float(uint16_t bits)
{
    return __uint_as_float((uint32_t)bits << 16);
}

/* float32 -> bfloat16, to nearest, ties to even; a NaN becomes 0x7FC0. The card's own conversion
 * (v_cvt_pk_bf16_f32) gives, for every float32 that is a number, the bits of (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16
 * (compared over all 2^32 inputs); it keeps a NaN's payload, hence the select. */
__device__ static __forceinline__ uint16_t float_to_bf16(float value)
{
    const uint16_t rounded = __builtin_bit_cast(uint16_t, (__bf16)value);
    return value != value ? (uint16_t)0x7FC0u : rounded;
}

__device__ static __forceinline__ float half_bits_to_float(uint16_t bits)
{
    return (float)__builtin_bit_cast(half_t, bits);
}

/* float32 -> fp16, to nearest even, of a value that already IS a float32: the empty asm keeps the compiler from
 * folding the multiplication that produced it into one mixed-precision instruction (v_fma_mixlo_f16), which would
 * round once where the contract rounds twice (to float32, then to fp16). */
__device__ static __forceinline__ uint16_t float_to_half_bits(float value)
{
    asm volatile("" : "+v"(value));
    return __builtin_bit_cast(uint16_t, (half_t)value); /* v_cvt_f16_f32 */
}

/* e^x by a fixed sequence of float32 operations: k = nearest(x log2 e), r = x - k ln 2 in two pieces, a degree-6
 * polynomial in fma form, scaling by ldexp. Written without contraction so that host and card agree bit for bit.
 * det_exp_sequence is the sequence alone, for an x it is defined for (-104 <= x <= 88.8 in det_expf). */
__device__ static __forceinline__ float det_exp_sequence(float x)
{
    const float k = __builtin_rintf(__fmul_rn(x, 1.44269502162933349609375f));
    float r = __fmaf_rn(k, -0.693145751953125f, x);
    r = __fmaf_rn(k, -1.42860676533018704503775e-06f, r);
    float p = 1.9875691500e-4f;
    p = __fmaf_rn(p, r, 1.3981999507e-3f);
    p = __fmaf_rn(p, r, 8.3334519073e-3f);
    p = __fmaf_rn(p, r, 4.1665795894e-2f);
    p = __fmaf_rn(p, r, 1.6666665459e-1f);
    p = __fmaf_rn(p, r, 5.0000001201e-1f);
    const float r2 = __fmul_rn(r, r);
    float y = __fmaf_rn(p, r2, r);
    y = __fadd_rn(y, 1.0f);
    return ldexpf(y, (int)k);
}

__device__ static __forceinline__ float det_expf(float x)
{
    if (x != x) {
        return x;
    }
    if (x > 88.8f) {
        return __builtin_huge_valf();
    }
    if (x < -104.0f) {
        return 0.0f;
    }
    return det_exp_sequence(x);
}

/* gate / (1 + e^(-gate)): the bits of __fdiv_rn(gate, __fadd_rn(1.0f, det_expf(-gate))) for every float32 gate (a NaN
 * for a NaN), without det_expf's three tests, each of which is a branch of its own and a wait for its comparison in a
 * kernel's epilogue. The sequence's argument is held inside [-104, 89.5] instead: above 88.8 the sequence overflows to
 * infinity by itself (k >= 128 and, where k = 128, r > 0.08, so the polynomial is above 1); below -104 det_expf gives 0
 * and the sequence at -104 something below 2^-148, and 1 plus either is 1; a NaN gate divides to a NaN whatever the
 * denominator. The library's arithmetic_selfcheck kernel compares the two over all 2^32 gates. */
__device__ static __forceinline__ float det_silu(float gate)
{
    const float x = __builtin_amdgcn_fmed3f(-gate, -104.0f, 89.5f);
    return __fdiv_rn(gate, __fadd_rn(1.0f, det_exp_sequence(x)));
}

/* One block of 128 values across a wavefront: lane l holds values l (v0) and l + 64 (v1). Seven stages, the
 * distance doubling from 1; a pair (lower, upper) becomes (lower + upper, lower - upper). No normalisation here. */
__device__ static __forceinline__ void wave_hadamard128(float &v0, float &v1, uint32_t lane)
{
#pragma unroll
    for (uint32_t distance = 1; distance < WAVE; distance *= 2u) {
        const float o0 = __shfl_xor(v0, (int)distance, WAVE);
        const float o1 = __shfl_xor(v1, (int)distance, WAVE);
        /* the lower of a pair becomes lower + upper, the upper lower - upper: other + own or other - own, one
         * rounding either way: a fused multiply-add of own by +1 or -1 (the product is exact) */
        const float sign = (lane & distance) == 0u ? 1.0f : -1.0f;
        v0 = __fmaf_rn(sign, v0, o0);
        v1 = __fmaf_rn(sign, v1, o1);
    }
    const float sum = __fadd_rn(v0, v1), difference = __fsub_rn(v0, v1);
    v0 = sum;
    v1 = difference;
}

/* The same transform with a block of 128 values across SIXTEEN lanes (a row of the wavefront): lane r of the row holds
 * values 8 r .. 8 r + 7. Distances 1, 2, 4 stay inside the lane; 8, 16, 32, 64 pair lane r with r ^ 1, ^ 2, ^ 4, ^ 8 of
 * the row, which the data-parallel primitives of a vector instruction reach without LDS: a permutation of four lanes
 * (^ 1, ^ 2), the mirror of eight lanes followed by the reversal of four (^ 4), the mirror of sixteen followed by the
 * mirror of eight (^ 8). Every pair (lower, upper) becomes (lower + upper, lower - upper), each one rounding: the bits of
 * wave_hadamard128. A row's sixteen lanes are all active or all idle. */
template <int control>
__device__ static __forceinline__ float row_lane_of(float value)
{
    /* every lane of an active row has a source lane in it: what a lane without one would keep is never read */
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, value), control, 0xF, 0xF, true));
}

__device__ static __forceinline__ void row_hadamard128(float (&v)[8], uint32_t lane)
{
    constexpr int SWAP_PAIRS = 0xB1 /* lanes 1, 0, 3, 2 of four */, SWAP_TWOS = 0x4E /* 2, 3, 0, 1 */, REVERSE_FOUR = 0x1B /* 3, 2, 1, 0 */,
                  MIRROR_SIXTEEN = 0x140, MIRROR_EIGHT = 0x141;
#pragma unroll
    for (uint32_t distance = 1; distance < 8u; distance *= 2u) {
#pragma unroll
        for (uint32_t i = 0; i < 8u; i++) {
            if ((i & distance) == 0u) {
                const float lower = v[i], upper = v[i + distance];
                v[i] = __fadd_rn(lower, upper);
                v[i + distance] = __fsub_rn(lower, upper);
            }
        }
    }
    /* other + own for the lower lane of a pair, other - own for the upper: own by +1 or -1 (exact), then one addition
     * whose first operand comes from the other lane inside the instruction */
    const float sign1 = (lane & 1u) == 0u ? 1.0f : -1.0f, sign2 = (lane & 2u) == 0u ? 1.0f : -1.0f;
    const float sign4 = (lane & 4u) == 0u ? 1.0f : -1.0f, sign8 = (lane & 8u) == 0u ? 1.0f : -1.0f;
#pragma unroll
    for (uint32_t i = 0; i < 8u; i++) {
        v[i] = __fadd_rn(row_lane_of<SWAP_PAIRS>(v[i]), __fmul_rn(sign1, v[i]));
    }
#pragma unroll
    for (uint32_t i = 0; i < 8u; i++) {
        v[i] = __fadd_rn(row_lane_of<SWAP_TWOS>(v[i]), __fmul_rn(sign2, v[i]));
    }
#pragma unroll
    for (uint32_t i = 0; i < 8u; i++) {
        v[i] = __fadd_rn(row_lane_of<REVERSE_FOUR>(row_lane_of<MIRROR_EIGHT>(v[i])), __fmul_rn(sign4, v[i]));
    }
#pragma unroll
    for (uint32_t i = 0; i < 8u; i++) {
        v[i] = __fadd_rn(row_lane_of<MIRROR_EIGHT>(row_lane_of<MIRROR_SIXTEEN>(v[i])), __fmul_rn(sign8, v[i]));
    }
}

/* eight bfloat16 or fp16 values of a 16-byte load as float32; eight float32 as fp16, one rounding each */
__device__ static __forceinline__ void unpack_bf16x8(uint4_t load, float (&values)[8])
{
#pragma unroll
    for (uint32_t i = 0; i < 8u; i++) {
        values[i] = __uint_as_float(i % 2u == 0u ? load[i / 2u] << 16 : load[i / 2u] & 0xFFFF0000u);
    }
}

__device__ static __forceinline__ void unpack_half8(uint4_t load, float (&values)[8])
{
#pragma unroll
    for (uint32_t i = 0; i < 8u; i++) {
        values[i] = half_bits_to_float((uint16_t)(i % 2u == 0u ? load[i / 2u] & 0xFFFFu : load[i / 2u] >> 16));
    }
}

__device__ static __forceinline__ uint4_t pack_half8(const float (&values)[8])
{
    uint4_t packed;
#pragma unroll
    for (uint32_t word = 0; word < 4u; word++) {
        packed[word] = (uint32_t)float_to_half_bits(values[2u * word]) | ((uint32_t)float_to_half_bits(values[2u * word + 1u]) << 16);
    }
    return packed;
}

/* mul1: two 16-bit states -> two fp16 weights in one register (low half: first) */
__device__ static __forceinline__ uint32_t exl3_decode_pair(uint32_t state_low, uint32_t state_high)
{
    const uint32_t product_low = state_low * EXL3_MUL1_MULTIPLIER;
    const uint32_t product_high = state_high * EXL3_MUL1_MULTIPLIER;
    /* byte sums with the codebook's base folded in as the accumulator: 0x6400 + b is the fp16 1024 + b. The first
     * sum lands in the low half on top of 0x64006400, the second is added into the high half. */
    const uint32_t low = __builtin_amdgcn_sad_u8(product_low, 0u, (uint32_t)EXL3_MUL1_BASE * 0x10001u);
    const uint32_t packed = __builtin_amdgcn_sad_hi_u8(product_high, 0u, low);
    const half2_t value = __builtin_bit_cast(half2_t, packed);
    const half2_t scale = __builtin_bit_cast(half2_t, (uint32_t)EXL3_MUL1_SCALE * 0x10001u);
    const half2_t bias = __builtin_bit_cast(half2_t, (uint32_t)EXL3_MUL1_BIAS * 0x10001u);
    const half2_t weight = __builtin_elementwise_fma(value, scale, bias); /* v_pk_fma_f16: one rounding each */
    return __builtin_bit_cast(uint32_t, weight);
}

__device__ static __forceinline__ uint16_t exl3_decode_one(uint32_t state)
{
    return (uint16_t)exl3_decode_pair(state & 0xFFFFu, 0u);
}

/* the geometry of one width, all compile time */
template <uint32_t bits_x2> struct exl3_width {
    static constexpr uint32_t ring_bits = EXL3_TILE_VALUES * bits_x2 / 2u;
    static constexpr uint32_t tile_words = ring_bits / 32u;
    static constexpr uint32_t tile_bytes = ring_bits / 8u;
    /* bits from the end of a run's first window to the end of symbol j's; a run starts at an even position */
    __host__ __device__ static constexpr uint32_t step(uint32_t j)
    {
        return (j + 1u) * bits_x2 / 2u - bits_x2 / 2u;
    }
    static_assert(16u + step(3) <= 32u, "a run of four windows fits one 32-bit funnel");
};

/* Where lane (row o, chunk t) finds its run of four symbols in a tile: two word indices and a funnel shift */
struct exl3_run_place {
    uint32_t word0, word1, shift; /* F = alignbit(word0, word1, shift): 32 stream bits from the run's start */
};

template <uint32_t bits_x2>
__device__ static __forceinline__ exl3_run_place exl3_run_of(uint32_t o, uint32_t t)
{
    typedef exl3_width<bits_x2> W;
    const uint32_t position = 8u * (4u * (o % 8u) + t) + 4u * (o / 8u);
    const uint32_t begin = (exl3_window_end(position, bits_x2) + W::ring_bits - 16u) % W::ring_bits;
    const uint32_t word = begin / 32u, offset = begin % 32u;
    exl3_run_place place;
    place.word0 = word;
    /* v_alignbit(hi, lo, s) takes ({hi, lo} >> s)[31:0] with s in 0..31: offset 0 needs lo = hi = word */
    place.word1 = offset == 0u ? word : (word + 1u) % W::tile_words;
    place.shift = (32u - offset) % 32u;
    return place;
}

/* four symbols of a run from its funnel word F -> two registers of two fp16 weights: (j = 0, 1) and (j = 2, 3) */
template <uint32_t bits_x2>
__device__ static __forceinline__ void exl3_decode_run(uint32_t funnel, uint32_t &first, uint32_t &second)
{
    typedef exl3_width<bits_x2> W;
    const uint32_t s0 = funnel >> 16;
    const uint32_t s1 = (funnel >> (16u - W::step(1))) & 0xFFFFu;
    const uint32_t s2 = (funnel >> (16u - W::step(2))) & 0xFFFFu;
    const uint32_t s3 = (funnel >> (16u - W::step(3))) & 0xFFFFu;
    first = exl3_decode_pair(s0, s1);
    second = exl3_decode_pair(s2, s3);
}

/* ---- the wavefront product ----
 *
 * One wavefront multiplies a strip of NT adjacent output tiles by the K tiles [first_tile, last_tile) against up to
 * 16 operand columns and returns, per output tile, the MFMA accumulator (lane l: outputs 4 (l / 16) + i, i = 0..3,
 * of column l % 16). Tile rows of the strip are contiguous in memory (NT tile_bytes bytes), so each K tile row is
 * one coalesced 16-byte-per-lane load; two rows make an MFMA step; the next step's rows are in flight while the
 * current ones are decoded. The rows pass through a private LDS window of the wavefront (no block barrier).
 *
 *   codes        the matrix's trellis, [inputs / 16][out_tiles][tile_words] uint32
 *   out_tiles    output tiles of the whole matrix; strip_tile the first of this strip
 *   operand      per lane: pointer to the fp16 operand row of column l % 16 (NULL: the column is zero)
 *   lds          this wavefront's 2 * NT * tile_bytes bytes of LDS, 16-byte aligned
 */
template <uint32_t bits_x2, uint32_t NT>
__device__ static __forceinline__ void
exl3_wave_product(const uint32_t *__restrict__ codes, uint32_t out_tiles, uint32_t strip_tile, uint32_t first_tile,
                  uint32_t last_tile, const half_t *__restrict__ operand, uint32_t *lds, uint32_t lane,
                  float4_t (&accumulator)[NT])
{
    typedef exl3_width<bits_x2> W;
    constexpr uint32_t row_bytes = NT * W::tile_bytes;      /* one K tile row of the strip */
    constexpr uint32_t row_lanes = row_bytes / 16u;         /* lanes that carry a 16-byte piece of it */
    static_assert(row_bytes % 16u == 0u && row_lanes <= WAVE, "a strip row is at most one load of the wavefront");
    const uint32_t o = lane % 16u, g = lane / 16u, tau = g / 2u, q = g % 2u;
    const exl3_run_place run0 = exl3_run_of<bits_x2>(o, 2u * q), run1 = exl3_run_of<bits_x2>(o, 2u * q + 1u);
    const uint32_t lane_base = tau * (row_bytes / 4u); /* the lane's tile row inside the LDS window, in words */
    const uint64_t row_stride = (uint64_t)out_tiles * W::tile_words; /* words between K tile rows */
    const uint32_t *source = codes + (uint64_t)first_tile * row_stride + (uint64_t)strip_tile * W::tile_words +
                             lane * 4u;
    const bool carries = lane < row_lanes;
    /* the operand's eight inputs of this lane in a step: 16 tau + 4 q + {0..3} and + {8..11}. They are asked for a
     * step ahead with the weights: loads return in order, so an operand asked for inside the step that uses it would
     * make that step wait for the weights prefetched just before it */
    const half_t *x = operand == nullptr ? nullptr : operand + (first_tile * 16u + 16u * tau + 4u * q);
    uint4_t next0 = {0, 0, 0, 0}, next1 = {0, 0, 0, 0};
    uint2_t next_low = {0, 0}, next_high = {0, 0};
    if (first_tile < last_tile) {
        if (carries) {
            next0 = *(const uint4_t *)source;
            next1 = *(const uint4_t *)(source + row_stride);
        }
        if (x != nullptr) {
            next_low = *(const uint2_t *)x;
            next_high = *(const uint2_t *)(x + 8);
        }
    }
#pragma unroll
    for (uint32_t n = 0; n < NT; n++) {
        accumulator[n] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
    }
    for (uint32_t tile = first_tile; tile < last_tile; tile += 2u) {
        const uint4_t row0 = next0, row1 = next1;
        const uint2_t b_low = next_low, b_high = next_high;
        source += 2u * row_stride;
        if (tile + 2u < last_tile) {
            if (carries) {
                next0 = *(const uint4_t *)source;
                next1 = *(const uint4_t *)(source + row_stride);
            }
            if (x != nullptr) {
                x += 32;
                next_low = *(const uint2_t *)x;
                next_high = *(const uint2_t *)(x + 8);
            }
        }
        if (carries) {
            *(uint4_t *)(lds + lane * 4u) = row0;
            *(uint4_t *)(lds + row_bytes / 4u + lane * 4u) = row1;
        }
        __builtin_amdgcn_s_waitcnt(0xc07f); /* lgkmcnt(0): the wavefront's own LDS writes have landed */
        __builtin_amdgcn_wave_barrier();
        const uint32_t b[4] = {b_low.x, b_low.y, b_high.x, b_high.y};
        const half8_t operand_b = __builtin_bit_cast(half8_t, *(const uint4_t *)b);
#pragma unroll
        for (uint32_t n = 0; n < NT; n++) {
            const uint32_t *tile_words = lds + lane_base + n * W::tile_words;
            const uint32_t f0 = __builtin_amdgcn_alignbit(tile_words[run0.word0], tile_words[run0.word1], run0.shift);
            const uint32_t f1 = __builtin_amdgcn_alignbit(tile_words[run1.word0], tile_words[run1.word1], run1.shift);
            uint32_t a[4];
            exl3_decode_run<bits_x2>(f0, a[0], a[2]); /* run 0: inputs 4 q + {0, 1} and {8, 9} */
            exl3_decode_run<bits_x2>(f1, a[1], a[3]); /* run 1: inputs 4 q + {2, 3} and {10, 11} */
            const half8_t weights = __builtin_bit_cast(half8_t, *(const uint4_t *)a);
            accumulator[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(weights, operand_b, accumulator[n], 0, 0, 0);
        }
        __builtin_amdgcn_wave_barrier(); /* the next step's writes stay behind these reads */
    }
}

#endif
