/*
 * exl3_stream_device.cuh -- the wavefront product of a decode-sized step: trellis codes go from memory straight into
 * the registers of the lane that decodes them (no LDS, no barrier, no lane-dependent bit positions).
 *
 * Definitions followed (reference tree): ring and window end include/anemone/exl3_records.h:111-119; position map
 * source/kernel_exl3.cu:18-29; codebook source/kernel_exl3.cu:58-65. The mapping below is this build's own.
 *
 * A lane's chunk. Ring position 8 (4 (o % 8) + t) + 4 (o / 8) + j holds output o and input 2 t + j % 2 + 8 (j / 2) of
 * a 16 x 16 tile, so the 32 consecutive positions 32 c .. 32 c + 31 are the outputs c and c + 8 by all sixteen inputs:
 * 16 bits_x2 consecutive ring bits that begin on a multiple of 16 bits_x2 (a whole number of words for a whole K).
 * Lane l = 16 g + i of a step takes the chunk c = i % 8 of output tile (i / 8) of a pair of adjacent tiles and of K tile
 * g of the step's four, with the word in front of it for the first windows' history. Symbol m of the chunk (position
 * 32 c + m) ends E(m) = floor((m + 1) bits_x2 / 2) bits into the chunk -- the same constant in every lane.
 *
 * The matrix instruction. v_mfma_f32_16x16x32_f16 takes from lane 16 g + i eight weights of row i and k group g. Four
 * instructions (h, v in {0, 1}) take symbols 8 t + 4 h + 2 v + {0, 1}, t = 0..3: output c + 8 h against the inputs
 * 8 v + {0..7} of K tile g, whose operand values are one 16-byte load. Row i of the instruction is therefore output
 * c + 8 h of tile i / 8: the sums of h = 0 and h = 1 are kept in two accumulators, and lane 16 g' + j of an accumulator
 * holds outputs 16 (g' / 2) + 8 h + 4 (g' % 2) + {0..3} of column j.
 */
#ifndef EXL3_STREAM_DEVICE_CUH
#define EXL3_STREAM_DEVICE_CUH

#include "exl3_device.cuh"

template <uint32_t bits_x2> struct exl3_chunk {
    static constexpr uint32_t bits = 16u * bits_x2;            /* 64, 80, 96, 128 */
    static constexpr uint32_t words = (bits + 31u) / 32u;      /* registers of a chunk that begins on a word */
    static constexpr bool halved = bits % 32u != 0u;           /* K 2.5: odd chunks begin on a half word */
    static constexpr uint32_t tile_words = EXL3_TILE_VALUES * bits_x2 / 64u;
    __host__ __device__ static constexpr uint32_t end(uint32_t m)
    {
        return (m + 1u) * bits_x2 / 2u;
    }
};

/* What a lane holds of one chunk: z[0] the word in front (only its low 16 bits are read), z[1 ..] the chunk. */
template <uint32_t bits_x2> struct exl3_chunk_words {
    uint32_t z[exl3_chunk<bits_x2>::words + 1u];
};

/* the word of the tile at which lane chunk c's own load begins, and the word in front of it */
template <uint32_t bits_x2>
__device__ static __forceinline__ void exl3_chunk_place(uint32_t c, uint32_t &own, uint32_t &front)
{
    typedef exl3_chunk<bits_x2> C;
    own = c * C::bits / 32u;
    front = (own + C::tile_words - 1u) % C::tile_words;
}

template <uint32_t bits_x2>
__device__ static __forceinline__ void exl3_chunk_load(const uint32_t *__restrict__ tile, uint32_t own, uint32_t front,
                                                       exl3_chunk_words<bits_x2> &out)
{
    typedef exl3_chunk<bits_x2> C;
    out.z[0] = tile[front];
    if constexpr (C::words == 2u) {
        const uint2_t load = *(const uint2_t *)(tile + own);
        out.z[1] = load.x;
        out.z[2] = load.y;
    } else if constexpr (C::words == 3u) {
        typedef uint32_t uint3_t __attribute__((ext_vector_type(3)));
        const uint3_t load = *(const uint3_t *)(tile + own);
        out.z[1] = load.x;
        out.z[2] = load.y;
        out.z[3] = load.z;
    } else {
        const uint4_t load = *(const uint4_t *)(tile + own);
        out.z[1] = load.x;
        out.z[2] = load.y;
        out.z[3] = load.z;
        out.z[4] = load.w;
    }
}

/* K 2.5: a chunk of an odd c begins 16 bits into its first word; bring it to the form of an even one */
template <uint32_t bits_x2>
__device__ static __forceinline__ void exl3_chunk_align(exl3_chunk_words<bits_x2> &held, bool odd)
{
    typedef exl3_chunk<bits_x2> C;
    if constexpr (C::halved) {
#pragma unroll
        for (uint32_t k = 0; k < C::words; k++) {
            const uint32_t moved = __builtin_amdgcn_alignbit(held.z[k], held.z[k + 1u], 16u);
            held.z[k] = odd ? moved : held.z[k];
        }
        held.z[C::words] = odd ? held.z[C::words] << 16 : held.z[C::words];
    }
}

/* the sixteen-bit state of symbol m: a constant field of one register, or of the funnel across two */
template <uint32_t bits_x2>
__device__ static __forceinline__ uint32_t exl3_chunk_state(const uint32_t (&z)[exl3_chunk<bits_x2>::words + 1u],
                                                            const uint32_t (&funnel)[exl3_chunk<bits_x2>::words], uint32_t m)
{
    const uint32_t begin = 32u + exl3_chunk<bits_x2>::end(m) - 16u, word = begin / 32u, offset = begin % 32u;
    if (offset == 0u) {
        return z[word] >> 16;
    }
    if (offset == 16u) {
        return z[word] & 0xFFFFu;
    }
    if (offset < 16u) {
        return __builtin_amdgcn_ubfe(z[word], 16u - offset, 16u);
    }
    return __builtin_amdgcn_ubfe(funnel[word], 32u - offset, 16u);
}

/* two states -> two fp16 values 1024 + b in one register (low half: first): the codebook before its scale and bias */
__device__ static __forceinline__ uint32_t exl3_byte_sums(uint32_t state_low, uint32_t state_high)
{
    const uint32_t product_low = state_low * EXL3_MUL1_MULTIPLIER;
    const uint32_t product_high = state_high * EXL3_MUL1_MULTIPLIER;
    const uint32_t low = __builtin_amdgcn_sad_u8(product_low, 0u, (uint32_t)EXL3_MUL1_BASE * 0x10001u);
    return __builtin_amdgcn_sad_hi_u8(product_high, 0u, low);
}

/* one step of a strip: the held chunks of its NP tile pairs and the sixteen operand values of the lane's K tile */
template <uint32_t bits_x2, uint32_t NP, bool EXACT>
__device__ static __forceinline__ void exl3_stream_step(exl3_chunk_words<bits_x2> (&held)[NP], const uint4_t (&x)[2], bool odd,
                                                        float4_t (&accumulator)[NP][2], float &operand_sum)
{
    typedef exl3_chunk<bits_x2> C;
    const half8_t operand_b[2] = {__builtin_bit_cast(half8_t, x[0]), __builtin_bit_cast(half8_t, x[1])};
    if constexpr (!EXACT) {
        const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
#pragma unroll
        for (uint32_t v = 0; v < 2u; v++) {
            const uint32_t words[4] = {x[v].x, x[v].y, x[v].z, x[v].w};
#pragma unroll
            for (uint32_t r = 0; r < 4u; r++) {
                operand_sum = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, words[r]), ones, operand_sum, false);
            }
        }
    }
#pragma unroll
    for (uint32_t p = 0; p < NP; p++) {
        exl3_chunk_align<bits_x2>(held[p], odd);
        uint32_t funnel[C::words];
#pragma unroll
        for (uint32_t k = 0; k < C::words; k++) {
            funnel[k] = __builtin_amdgcn_alignbit(held[p].z[k], held[p].z[k + 1u], 16u);
        }
#pragma unroll
        for (uint32_t h = 0; h < 2u; h++) {
#pragma unroll
            for (uint32_t v = 0; v < 2u; v++) {
                uint32_t a[4];
#pragma unroll
                for (uint32_t t = 0; t < 4u; t++) {
                    const uint32_t m = 8u * t + 4u * h + 2u * v;
                    const uint32_t sums = exl3_byte_sums(exl3_chunk_state<bits_x2>(held[p].z, funnel, m),
                                                         exl3_chunk_state<bits_x2>(held[p].z, funnel, m + 1u));
                    if constexpr (EXACT) {
                        const half2_t scale = __builtin_bit_cast(half2_t, (uint32_t)EXL3_MUL1_SCALE * 0x10001u);
                        const half2_t bias = __builtin_bit_cast(half2_t, (uint32_t)EXL3_MUL1_BIAS * 0x10001u);
                        a[t] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(half2_t, sums), scale, bias));
                    } else {
                        a[t] = sums;
                    }
                }
                const uint4_t packed = {a[0], a[1], a[2], a[3]};
                accumulator[p][h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, packed), operand_b[v], accumulator[p][h], 0, 0, 0);
            }
        }
    }
}

/*
 * One wavefront multiplies a strip of 2 NP adjacent output tiles by the K tiles [first_tile, last_tile) (a multiple
 * of four of them; both the same in every lane) against up to 16 operand columns.
 *
 *   EXACT   true: every weight is the codebook's fp16 value (one v_pk_fma_f16 a pair), the sums are the products'
 *           false: the matrix instruction takes 1024 + b itself and the scale and bias enter once a sum,
 *                  s . sum((1024 + b) x) + c . sum(x): the weights' rounding to fp16 is left out (a tolerance form)
 *   codes        the matrix's trellis, [inputs / 16][out_tiles][tile_words] uint32
 *   operand      per lane: the fp16 operand row of column l % 16; a column that is not live names any live column's
 *                row (its sums are never stored, and the instruction keeps columns apart)
 *   accumulator  [p][h]: lane 16 g' + j holds outputs 16 (2 p + g' / 2) + 8 h + 4 (g' % 2) + {0..3} of the strip, column j
 *
 * The loads of a step are asked for a step ahead into the registers the other step of a pair of steps does not use
 * (two steps a trip, each with its own registers: no copies between them).
 */
template <uint32_t bits_x2, uint32_t NP, bool EXACT>
__device__ static __forceinline__ void
exl3_stream_product(const uint32_t *__restrict__ codes, uint32_t out_tiles, uint32_t strip_tile, uint32_t first_tile,
                    uint32_t last_tile, const half_t *__restrict__ operand, uint32_t lane, float4_t (&accumulator)[NP][2])
{
    typedef exl3_chunk<bits_x2> C;
    const uint32_t g = lane / 16u, i = lane % 16u, c = i % 8u;
    const bool odd = (c & 1u) != 0u;
    uint32_t own, front;
    exl3_chunk_place<bits_x2>(c, own, front);
    const uint64_t step_stride = 4u * (uint64_t)out_tiles * C::tile_words; /* words between steps */
    const uint32_t *tile = codes + ((uint64_t)(first_tile + g) * out_tiles + strip_tile + i / 8u) * C::tile_words;
    const half_t *x = operand + (first_tile + g) * EXL3_TILE;
#pragma unroll
    for (uint32_t p = 0; p < NP; p++) {
        accumulator[p][0] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
        accumulator[p][1] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
    }
    float operand_sum = 0.0f;
    exl3_chunk_words<bits_x2> first[NP], second[NP];
    uint4_t first_x[2], second_x[2];
    if (first_tile < last_tile) {
#pragma unroll
        for (uint32_t p = 0; p < NP; p++) {
            exl3_chunk_load<bits_x2>(tile + p * 2u * C::tile_words, own, front, first[p]);
        }
        first_x[0] = *(const uint4_t *)x;
        first_x[1] = *(const uint4_t *)(x + 8);
    }
    for (uint32_t step = first_tile; step < last_tile; step += 8u) {
        const bool more = step + 4u < last_tile; /* the same in every lane */
        if (more) {
            tile += step_stride;
            x += 4u * EXL3_TILE;
#pragma unroll
            for (uint32_t p = 0; p < NP; p++) {
                exl3_chunk_load<bits_x2>(tile + p * 2u * C::tile_words, own, front, second[p]);
            }
            second_x[0] = *(const uint4_t *)x;
            second_x[1] = *(const uint4_t *)(x + 8);
        }
        exl3_stream_step<bits_x2, NP, EXACT>(first, first_x, odd, accumulator, operand_sum);
        if (!more) {
            break;
        }
        if (step + 8u < last_tile) {
            tile += step_stride;
            x += 4u * EXL3_TILE;
#pragma unroll
            for (uint32_t p = 0; p < NP; p++) {
                exl3_chunk_load<bits_x2>(tile + p * 2u * C::tile_words, own, front, first[p]);
            }
            first_x[0] = *(const uint4_t *)x;
            first_x[1] = *(const uint4_t *)(x + 8);
        }
        exl3_stream_step<bits_x2, NP, EXACT>(second, second_x, odd, accumulator, operand_sum);
    }
    if constexpr (!EXACT) {
        /* the column's sum of operand values over the four k groups, then y = s . sum + c . sum(x) */
        operand_sum = __fadd_rn(operand_sum, __shfl_xor(operand_sum, 16, WAVE));
        operand_sum = __fadd_rn(operand_sum, __shfl_xor(operand_sum, 32, WAVE));
        const float scale = half_bits_to_float(EXL3_MUL1_SCALE), bias = __fmul_rn(half_bits_to_float(EXL3_MUL1_BIAS), operand_sum);
#pragma unroll
        for (uint32_t p = 0; p < NP; p++) {
#pragma unroll
            for (uint32_t h = 0; h < 2u; h++) {
#pragma unroll
                for (uint32_t r = 0; r < 4u; r++) {
                    accumulator[p][h][r] = __fmaf_rn(scale, accumulator[p][h][r], bias);
                }
            }
        }
    }
}

/* where lane (g', column) stores accumulator [p][h] of a strip: four consecutive outputs from this one */
__device__ static __forceinline__ uint32_t exl3_stream_output(uint32_t strip_tile, uint32_t p, uint32_t h, uint32_t lane)
{
    const uint32_t group = lane / 16u;
    return EXL3_TILE * (strip_tile + 2u * p + group / 2u) + 8u * h + 4u * (group % 2u);
}

#endif
