/*
 * native_device.cuh -- a block's pipeline over weights stored in gfx950's own lane order (WEIGHT_FORMAT_E2M1_GFX950,
 * WEIGHT_FORMAT_E4M3_GFX950): a tile's K step of 128 inputs lies in memory as the 64 lanes' A operand of
 * v_mfma_scale_f32_16x16x128_f8f6f4, 16 bytes a lane (32 of one-byte weights, as two halves of 16), and goes from memory
 * into the wavefront's registers with one 16-byte load a lane and half: no LDS stage, no vector instruction between the
 * load and the matrix instruction. A tile's scale codes of a K step are one byte a lane, loaded as such. Only the
 * columns (the vectors' codes, which every wavefront of the block reads) pass through LDS, as in wide_device.cuh: brought
 * by LDS DMA, turned into the B operand's order in place by the wavefront that brought them.
 *
 * A block is COLUMN_BLOCKS x 16 columns (pairs of one expert) by four wavefronts' strips of weight tiles. A wavefront
 * keeps several sets of weight registers: while one step is multiplied, the loads of the steps behind it are on their way.
 */
#ifndef NATIVE_DEVICE_CUH
#define NATIVE_DEVICE_CUH

#include "linear_device.cuh"
#include "native_waits.h"

#define NATIVE_WAVES 4u
/* one-byte weights: a step's next weights are asked for at its top, ahead of the columns' preparation and the barrier
 * (gate/up 953 -> 933 us, down 462 -> 456); 4-bit weights: in the middle of its matrix instructions (at the top: gate/up
 * 1 % shorter, down 3 % longer) */
#define NATIVE_WEIGHTS_FIRST_OF(bytes) (bytes)
#define NATIVE_THREADS (NATIVE_WAVES * WAVE)

/* memory into registers, 16 bytes or one byte a lane: the address is a base common to the wavefront plus the lane's own
 * byte offset (plus 1,024: the second half of a tile of one-byte weights). Assembly, like the loads into LDS beside which
 * they are counted: the compiler keeps no book on them, native_landed is the wait (so a kernel of these loads must spill
 * no vector register: one saved between its load and the wait is saved before it is filled, and the build refuses such
 * a kernel). ONCE: the bytes are read by this
 * block alone (an expert's one-byte weights in a block that holds all its pairs): asked for as a stream, so that they do
 * not push the columns, which every block of the expert reads, out of the level-2 cache. */
template <bool ONCE>
__device__ static __forceinline__ void load_16(uint4_t &into, const unsigned char *base, uint32_t lane_offset)
{
    if constexpr (ONCE) {
        asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=v"(into) : "v"(lane_offset), "s"(base) : "memory");
    } else {
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(into) : "v"(lane_offset), "s"(base) : "memory");
    }
}

template <bool ONCE>
__device__ static __forceinline__ void load_16_second(uint4_t &into, const unsigned char *base, uint32_t lane_offset)
{
    if constexpr (ONCE) {
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024 nt" : "=v"(into) : "v"(lane_offset), "s"(base) : "memory");
    } else {
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024" : "=v"(into) : "v"(lane_offset), "s"(base) : "memory");
    }
}

__device__ static __forceinline__ void load_1(uint32_t &into, const unsigned char *base, uint32_t lane_offset)
{
    asm volatile("global_load_ubyte %0, %1, %2" : "=v"(into) : "v"(lane_offset), "s"(base) : "memory");
}

__device__ static __forceinline__ void load_4(uint32_t &into, const unsigned char *base, uint32_t lane_offset)
{
    asm volatile("global_load_dword %0, %1, %2" : "=v"(into) : "v"(lane_offset), "s"(base) : "memory");
}

/* behind wait_loads: the value the load left in the register is this statement's result, so that nothing that uses it
 * can be placed ahead of the wait */
__device__ static __forceinline__ void native_landed(uint4_t &value)
{
    asm volatile("" : "+v"(value));
}

__device__ static __forceinline__ void native_landed(uint32_t &value)
{
    asm volatile("" : "+v"(value));
}

/* SLOTS: sets of weight registers a wavefront keeps (the weights of SLOTS - 1 steps are on their way while one is
 * multiplied); DEPTH: stages of columns in LDS, likewise */
/* B128 (one-byte weights alone): float32 scales, one for every 128 outputs x 128 inputs of a matrix and one for every 128
 * values of a column, in place of the E8M0 codes (the same bytes a K step: a word where four codes were): a K step's
 * matrix instruction runs from zero with scale codes of one and its sums enter the chain by one fused multiply-add with
 * the product of the two scales, as the reference-order kernels of that scaling add them */
template <uint32_t MATRICES, bool BYTES, uint32_t STRIP_TILES, uint32_t COLUMN_BLOCKS, uint32_t SLOTS, uint32_t DEPTH, bool B128 = false>
struct native_chain {
    static_assert(BYTES || !B128, "float32 scales go with one-byte weights");
    static_assert(COLUMN_BLOCKS == 4u || COLUMN_BLOCKS == 8u, "a wavefront brings one or two column blocks");
    static constexpr uint32_t STRIP = STRIP_TILES;
    static constexpr uint32_t TILES = MATRICES * STRIP;
    static constexpr uint32_t STEP_BYTES = BYTES ? BYTE_STEP_BYTES : NIBBLE_STEP_BYTES;
    static constexpr uint32_t HALVES = STEP_BYTES / 1024u;
    static constexpr uint32_t WAVE_BLOCKS = COLUMN_BLOCKS / NATIVE_WAVES;     /* column blocks a wavefront brings and prepares */
    static constexpr uint32_t VECTOR_BYTES = COLUMN_BLOCKS * 2048u;            /* a K step of the block's columns' codes */
    static constexpr uint32_t STAGE_BYTES = VECTOR_BYTES + COLUMN_BLOCKS * 64u; /* and their scale words behind them */
    static constexpr uint32_t WINDOW_BYTES = DEPTH * STAGE_BYTES;
    static constexpr uint32_t VECTOR_LOADS = 2u * WAVE_BLOCKS + 1u;
    /* scale codes: of one-byte weights a byte a lane a tile (a row of 32 outputs' codes, as the reference stores them); of
     * 4-bit weights a word a lane a matrix: its bytes are the codes of the lane's row and inputs in the four tiles of a group
     * of 64 outputs, which the matrix instruction picks by number */
    static constexpr uint32_t SCALE_LOADS = BYTES && !B128 ? TILES : MATRICES;
    static constexpr uint32_t WEIGHT_LOADS = TILES * HALVES + SCALE_LOADS;
    static_assert(BYTES || STRIP == 2u || STRIP == 4u, "a strip of 4-bit weights is half a group of four tiles, or a whole one");
    static_assert((DEPTH - 1u) * VECTOR_LOADS + (SLOTS - 1u) * WEIGHT_LOADS < 64u, "vmcnt has six bits");

    struct slot {
        uint4_t words[TILES][HALVES];
        uint32_t scale[SCALE_LOADS];
    };

    const unsigned char *words[MATRICES], *scales[MATRICES], *codes, *exponents;
    uint32_t step_stride; /* from a tile's K step to its next */
    uint32_t window, wave, word_offset[STRIP], scale_offset[STRIP], codes_offset[WAVE_BLOCKS][2], exponents_offset;
    uint32_t vector_at[BYTES ? 8 : 4], vector_scale_at, operand_at, scale_shift;
    bool scale_lane;

    template <typename T>
    __device__ static __forceinline__ T lds_read(uint32_t address)
    {
        return *(const __attribute__((address_space(3))) T *)(uintptr_t)address;
    }

    template <typename T>
    __device__ static __forceinline__ void lds_write(uint32_t address, T value)
    {
        *(__attribute__((address_space(3))) T *)(uintptr_t)address = value;
    }

    /* the block's columns of K step `at` into stage `stage`: this wavefront's column blocks and their scale words */
    __device__ __forceinline__ void issue_vectors(uint32_t stage, uint32_t at) const
    {
        const uint32_t base = window + stage * STAGE_BYTES;
#pragma unroll
        for (uint32_t i = 0; i < WAVE_BLOCKS; i++) {
#pragma unroll
            for (uint32_t part = 0; part < 2u; part++) {
                load_to_lds_16(codes + (uint64_t)at * 128u, codes_offset[i][part], base + (wave * WAVE_BLOCKS + i) * 2048u + part * 1024u);
            }
        }
        if (scale_lane) { /* a lane a column: sixteen cache lines a column block */
            load_to_lds_4(exponents + (uint64_t)at * 4u, exponents_offset, base + VECTOR_BYTES + wave * WAVE_BLOCKS * 64u);
        }
    }

    /* the wavefront's weights and scale codes of K step `at` into a set of registers */
    __device__ __forceinline__ void issue_weights(slot &into, uint32_t at) const
    {
#pragma unroll
        for (uint32_t m = 0; m < MATRICES; m++) {
            const unsigned char *step_words = words[m] + (uint64_t)at * step_stride;
#pragma unroll
            for (uint32_t n = 0; n < STRIP; n++) {
                load_16<BYTES>(into.words[m * STRIP + n][0], step_words, word_offset[n]);
                if constexpr (BYTES) {
                    load_16_second<BYTES>(into.words[m * STRIP + n][1], step_words, word_offset[n]);
                }
            }
        }
#pragma unroll
        for (uint32_t m = 0; m < MATRICES; m++) {
            const unsigned char *step_scales = scales[m] + (uint64_t)at * (BYTES ? 4u : 256u);
            if constexpr (BYTES && !B128) {
#pragma unroll
                for (uint32_t n = 0; n < STRIP; n++) {
                    load_1(into.scale[m * STRIP + n], step_scales, scale_offset[n]);
                }
            } else { /* a word a lane of a group of four tiles' codes, or the strip's one float32 scale in every lane */
                load_4(into.scale[m], step_scales, scale_offset[0]);
            }
        }
    }

    __device__ static __forceinline__ void landed(slot &set)
    {
#pragma unroll
        for (uint32_t t = 0; t < TILES; t++) {
#pragma unroll
            for (uint32_t h = 0; h < HALVES; h++) {
                native_landed(set.words[t][h]);
            }
        }
#pragma unroll
        for (uint32_t k = 0; k < SCALE_LOADS; k++) {
            native_landed(set.scale[k]);
        }
    }

    /* this wavefront's column blocks of a stage, from the codes as they landed (a column's 128 bytes in the order the
     * quantizer writes them) to the B operand, in place: [half of the operand][lane][16 bytes]; only this wavefront
     * touches them before the next barrier */
    __device__ __forceinline__ void prepare_columns(uint32_t stage) const
    {
#pragma unroll
        for (uint32_t i = 0; i < WAVE_BLOCKS; i++) {
            uint32_t at = window + stage * STAGE_BYTES + (wave * WAVE_BLOCKS + i) * 2048u;
            asm volatile("" : "+s"(at));
            int8_vector b;
            if constexpr (BYTES) {
#pragma unroll
                for (uint32_t v = 0; v < 8u; v++) {
                    b[v] = (int)lds_read<uint32_t>(at + vector_at[v]);
                }
            } else {
#pragma unroll
                for (uint32_t part = 0; part < 4u; part++) {
                    const uint2_t pair = lds_read<uint2_t>(at + vector_at[part]);
                    b[2u * part] = (int)__builtin_amdgcn_perm(pair.y, pair.x, 0x05010400u);
                    b[2u * part + 1u] = (int)__builtin_amdgcn_perm(pair.y, pair.x, 0x07030602u);
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* every lane has read before any lane writes */
            lds_write<uint4_t>(at + operand_at, (uint4_t){(uint32_t)b[0], (uint32_t)b[1], (uint32_t)b[2], (uint32_t)b[3]});
            lds_write<uint4_t>(at + operand_at + 1024u, (uint4_t){(uint32_t)b[4], (uint32_t)b[5], (uint32_t)b[6], (uint32_t)b[7]});
        }
    }

    /* tile T and the tiles behind it of the wavefront's strip against column block j (the number of the scale code's byte
     * is part of the instruction: a constant) */
    template <uint32_t T>
    __device__ static __forceinline__ void multiply_tiles(const slot &set, const uint32_t (&scale_a)[SCALE_LOADS], const int8_vector &b,
                                                          uint32_t scale_b, uint32_t j, float4_t (&chain)[TILES][COLUMN_BLOCKS])
    {
        if constexpr (B128) {
            const uint4_t first = set.words[T][0], second = set.words[T][HALVES - 1u];
            const int8_vector a = {(int)first.x, (int)first.y, (int)first.z, (int)first.w, (int)second.x, (int)second.y, (int)second.z, (int)second.w};
            const float scale = __fmul_rn(__uint_as_float(scale_a[T / STRIP]), __uint_as_float(scale_b));
            const float4_t step = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, (float4_t){0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0, 127, 0, 127);
#pragma unroll
            for (uint32_t v = 0; v < 4u; v++) {
                chain[T][j][v] = __fmaf_rn(step[v], scale, chain[T][j][v]);
            }
        } else if constexpr (BYTES) {
            const uint4_t first = set.words[T][0], second = set.words[T][HALVES - 1u];
            const int8_vector a = {(int)first.x, (int)first.y, (int)first.z, (int)first.w, (int)second.x, (int)second.y, (int)second.z, (int)second.w};
            chain[T][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, chain[T][j], 0, 0, 0, (int)scale_a[T], 0, (int)scale_b);
        } else {
            const uint4_t w = set.words[T][0];
            const int8_vector a = {(int)w.x, (int)w.y, (int)w.z, (int)w.w, 0, 0, 0, 0};
            chain[T][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, chain[T][j], 4, 0, T % STRIP, (int)scale_a[T / STRIP], 0, (int)scale_b);
        }
        if constexpr (T + 1u < TILES) {
            multiply_tiles<T + 1u>(set, scale_a, b, scale_b, j, chain);
        }
    }

    /* one K step of LIVE column blocks from a stage's columns and a set of weight registers; `between` runs behind the
     * middle column block's matrix instructions */
    template <uint32_t LIVE, typename BETWEEN>
    __device__ __forceinline__ void consume(uint32_t stage, const slot &set, float4_t (&chain)[TILES][COLUMN_BLOCKS], BETWEEN between) const
    {
        uint32_t base = window + stage * STAGE_BYTES;
        asm volatile("" : "+s"(base));
        uint32_t b_at = base + operand_at, b_scale_at = base + VECTOR_BYTES + vector_scale_at;
        asm volatile("" : "+v"(b_at), "+v"(b_scale_at));
        uint32_t scale_a[SCALE_LOADS];
#pragma unroll
        for (uint32_t k = 0; k < SCALE_LOADS; k++) { /* 4-bit weights, two tiles a strip: the group's upper two tiles' codes down */
            scale_a[k] = BYTES ? set.scale[k] : set.scale[k] >> scale_shift;
        }
        __builtin_amdgcn_s_setprio(1);
        /* a column block's operand is read while the block before it is multiplied: two blocks' registers, not LIVE */
        uint4_t low = lds_read<uint4_t>(b_at), high = lds_read<uint4_t>(b_at + 1024u);
        uint32_t scale_b = B128 ? lds_read<uint32_t>(b_scale_at) : lds_read<unsigned char>(b_scale_at); /* a code, or a float32's bits */
#pragma unroll
        for (uint32_t j = 0; j < LIVE; j++) {
            const int8_vector b = {(int)low.x, (int)low.y, (int)low.z, (int)low.w, (int)high.x, (int)high.y, (int)high.z, (int)high.w};
            const uint32_t scale_now = scale_b;
            asm volatile("" ::: "memory"); /* the reads below stay below the reads above, and above those of the next block */
            if (j + 1u < LIVE) {
                low = lds_read<uint4_t>(b_at + (j + 1u) * 2048u);
                high = lds_read<uint4_t>(b_at + (j + 1u) * 2048u + 1024u);
                scale_b = B128 ? lds_read<uint32_t>(b_scale_at + (j + 1u) * 64u) : lds_read<unsigned char>(b_scale_at + (j + 1u) * 64u);
            }
            multiply_tiles<0>(set, scale_a, b, scale_now, j, chain);
            if (j == (LIVE - 1u) / 2u) {
                between();
            }
        }
        __builtin_amdgcn_s_setprio(0);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* the stage is read before the next barrier */
    }

    /* how many loads may be outstanding at the top of a K step for its columns and weights to have landed: native_waits.h */
    static constexpr bool WEIGHTS_FIRST = NATIVE_WEIGHTS_FIRST_OF(BYTES); /* inside a step: the weights asked for ahead of the columns */
    typedef native_waits<SLOTS, DEPTH, WEIGHTS_FIRST, VECTOR_LOADS, WEIGHT_LOADS> waits;
    __device__ static __forceinline__ uint32_t loads_behind(uint32_t step, uint32_t total)
    {
        return waits::loads_behind(step, total);
    }

    /* s_waitcnt takes its count as a constant: one instruction a count that loads_behind can come to */
    template <uint32_t WEIGHTS = 0, uint32_t VECTORS = 0>
    __device__ static __forceinline__ void wait_behind(uint32_t count)
    {
        if (count == WEIGHTS * WEIGHT_LOADS + VECTORS * VECTOR_LOADS) {
            wait_loads<WEIGHTS * WEIGHT_LOADS + VECTORS * VECTOR_LOADS>();
            return;
        }
        if constexpr (VECTORS + 1u < DEPTH - 1u) {
            wait_behind<WEIGHTS, VECTORS + 1u>(count);
        } else if constexpr (WEIGHTS + 1u < SLOTS) {
            wait_behind<WEIGHTS + 1u, 0u>(count);
        } else {
            wait_loads<0>(); /* not reached: every count is one of the above */
        }
    }

    /* K step `step` of `total` out of set K of the wavefront's sets of weight registers; the weights of step
     * `step` + SLOTS - 1 take the set the step before this one used */
    template <uint32_t LIVE, uint32_t K>
    __device__ __forceinline__ void one_step(uint32_t step, uint32_t total, slot (&sets)[SLOTS], float4_t (&chain)[TILES][COLUMN_BLOCKS]) const
    {
        wait_behind(loads_behind(step, total));
        landed(sets[K]);
        const auto ask = [&]() {
            if (step + SLOTS - 1u < total) {
                issue_weights(sets[(K + SLOTS - 1u) % SLOTS], step + SLOTS - 1u);
            }
        };
        if constexpr (WEIGHTS_FIRST) {
            ask(); /* into the set the step before this one used: nothing of the block's is waited for */
        }
        /* where the sets and the stages go round together the stage is a constant of the instance */
        const uint32_t stage = SLOTS % DEPTH == 0u ? K % DEPTH : step % DEPTH;
        prepare_columns(stage);
        __syncthreads(); /* every wavefront has read the step before and prepared its columns of this one */
        if (step + DEPTH - 1u < total) {
            issue_vectors((stage + DEPTH - 1u) % DEPTH, step + DEPTH - 1u);
        }
        /* 4-bit weights: the next weights are asked for in the middle of the step's matrix instructions (a launch 1.7 %
         * shorter than asking ahead of them: the requests spread over the step); one-byte weights in the middle: a quarter
         * slower */
        if constexpr (WEIGHTS_FIRST) {
            consume<LIVE>(stage, sets[K], chain, []() {});
        } else if constexpr (BYTES) {
            ask();
            consume<LIVE>(stage, sets[K], chain, []() {});
        } else {
            consume<LIVE>(stage, sets[K], chain, ask);
        }
    }

    template <uint32_t LIVE, uint32_t K>
    __device__ __forceinline__ void round_of_steps(uint32_t step, uint32_t total, slot (&sets)[SLOTS], float4_t (&chain)[TILES][COLUMN_BLOCKS]) const
    {
        if (step + K < total) {
            one_step<LIVE, K>(step + K, total, sets, chain);
        }
        if constexpr (K + 1u < SLOTS) {
            round_of_steps<LIVE, K + 1u>(step, total, sets, chain);
        }
    }

    template <uint32_t K>
    __device__ __forceinline__ void first_weights(uint32_t total, slot (&sets)[SLOTS]) const
    {
        if (K < total) {
            issue_weights(sets[K], K);
        }
        if constexpr (K + 2u < SLOTS) {
            first_weights<K + 1u>(total, sets);
        }
    }

    template <uint32_t LIVE>
    __device__ __forceinline__ void steps(uint32_t total, float4_t (&chain)[TILES][COLUMN_BLOCKS]) const
    {
        slot sets[SLOTS];
#pragma unroll
        for (uint32_t k = 0; k + 1u < DEPTH; k++) {
            if (k < total) {
                issue_vectors(k, k);
            }
        }
        first_weights<0>(total, sets);
        for (uint32_t step = 0; step < total; step += SLOTS) {
            round_of_steps<LIVE, 0>(step, total, sets, chain);
        }
    }

    /* live_blocks: the column blocks that hold a pair, the same in every lane of the block */
    __device__ __forceinline__ void whole(uint32_t total, uint32_t live_blocks, float4_t (&chain)[TILES][COLUMN_BLOCKS]) const
    {
        if constexpr (COLUMN_BLOCKS == 4u) {
            switch (live_blocks) {
            case 1u: steps<1>(total, chain); break;
            case 2u: steps<2>(total, chain); break;
            case 3u: steps<3>(total, chain); break;
            default: steps<4>(total, chain); break;
            }
        } else { /* five and seven run as six and eight: a block of columns past the last pair reads the first pair's again */
            switch (live_blocks) {
            case 1u: steps<1>(total, chain); break;
            case 2u: steps<2>(total, chain); break;
            case 3u: steps<3>(total, chain); break;
            case 4u: steps<4>(total, chain); break;
            case 5u:
            case 6u: steps<6>(total, chain); break;
            default: steps<8>(total, chain); break;
            }
        }
    }

    /* matrices: arena addresses of the stored matrices; the block's first strip is NATIVE_WAVES block_strip;
     * code_vectors[i][part]: the vector of column lane / 8 of group `part` of this wavefront's i-th column block;
     * exponent_vector: the vector of column lane of this wavefront's column blocks (lanes below 16 WAVE_BLOCKS) */
    __device__ __forceinline__ void place(const unsigned char *const (&matrices)[MATRICES], uint32_t outputs, uint32_t inputs,
                                          uint32_t block_strip, const unsigned char *vector_codes, const unsigned char *vector_exponents,
                                          const uint32_t (&code_vectors)[WAVE_BLOCKS][2], uint32_t exponent_vector, uint32_t window_address,
                                          uint32_t wave_index, uint32_t lane, uint32_t &tile0_out)
    {
        const uint32_t tiles = outputs / 16u, steps = inputs / 128u;
        const uint32_t o = lane % 16u, g = lane / 16u;
        const uint32_t strip = block_strip * NATIVE_WAVES + wave_index;
        /* a strip that reaches past the last tile reads the last tiles again; its surplus sums are not stored */
        const uint32_t tile0 = strip * STRIP + STRIP <= tiles ? strip * STRIP : tiles - STRIP;
        tile0_out = tile0;
        const uint32_t tile_bytes = steps * STEP_BYTES;
        step_stride = STEP_BYTES;
        window = window_address;
        wave = wave_index;
        codes = vector_codes;
        exponents = vector_exponents;
#pragma unroll
        for (uint32_t m = 0; m < MATRICES; m++) {
            words[m] = matrices[m] + (uint64_t)tile0 * tile_bytes;
            if constexpr (B128) { /* float32 [outputs / 128][inputs / 128] behind the codes: the strip's row, a word a K step */
                scales[m] = matrices[m] + (uint64_t)outputs * inputs + (uint64_t)(tile0 / 8u) * (inputs / 32u);
            } else if constexpr (BYTES) { /* the scale codes as the reference stores them: a row of inputs / 32 bytes for every 32 outputs */
                scales[m] = matrices[m] + (uint64_t)outputs * inputs + (uint64_t)(tile0 / 2u) * (inputs / 32u);
            } else { /* a word a lane a K step of a group of four tiles */
                scales[m] = matrices[m] + (uint64_t)outputs * inputs / 2u + (uint64_t)(tile0 / 4u) * steps * 256u;
            }
        }
#pragma unroll
        for (uint32_t n = 0; n < STRIP; n++) {
            word_offset[n] = n * tile_bytes + 16u * lane;
            scale_offset[n] = B128 ? 0u : BYTES ? ((tile0 + n) / 2u - tile0 / 2u) * (inputs / 32u) + g : 4u * lane;
        }
#pragma unroll
        for (uint32_t i = 0; i < WAVE_BLOCKS; i++) {
#pragma unroll
            for (uint32_t part = 0; part < 2u; part++) {
                codes_offset[i][part] = code_vectors[i][part] * inputs + 16u * ((lane % 8u) ^ (lane / 8u) ^ part);
            }
        }
        exponents_offset = exponent_vector * (inputs / 32u);
        scale_lane = lane < 16u * WAVE_BLOCKS;
        const uint32_t column = o % 8u, group_bytes = (o / 8u) * 1024u;
        if constexpr (BYTES) {
#pragma unroll
            for (uint32_t v = 0; v < 8u; v++) {
                vector_at[v] = group_bytes + 16u * (8u * column + (v ^ column ^ (o / 8u))) + 4u * g;
            }
        } else {
#pragma unroll
            for (uint32_t part = 0; part < 4u; part++) {
                const uint32_t piece = 4u * (part / 2u) + part % 2u + 2u * (g % 2u);
                vector_at[part] = group_bytes + 16u * (8u * column + (piece ^ column ^ (o / 8u))) + 8u * (g / 2u);
            }
        }
        vector_scale_at = B128 ? 4u * o : 4u * o + g;
        operand_at = 16u * lane;
        scale_shift = 8u * (tile0 % 4u);
    }
};

#endif
