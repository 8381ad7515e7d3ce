/*
 * wide_device.cuh -- a block's pipeline over one tile of at most 64 vectors (four MFMA column blocks) by four
 * wavefronts' strips of weight tiles: what the wide routed experts and the trunk's many-row kernel share.
 */
#ifndef WIDE_DEVICE_CUH
#define WIDE_DEVICE_CUH

#include "linear_device.cuh"

#define WIDE_WAVES 4u
#define WIDE_THREADS (WIDE_WAVES * WAVE)
#define WIDE_COLUMN_BLOCKS (WIDE_TILE_PAIRS / 16u)
#define WIDE_DEPTH 3u
#define WIDE_VECTOR_BYTES (WIDE_TILE_PAIRS * 128u) /* a K step of the tile's columns' codes */

/* One block's pipeline: MATRICES matrices x STRIP tiles a wavefront, the tile's columns shared. */
/* B128: float32 scales of 128 x 128 blocks and of 128 values in place of the E8M0 codes, as in strip_device.cuh. */
template <uint32_t MATRICES, bool BYTES, uint32_t STRIP_TILES, uint32_t DEPTH = WIDE_DEPTH, bool B128 = false>
struct wide_chain {
    static_assert(BYTES || !B128, "float32 scales go with one-byte weights");
    static constexpr uint32_t STRIP = STRIP_TILES;
    static constexpr uint32_t STEP_BYTES = BYTES ? BYTE_STEP_BYTES : NIBBLE_STEP_BYTES;
    static constexpr uint32_t TILE_LOADS = STEP_BYTES / 1024u;
    static constexpr uint32_t TILES = MATRICES * STRIP;
    static constexpr uint32_t SCALES_AT = TILES * STEP_BYTES;                    /* inside a wavefront's part */
    static constexpr uint32_t WAVE_BYTES = SCALES_AT + MATRICES * 256u;          /* a wavefront's part of a stage */
    static constexpr uint32_t VECTOR_AT = WIDE_WAVES * WAVE_BYTES;               /* inside a stage */
    static constexpr uint32_t VECTOR_SCALE_AT = VECTOR_AT + WIDE_VECTOR_BYTES;
    static constexpr uint32_t STAGE_BYTES = VECTOR_SCALE_AT + 256u;
    static constexpr uint32_t WINDOW_BYTES = DEPTH * STAGE_BYTES;
    static constexpr uint32_t VECTOR_LOADS = 2u + 1u;                            /* issued first: two column groups, the scale words */
    static constexpr uint32_t WEIGHT_LOADS = TILES * TILE_LOADS + MATRICES;
    static constexpr uint32_t STAGE_LOADS = VECTOR_LOADS + WEIGHT_LOADS;         /* a wavefront's loads a stage */
    static_assert(STAGE_LOADS * (DEPTH - 1u) < 64u && WINDOW_BYTES <= 160u * 1024u, "vmcnt has six bits; LDS 160 KB");

    const unsigned char *words[MATRICES], *scales[MATRICES], *codes, *exponents;
    uint32_t tile_bytes, window, wave, piece_offset, scale_offset, codes_offset[2], exponents_offset;
    bool scale_lane; /* lanes 0..15: the ones that bring the scale words of the wavefront's own column block */
    uint32_t read_at[BYTES ? 8 : 4], scale_at[STRIP], vector_at[BYTES ? 8 : 4], vector_scale_at, operand_at, shift;

    /* the tile's columns of K step `at` into stage `stage` (every wavefront reads them: behind the barrier that ends the
     * reads of the stage): eight groups of eight columns, two a wavefront: the column block it prepares, and that block's
     * scale words (every wavefront issues the same number of loads: the waits count them) */
    __device__ __forceinline__ void issue_vectors(uint32_t stage, uint32_t at) const
    {
        const uint32_t base = window + stage * STAGE_BYTES;
#pragma unroll
        for (uint32_t part = 0; part < 2u; part++) {
            load_to_lds_16(codes + (uint64_t)at * 128u, codes_offset[part], base + VECTOR_AT + (2u * wave + part) * 1024u);
        }
        if (scale_lane) { /* its own sixteen columns' scale words, a lane a column: sixteen cache lines a wavefront, not 64 */
            load_to_lds_4(exponents + (uint64_t)at * 4u, exponents_offset, base + VECTOR_SCALE_AT + wave * 64u);
        }
    }

    /* the wavefront's own weights and their scales of K step `at` into its part of stage `stage` (no other wavefront
     * reads that part: once this one has read it, it may be asked for again) */
    __device__ __forceinline__ void issue_weights(uint32_t stage, uint32_t at) const
    {
        const uint32_t mine = window + stage * STAGE_BYTES + wave * WAVE_BYTES;
#pragma unroll
        for (uint32_t m = 0; m < MATRICES; m++) {
#pragma unroll
            for (uint32_t n = 0; n < STRIP; n++) {
#pragma unroll
                for (uint32_t part = 0; part < TILE_LOADS; part++) {
                    load_to_lds_16(words[m] + (uint64_t)n * tile_bytes + (uint64_t)at * STEP_BYTES + part * 1024u, piece_offset,
                                   mine + (m * STRIP + n) * STEP_BYTES + part * 1024u);
                }
            }
        }
#pragma unroll
        for (uint32_t m = 0; m < MATRICES; m++) {
            load_to_lds_4(scales[m] + (uint64_t)at * (BYTES ? 4u : 64u), scale_offset, mine + SCALES_AT + m * 256u);
        }
    }

    __device__ __forceinline__ void issue(uint32_t stage, uint32_t at) const
    {
        issue_vectors(stage, at); /* first: this wavefront waits for them a step before the weights */
        issue_weights(stage, at);
    }

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

    /* The wavefront's own column block of a stage, from the codes as they landed (a column's 128 bytes in the order the
     * quantizer writes them) to the MFMA's operand, in place: [half of the operand][lane][16 bytes], which every
     * wavefront then reads with two 16-byte reads a lane and no bank conflict. Only this wavefront touches the block
     * before the next barrier. */
    __device__ __forceinline__ void prepare_columns(uint32_t stage) const
    {
        uint32_t at = window + stage * STAGE_BYTES + VECTOR_AT + wave * 2048u;
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

    /* one K step of LIVE column blocks (a constant: the MFMAs of a step stay one straight line) */
    template <uint32_t LIVE>
    __device__ __forceinline__ void consume(uint32_t stage, float4_t (&chain)[TILES][WIDE_COLUMN_BLOCKS]) const
    {
        /* the stage's addresses, once a step: every read below is one of them plus a constant */
        uint32_t base = window + stage * STAGE_BYTES, mine = base + wave * WAVE_BYTES;
        asm volatile("" : "+s"(base), "+s"(mine));
        uint32_t a_at[BYTES ? 8 : 4], a_scale_at[STRIP], b_at = base + operand_at, b_scale_at = base + vector_scale_at;
#pragma unroll
        for (uint32_t v = 0; v < (BYTES ? 8u : 4u); v++) {
            a_at[v] = mine + read_at[v];
            asm volatile("" : "+v"(a_at[v]));
        }
#pragma unroll
        for (uint32_t n = 0; n < STRIP; n++) {
            a_scale_at[n] = mine + scale_at[n];
            asm volatile("" : "+v"(a_scale_at[n]));
        }
        asm volatile("" : "+v"(b_at), "+v"(b_scale_at));
        int8_vector b[LIVE];
        uint32_t scale_b[LIVE];
        float float_scale_b[LIVE];
#pragma unroll
        for (uint32_t j = 0; j < LIVE; j++) {
            const uint4_t low = lds_read<uint4_t>(b_at + VECTOR_AT + j * 2048u), high = lds_read<uint4_t>(b_at + VECTOR_AT + j * 2048u + 1024u);
            b[j] = (int8_vector){(int)low.x, (int)low.y, (int)low.z, (int)low.w, (int)high.x, (int)high.y, (int)high.z, (int)high.w};
            if constexpr (B128) {
                float_scale_b[j] = lds_read<float>(b_scale_at + VECTOR_SCALE_AT + j * 64u);
            } else {
                scale_b[j] = lds_read<unsigned char>(b_scale_at + VECTOR_SCALE_AT + j * 64u);
            }
        }
        __builtin_amdgcn_s_setprio(1); /* the wavefront that feeds the matrix unit goes first at the issue */
#pragma unroll
        for (uint32_t tile = 0; tile < TILES; tile++) {
            int8_vector a = {0, 0, 0, 0, 0, 0, 0, 0};
            if constexpr (B128) {
                const float float_scale_a = lds_read<float>(mine + SCALES_AT + (tile / STRIP) * 256u);
#pragma unroll
                for (uint32_t v = 0; v < 8u; v++) {
                    const uint2_t w = lds_read<uint2_t>(a_at[v] + tile * STEP_BYTES);
                    a[v] = (int)__builtin_amdgcn_perm(w.y, w.x, shift);
                }
#pragma unroll
                for (uint32_t j = 0; j < LIVE; j++) {
                    const float scale = __fmul_rn(float_scale_a, float_scale_b[j]);
                    const float4_t step = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b[j], (float4_t){0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0, 127, 0, 127);
#pragma unroll
                    for (uint32_t v = 0; v < 4u; v++) {
                        chain[tile][j][v] = __fmaf_rn(step[v], scale, chain[tile][j][v]);
                    }
                }
                continue;
            }
            const uint32_t scale_a = lds_read<unsigned char>(a_scale_at[tile % STRIP] + SCALES_AT + (tile / STRIP) * 256u);
            if constexpr (BYTES) {
#pragma unroll
                for (uint32_t v = 0; v < 8u; v++) {
                    const uint2_t w = lds_read<uint2_t>(a_at[v] + tile * STEP_BYTES);
                    a[v] = (int)__builtin_amdgcn_perm(w.y, w.x, shift);
                }
            } else {
#pragma unroll
                for (uint32_t T = 0; T < 4u; T++) {
                    /* a byte of the result: the output's nibble of w.x below that of w.y. Rotating w.x right by 0 or 4
                     * and w.y left by 4 or 0 puts them there; the mask picks */
                    const uint2_t w = lds_read<uint2_t>(a_at[T] + tile * STEP_BYTES);
                    const uint32_t low = __builtin_amdgcn_alignbit(w.x, w.x, shift), high = __builtin_amdgcn_alignbit(w.y, w.y, 28u + shift);
                    a[T] = (int)((low & NIBBLE_MASK) | (high & ~NIBBLE_MASK));
                }
            }
#pragma unroll
            for (uint32_t j = 0; j < LIVE; j++) {
                if constexpr (BYTES) {
                    chain[tile][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b[j], chain[tile][j], 0, 0, 0, (int)scale_a, 0, (int)scale_b[j]);
                } else {
                    chain[tile][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b[j], chain[tile][j], 4, 0, 0, (int)scale_a, 0, (int)scale_b[j]);
                }
            }
        }
        __builtin_amdgcn_s_setprio(0);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* the stage is read before the next barrier */
    }

    /* K step `step` of `total`, in stage `stage`; AHEAD = how many steps follow it, capped at 2 (a constant, so that
     * the steady loop carries no test) */
    template <uint32_t LIVE, uint32_t AHEAD>
    __device__ __forceinline__ void one_step(uint32_t step, uint32_t stage, float4_t (&chain)[TILES][WIDE_COLUMN_BLOCKS]) const
    {
        /* loads complete in the order they are issued: "at most N outstanding" names the oldest that have landed.
         * This step's have landed once nothing but the later step's is outstanding */
        wait_loads<AHEAD >= 1u ? STAGE_LOADS : 0u>();
        /* behind this barrier every wavefront's weights and prepared column block of this step are in LDS, and
         * every wavefront has read the step before: its stage may be asked for again */
        __syncthreads();
        const uint32_t behind = stage == 0u ? DEPTH - 1u : stage - 1u, ahead = stage + 1u == DEPTH ? 0u : stage + 1u;
        if constexpr (AHEAD >= 2u) {
            issue(behind, step + 2u);
        }
        consume<LIVE>(stage, chain);
        if constexpr (AHEAD >= 1u) { /* the next step's columns, which this wavefront asked for, have landed: prepare them */
            wait_loads<WEIGHT_LOADS + (AHEAD >= 2u ? STAGE_LOADS : 0u)>();
            prepare_columns(ahead);
        }
    }

    /* all `total` K steps of LIVE live column blocks; every wavefront of the block calls it (barriers inside) */
    template <uint32_t LIVE>
    __device__ __forceinline__ void steps(uint32_t total, float4_t (&chain)[TILES][WIDE_COLUMN_BLOCKS]) const
    {
        if constexpr (DEPTH == 2u) {
            /* Two stages. A wavefront's weights of a step are asked for two steps ahead, as soon as the wavefront itself has
             * read the stage they go to (its part is its own); the tile's columns one step ahead, behind the barrier that
             * ends every wavefront's reads of their stage; they are prepared once they have landed, before the barrier
             * that opens their step. Outstanding at the top of step k, oldest first: the weights of k, the columns of k,
             * the weights of k + 1. */
            issue(0u, 0u);
            if (total > 1u) {
                issue_weights(1u, 1u);
            }
            for (uint32_t step = 0; step < total; step++) {
                if (step + 1u < total) {
                    wait_loads<WEIGHT_LOADS>();
                } else {
                    wait_loads<0>();
                }
                prepare_columns(step % 2u);
                __syncthreads(); /* every wavefront has read the step before and brought and prepared its part of this one */
                if (step + 1u < total) {
                    issue_vectors((step + 1u) % 2u, step + 1u);
                }
                consume<LIVE>(step % 2u, chain);
                if (step + 2u < total) {
                    issue_weights(step % 2u, step + 2u);
                }
            }
            return;
        }
        static_assert(DEPTH == 2u || DEPTH == 3u, "the waits are written out for one or two stages ahead");
        issue(0u, 0u);
        if (total > 1u) {
            issue(1u, 1u);
            wait_loads<WEIGHT_LOADS + STAGE_LOADS>();
        } else {
            wait_loads<WEIGHT_LOADS>();
        }
        prepare_columns(0u);
        uint32_t stage = 0, step = 0;
        for (; step + 2u < total; step++) {
            one_step<LIVE, 2u>(step, stage, chain);
            stage = stage + 1u == DEPTH ? 0u : stage + 1u;
        }
        if (step + 1u < total) {
            one_step<LIVE, 1u>(step, stage, chain);
            stage = stage + 1u == DEPTH ? 0u : stage + 1u;
            step++;
        }
        one_step<LIVE, 0u>(step, stage, chain);
    }

    /* live_blocks: the tile's column blocks that hold a pair, the same in every lane of the block; the sums of the
     * others stay what they were */
    __device__ __forceinline__ void whole(uint32_t total, uint32_t live_blocks, float4_t (&chain)[TILES][WIDE_COLUMN_BLOCKS]) const
    {
        static_assert(WIDE_COLUMN_BLOCKS == 4u, "one instance a count of live column blocks");
        switch (live_blocks) {
        case 1u:
            steps<1>(total, chain);
            break;
        case 2u:
            steps<2>(total, chain);
            break;
        case 3u:
            steps<3>(total, chain);
            break;
        default:
            steps<4>(total, chain);
            break;
        }
    }

    /* matrices: arena addresses of the stored matrices; block_strip: the block's first strip (of STRIP tiles) is
     * WIDE_WAVES block_strip; vector_codes / vector_exponents: vector 0's codes and scale codes; vectors: this lane's
     * two columns' vectors for the codes' loads (lane / 8 of groups 2 wave, 2 wave + 1) and its column's for the scale
     * words' load (column 16 wave + lane % 16: lanes 0..15 bring them) */
    __device__ __forceinline__ void place(const unsigned char *const (&matrices)[MATRICES], uint32_t outputs, uint32_t inputs,
                                          uint32_t block_strip, const unsigned char *vector_codes, const unsigned char *vector_exponents,
                                          const uint32_t (&code_vectors)[2], uint32_t exponent_vector, uint32_t window_address,
                                          uint32_t wave_index, uint32_t lane, uint32_t &tile0_out)
    {
        const uint32_t tiles = outputs / 16u;
        const uint32_t o = lane % 16u, g = lane / 16u, G = o % 8u, parity = o / 8u, ld = g / 2u, q = g % 2u;
        const uint32_t strip = block_strip * WIDE_WAVES + wave_index;
        /* a strip that reaches past the last tile reads the last tiles again; its surplus sums are not stored */
        const uint32_t tile0 = strip * STRIP + STRIP <= tiles ? strip * STRIP : tiles - STRIP;
        tile0_out = tile0;
        const uint32_t steps = inputs / 128u;
        tile_bytes = steps * STEP_BYTES;
        window = window_address;
        wave = wave_index;
        codes = vector_codes;
        exponents = vector_exponents;
        if constexpr (BYTES) {
            const uint32_t scale_rows = (outputs + 31u) / 32u, row0 = B128 ? tile0 / 8u : tile0 / 2u;
#pragma unroll
            for (uint32_t m = 0; m < MATRICES; m++) {
                words[m] = matrices[m] + (uint64_t)tile0 * steps * STEP_BYTES;
                scales[m] = matrices[m] + (uint64_t)outputs * inputs + (uint64_t)row0 * (inputs / 32u);
            }
            piece_offset = 16u * (lane ^ ((lane >> 3) & 3u));
            /* the strip's tiles lie in one or two rows of scales (32 outputs a row): lanes past them ask for the last again,
             * so that a load touches two cache lines and not one a lane */
            const uint32_t rows_needed = (tile0 + STRIP - 1u) / 2u - row0;
            static_assert(STRIP <= 2u, "a strip of one-byte weights spans two rows of scales at most");
            (void)scale_rows;
            scale_offset = B128 ? 0u : (lane < rows_needed ? lane : rows_needed) * (inputs / 32u);
#pragma unroll
            for (uint32_t v = 0; v < 8u; v++) {
                const uint32_t group = 2u * (v / 4u) + g / 2u, t = v % 4u;
                read_at[v] = 16u * (32u * group + 4u * G + (t ^ (G / 2u))) + 8u * (g % 2u);
            }
#pragma unroll
            for (uint32_t n = 0; n < STRIP; n++) {
                scale_at[n] = 4u * ((tile0 + n) / 2u - row0) + g;
            }
            shift = parity == 0u ? 0x06020400u : 0x07030501u;
        } else {
            const uint32_t loads = inputs / 64u;
#pragma unroll
            for (uint32_t m = 0; m < MATRICES; m++) {
                words[m] = matrices[m] + (uint64_t)tile0 * steps * STEP_BYTES;
                scales[m] = matrices[m] + (uint64_t)outputs * inputs / 2u + (uint64_t)tile0 * loads * 32u;
            }
            /* piece p of a tile's K step lands in slot p ^ ((p / 8) % 4): LDS has 32 banks of 4 bytes, and the eight 8-byte
             * reads of sixteen lanes (G = 0 .. 7, twice) then fall on sixteen different banks */
            piece_offset = 16u * (lane ^ ((lane >> 3) & 3u));
            /* lanes past the strip's tiles read its last tile's words again */
            scale_offset = (lane / 16u < STRIP ? lane / 16u : STRIP - 1u) * (loads * 32u) + (lane % 16u) * 4u;
#pragma unroll
            for (uint32_t T = 0; T < 4u; T++) {
                read_at[T] = 16u * (32u * ld + 4u * G + (T ^ (G / 2u))) + 8u * q;
            }
#pragma unroll
            for (uint32_t n = 0; n < STRIP; n++) {
                scale_at[n] = n * 64u + (8u * ld + G) * 4u + 2u * q + parity;
            }
            shift = 4u * parity;
        }
        /* the columns' codes: lane L of a load holds slot L % 8 of column L / 8 of its group of eight and asks for
         * that column's piece (L % 8) ^ (L / 8) ^ (the group's parity); a column block of 16 columns is two groups
         * (2,048 bytes). With the parity the 32 lanes of a pass of prepare_columns' reads fall on every bank pair of
         * their half twice, not four times */
#pragma unroll
        for (uint32_t part = 0; part < 2u; part++) {
            codes_offset[part] = code_vectors[part] * inputs + 16u * ((lane % 8u) ^ (lane / 8u) ^ part);
        }
        exponents_offset = exponent_vector * (inputs / 32u);
        scale_lane = lane < 16u;
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
    }
};

#endif
