/*
 * strip_device.cuh -- a wavefront's chain over a strip of weight tiles for a few vectors (at most eight columns): what
 * the routed experts' job-table kernels and the trunk's thin kernels share. MFMA operand layout on gfx950, as measured
 * on the card: A (fp4) lane l: row l % 16, element e = 8 v + n (register v, nibble n) is k = 32 (l / 16) + e; B (fp8)
 * lane l: column l % 16, element e = 4 v + b is k = 64 (e / 16) + 16 (l / 16) + e % 16; scale of lane l: row or column
 * l % 16, inputs block l / 16; D lane l: column l % 16, rows 4 (l / 16) + v.
 */
#ifndef STRIP_DEVICE_CUH
#define STRIP_DEVICE_CUH

#include "linear_device.cuh"

/* A wavefront's part of a strip: MATRICES matrices (gate and up, or down alone) x STRIP tiles, K steps [first, last).
 * LDS window of a wavefront: DEPTH stages; a stage: MATRICES x STRIP x 1,024 bytes of weights, MATRICES x 256 bytes
 * of their scales (a matrix's STRIP tiles x 64), 1,024 bytes of the vectors' codes (8 columns x 128) and 256 bytes
 * holding their scale words. */
/* B128 (one-byte weights alone): the scales are float32, one for every 128 outputs x 128 inputs of a matrix and one for
 * every 128 values of a vector, in place of the E8M0 codes; a K step's MFMA then runs from zero with scales of one and its
 * sums enter the chain by one fused multiply-add with the product of the two scales. */
/* NATIVE: the matrices are stored in gfx950's lane order (WEIGHT_FORMAT_E2M1_GFX950, _E4M3_GFX950): a lane's 16 bytes of
 * a tile's K step (and, of one-byte weights, the 16 bytes 1,024 further) are its A operand as they lie, so a stage's
 * tiles are read with one or two 16-byte LDS reads and no arithmetic; the scale codes of 4-bit weights are a word a lane
 * for the strip's four tiles (a group of 64 outputs), its byte picked by the matrix instruction; with B128 the scales are
 * E4M3_BLOCK128's float32 words where they are. */
template <uint32_t MATRICES, bool BYTES, bool B128 = false, bool NATIVE = false>
struct strip_chain {
    static_assert(BYTES || !B128, "float32 scales go with one-byte weights");
    static constexpr uint32_t STRIP = BYTES ? 2u : 4u; /* tiles of a strip: 4 KB of every matrix a stage either way */
    static constexpr uint32_t STEP_BYTES = BYTES ? BYTE_STEP_BYTES : NIBBLE_STEP_BYTES;
    static constexpr uint32_t TILE_LOADS = STEP_BYTES / 1024u; /* 16-byte-a-lane loads of a tile's step */
    static constexpr uint32_t TILES = MATRICES * STRIP;
    static constexpr uint32_t DEPTH = MATRICES == 2u ? 2u : 3u;
    static constexpr uint32_t SCALES_AT = TILES * STEP_BYTES;
    static constexpr uint32_t VECTOR_AT = SCALES_AT + MATRICES * 256u;
    static constexpr uint32_t VECTOR_SCALE_AT = VECTOR_AT + 1024u;
    static constexpr uint32_t STAGE_BYTES = VECTOR_SCALE_AT + 256u;
    static constexpr uint32_t WINDOW_BYTES = DEPTH * STAGE_BYTES;
    static constexpr uint32_t STAGE_LOADS = TILES * TILE_LOADS + MATRICES + 2u;
    static_assert(STAGE_LOADS * (DEPTH - 1u) < 64u, "vmcnt has six bits");

    const unsigned char *words[MATRICES];  /* the strip's first tile, the chain's first step, of each matrix */
    const unsigned char *scales[MATRICES]; /* the same of the scale words */
    const unsigned char *codes;            /* the vectors' codes at the chain's first step (row 0) */
    const unsigned char *exponents;        /* the vectors' scale codes at the chain's first step (row 0) */
    uint32_t tile_bytes;                    /* from a tile to the next */
    uint32_t window;                        /* LDS address of the wavefront's window */
    uint32_t piece_offset;                  /* this lane's 16-byte piece of a step of a tile */
    uint32_t scale_offset;                  /* this lane's scale word of a stage: tile lane / 16, word lane % 16 */
    uint32_t codes_offset;                  /* this lane's 16-byte piece of the vectors' codes of a step */
    uint32_t exponents_offset;              /* this lane's vector's scale word of a step */
    uint32_t read_at[BYTES ? 8 : 4];        /* LDS byte offsets of its 8-byte pieces inside a tile of a stage */
    uint32_t scale_at[STRIP];               /* LDS byte offset of its scale byte of tile n inside a matrix's scales */
    uint32_t vector_at[BYTES ? 8 : 4];      /* LDS byte offsets of its pieces of its vector */
    uint32_t vector_scale_at;               /* LDS byte offset of its vector's scale byte */
    uint32_t shift;                         /* nibbles: 0 the even ones (outputs 0..7 of a tile), 4 the odd ones;
                                             * bytes: the byte selector of the same choice */

    __device__ __forceinline__ void issue(uint32_t stage, uint32_t at) const
    {
        const uint32_t base = window + stage * STAGE_BYTES;
#pragma unroll
        for (uint32_t m = 0; m < MATRICES; m++) {
#pragma unroll
            for (uint32_t n = 0; n < STRIP; n++) {
#pragma unroll
                for (uint32_t part = 0; part < TILE_LOADS; part++) {
                    load_to_lds_16(words[m] + (uint64_t)n * tile_bytes + (uint64_t)at * STEP_BYTES + part * 1024u, piece_offset,
                                   base + (m * STRIP + n) * STEP_BYTES + part * 1024u);
                }
            }
        }
#pragma unroll
        for (uint32_t m = 0; m < MATRICES; m++) {
            load_to_lds_4(scales[m] + (uint64_t)at * (BYTES ? 4u : NATIVE ? 256u : 64u), scale_offset, base + SCALES_AT + m * 256u);
        }
        load_to_lds_16(codes + (uint64_t)at * 128u, codes_offset, base + VECTOR_AT);
        load_to_lds_4(exponents + (uint64_t)at * 4u, exponents_offset, base + VECTOR_SCALE_AT);
    }

    template <typename T>
    __device__ static __forceinline__ T lds_read(uint32_t address)
    {
        return *(const __attribute__((address_space(3))) T *)(uintptr_t)address;
    }

    /* tile T of a stage and the tiles behind it, stored in gfx950's lane order (the number of the scale code's byte in
     * its word is part of the instruction: a constant) */
    template <uint32_t T>
    __device__ __forceinline__ void native_tiles(uint32_t base, const int8_vector &b, uint32_t scale_b, float4_t (&chain)[TILES]) const
    {
        const uint4_t first = lds_read<uint4_t>(base + T * STEP_BYTES + piece_offset);
        if constexpr (B128) { /* scale_b: the bits of the column's float32 scale */
            const uint4_t second = lds_read<uint4_t>(base + T * STEP_BYTES + 1024u + piece_offset);
            const float scale = __fmul_rn(lds_read<float>(base + SCALES_AT + (T / STRIP) * 256u), __uint_as_float(scale_b));
            const int8_vector a = {(int)first.x, (int)first.y, (int)first.z, (int)first.w, (int)second.x, (int)second.y, (int)second.z, (int)second.w};
            const float4_t step = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, (float4_t){0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0, 127, 0, 127);
#pragma unroll
            for (uint32_t v = 0; v < 4u; v++) {
                chain[T][v] = __fmaf_rn(step[v], scale, chain[T][v]);
            }
        } else if constexpr (BYTES) {
            const uint4_t second = lds_read<uint4_t>(base + T * STEP_BYTES + 1024u + piece_offset);
            const uint32_t scale_a = lds_read<unsigned char>(base + SCALES_AT + (T / STRIP) * 256u + scale_at[T % STRIP]);
            const int8_vector a = {(int)first.x, (int)first.y, (int)first.z, (int)first.w, (int)second.x, (int)second.y, (int)second.z, (int)second.w};
            chain[T] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, chain[T], 0, 0, 0, (int)scale_a, 0, (int)scale_b);
        } else {
            const uint32_t scale_a = lds_read<uint32_t>(base + SCALES_AT + (T / STRIP) * 256u + scale_offset);
            const int8_vector a = {(int)first.x, (int)first.y, (int)first.z, (int)first.w, 0, 0, 0, 0};
            chain[T] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, chain[T], 4, 0, T % STRIP, (int)scale_a, 0, (int)scale_b);
        }
        if constexpr (T + 1u < TILES) {
            native_tiles<T + 1u>(base, b, scale_b, chain);
        }
    }

    __device__ __forceinline__ void consume(uint32_t stage, float4_t (&chain)[TILES]) const
    {
        const uint32_t base = window + stage * STAGE_BYTES;
        int8_vector b;
        if constexpr (BYTES) {
#pragma unroll
            for (uint32_t v = 0; v < 8u; v++) {
                b[v] = (int)lds_read<uint32_t>(base + VECTOR_AT + vector_at[v]);
            }
        } else {
#pragma unroll
            for (uint32_t part = 0; part < 4u; part++) {
                const uint2_t pair = lds_read<uint2_t>(base + VECTOR_AT + vector_at[part]);
                b[2u * part] = (int)__builtin_amdgcn_perm(pair.y, pair.x, 0x05010400u);
                b[2u * part + 1u] = (int)__builtin_amdgcn_perm(pair.y, pair.x, 0x07030602u);
            }
        }
        uint32_t scale_b = 0;
        float float_scale_b = 0.0f;
        if constexpr (B128) {
            float_scale_b = lds_read<float>(base + VECTOR_SCALE_AT + vector_scale_at);
        } else {
            scale_b = lds_read<unsigned char>(base + VECTOR_SCALE_AT + vector_scale_at);
        }
        if constexpr (NATIVE) {
            native_tiles<0>(base, b, B128 ? __float_as_uint(float_scale_b) : scale_b, chain);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            return;
        }
#pragma unroll
        for (uint32_t tile = 0; tile < TILES; tile++) {
            int8_vector a = {0, 0, 0, 0, 0, 0, 0, 0};
            if constexpr (B128) {
                const float scale = __fmul_rn(lds_read<float>(base + SCALES_AT + (tile / STRIP) * 256u), float_scale_b);
#pragma unroll
                for (uint32_t v = 0; v < 8u; v++) {
                    const uint2_t w = lds_read<uint2_t>(base + tile * STEP_BYTES + read_at[v]);
                    a[v] = (int)__builtin_amdgcn_perm(w.y, w.x, shift);
                }
                const float4_t step = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, (float4_t){0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0, 127, 0, 127);
#pragma unroll
                for (uint32_t v = 0; v < 4u; v++) {
                    chain[tile][v] = __fmaf_rn(step[v], scale, chain[tile][v]);
                }
                continue;
            }
            const uint32_t scale_a = lds_read<unsigned char>(base + SCALES_AT + (tile / STRIP) * 256u + scale_at[tile % STRIP]);
            if constexpr (BYTES) {
#pragma unroll
                for (uint32_t v = 0; v < 8u; v++) { /* every other byte of eight: this lane's output row of the two */
                    const uint2_t w = lds_read<uint2_t>(base + tile * STEP_BYTES + read_at[v]);
                    a[v] = (int)__builtin_amdgcn_perm(w.y, w.x, shift);
                }
                chain[tile] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, chain[tile], 0, 0, 0, (int)scale_a, 0, (int)scale_b);
            } else {
#pragma unroll
                for (uint32_t T = 0; T < 4u; T++) {
                    const uint2_t w = lds_read<uint2_t>(base + tile * STEP_BYTES + read_at[T]);
                    a[T] = (int)(((w.x >> shift) & NIBBLE_MASK) | (((w.y >> shift) & NIBBLE_MASK) << 4));
                }
                chain[tile] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, chain[tile], 4, 0, 0, (int)scale_a, 0, (int)scale_b);
            }
        }
        /* the stage is read once its values are in registers; only then may it be filled again */
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }

    /* The whole chain of `total` steps (the same in every lane). The window is idle on entry and on return. */
    __device__ __forceinline__ void whole(uint32_t total, float4_t (&chain)[TILES]) const
    {
        uint32_t done = 0;
        if (total >= 2u * DEPTH) {
#pragma unroll
            for (uint32_t i = 0; i < DEPTH; i++) {
                issue(i, i);
            }
            /* the steady state: a step consumed has DEPTH - 1 whole stages asked for behind it, and asks for one more */
            for (; done + 2u * DEPTH <= total; done += DEPTH) {
#pragma unroll
                for (uint32_t i = 0; i < DEPTH; i++) {
                    wait_loads<STAGE_LOADS * (DEPTH - 1u)>();
                    consume(i, chain);
                    issue(i, done + i + DEPTH);
                }
            }
        } else {
#pragma unroll
            for (uint32_t i = 0; i < DEPTH; i++) {
                if (i < total) {
                    issue(i, i);
                }
            }
        }
        /* the last steps, fewer than 2 DEPTH: the stages behind a step grow fewer */
#pragma unroll
        for (uint32_t round = 0; round < 2u; round++) {
#pragma unroll
            for (uint32_t i = 0; i < DEPTH; i++) {
                const uint32_t at = done + round * DEPTH + i;
                if (at < total) {
                    const uint32_t behind = total - 1u - at;
                    if (behind >= DEPTH - 1u) {
                        wait_loads<STAGE_LOADS * (DEPTH - 1u)>();
                    } else if (behind == 1u) {
                        wait_loads<STAGE_LOADS>();
                    } else {
                        wait_loads<0>();
                    }
                    consume(i, chain);
                    if (at + DEPTH < total) {
                        issue(i, at + DEPTH);
                    }
                }
            }
        }
    }

    /* matrices: arena addresses of the MATRICES stored matrices; strip: the strip of tiles; first: the chain's first K
     * step; vector_codes / vector_exponents: row 0 of the vectors' codes and scale codes; vector_rows: the rows of
     * columns 0..7 (columns 8..15 never hold a row of a job: they mirror columns 0..7 and are not stored) */
    __device__ __forceinline__ void place(const unsigned char *const (&matrices)[MATRICES], uint32_t outputs, uint32_t inputs,
                                          uint32_t strip, uint32_t first, const unsigned char *vector_codes,
                                          const unsigned char *vector_exponents, const uint32_t (&vector_rows)[8],
                                          uint32_t window_address, uint32_t lane)
    {
        static_assert(DEPTH == 2u || DEPTH == 3u, "the waits of whole() are written out for two or three stages");
        const uint32_t tiles = outputs / 16u;
        const uint32_t o = lane % 16u, g = lane / 16u, G = o % 8u, parity = o / 8u, ld = g / 2u, q = g % 2u;
        /* a strip that reaches past the last tile reads the last tiles again; its surplus sums are not stored */
        const uint32_t tile0 = strip * STRIP + STRIP <= tiles ? strip * STRIP : tiles - STRIP;
        const uint32_t steps = inputs / 128u;
        tile_bytes = steps * STEP_BYTES;
        window = window_address;
        codes = vector_codes + 128u * first;
        exponents = vector_exponents + 4u * first;
        if constexpr (BYTES) {
            /* WEIGHT_FORMAT_E4M3_SCALED (include/anemone/weight_format_seam.h:35-42 of the reference): bytes
             * [tile][group of 32 inputs][lane = 4 G + t][16], byte b of a lane: output 16 tile + G + 8 (b % 2), input
             * 32 group + 8 (b / 4) + 2 t + (b / 2) % 2; then one scale code for every 32 outputs x 32 inputs,
             * [ceil(outputs / 32)][inputs / 32]. A step is four groups, 128 pieces of 16 bytes. */
            /* B128: float32 [outputs / 128][inputs / 128] behind the codes: the strip's row of them, a word a K step (a row
             * of either kind of scales is inputs / 32 bytes) */
            const uint32_t scale_rows = (outputs + 31u) / 32u, row0 = B128 ? tile0 / 8u : tile0 / 2u;
#pragma unroll
            for (uint32_t m = 0; m < MATRICES; m++) {
                words[m] = matrices[m] + ((uint64_t)tile0 * steps + first) * STEP_BYTES;
                scales[m] = matrices[m] + (uint64_t)outputs * inputs + (uint64_t)row0 * (inputs / 32u) + 4u * first;
            }
            /* lane L of a load lands at slot L and asks for the piece L ^ (bits 3, 4 of L, as a number): the pieces
             * (group, G, t) of one t then lie in different banks for the readers */
            piece_offset = NATIVE ? 16u * lane : 16u * (lane ^ ((lane >> 3) & 3u)); /* gfx950's order: as stored */
            /* the strip's tiles lie in one or two rows of scales (32 outputs a row): lanes past them ask for the last again,
             * so that a load touches two cache lines and not one a lane */
            const uint32_t rows_needed = (tile0 + STRIP - 1u) / 2u - row0;
            static_assert(STRIP <= 2u, "a strip of one-byte weights spans two rows of scales at most");
            (void)scale_rows;
            scale_offset = B128 ? 0u : (lane < rows_needed ? lane : rows_needed) * (inputs / 32u);
            /* this lane's operand registers 4 L + t: group 2 L + g / 2, piece t of output row G, its half g % 2 */
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
            /* WEIGHT_FORMAT_E2M1_SCALED (include/anemone/weight_format_seam.h:26-34 of the reference) */
            const uint32_t loads = inputs / 64u;
#pragma unroll
            for (uint32_t m = 0; m < MATRICES; m++) {
                words[m] = matrices[m] + ((uint64_t)tile0 * steps + first) * STEP_BYTES;
                scales[m] = matrices[m] + (uint64_t)outputs * inputs / 2u + ((uint64_t)tile0 * loads + 2u * first) * 32u;
            }
            if constexpr (NATIVE) {
                /* WEIGHT_FORMAT_E2M1_GFX950: words [tile][K step][lane][16 bytes]; scale codes uint32
                 * [group of four tiles][K step][lane], byte n of a word the code of tile n of the group. The format holds
                 * whole groups (outputs a multiple of 64), so a strip is one. */
#pragma unroll
                for (uint32_t m = 0; m < MATRICES; m++) {
                    scales[m] = matrices[m] + (uint64_t)outputs * inputs / 2u + ((uint64_t)(tile0 / 4u) * steps + first) * 256u;
                }
                piece_offset = 16u * lane;
                scale_offset = 4u * lane;
                shift = 0;
            } else {
                /* lane L of a 16-byte load lands at bytes 16 L of the tile's stage and asks for the piece
                 * p = L ^ ((L / 8) % 4) of the step: LDS has 32 banks of 4 bytes, and the pieces of one T (p = 32 ld + 4 G + T,
                 * G = 0 .. 7) then lie in eight different groups of four banks for the sixteen lanes that read them together
                 * (measured: SQ_LDS_BANK_CONFLICT of the wide gate/up launch 1.68e8 -> 1.9e7 cycles); every 16 lanes still read
                 * 256 contiguous bytes of memory */
                piece_offset = 16u * (lane ^ ((lane >> 3) & 3u));
                /* scales: uint32 [tile][load][G]; lane L of the 4-byte load: tile L / 16, word L % 16 = 8 ld + G */
                scale_offset = (lane / 16u) * (loads * 32u) + (lane % 16u) * 4u;
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
        }
        /* the vectors: lane L of the 16-byte load holds slot L % 8 of column L / 8 and asks for that column's piece
         * (L % 8) ^ (L / 8) of the step, so that one piece of all columns lies in different banks; lane L of the
         * 4-byte load of their scale words serves column L % 8 (the readers take the copies of lanes 0..7) */
        uint32_t row_of_codes = 0, row_of_exponents = 0;
#pragma unroll
        for (uint32_t c = 0; c < 8u; c++) {
            row_of_codes = lane / 8u == c ? vector_rows[c] : row_of_codes;
            row_of_exponents = lane % 8u == c ? vector_rows[c] : row_of_exponents;
        }
        codes_offset = row_of_codes * inputs + 16u * ((lane % 8u) ^ (lane / 8u));
        exponents_offset = row_of_exponents * (inputs / 32u);
        const uint32_t column = o % 8u;
        if constexpr (BYTES) {
            /* register 4 L + t: word g of piece 4 L + t of the lane's column, as stored */
#pragma unroll
            for (uint32_t v = 0; v < 8u; v++) {
                vector_at[v] = 16u * (8u * column + (v ^ column)) + 4u * g;
            }
        } else {
            /* piece 4 (part / 2) + part % 2 + 2 (g % 2) of its column, bytes 8 (g / 2) .. + 7 */
#pragma unroll
            for (uint32_t part = 0; part < 4u; part++) {
                const uint32_t piece = 4u * (part / 2u) + part % 2u + 2u * (g % 2u);
                vector_at[part] = 16u * (8u * column + (piece ^ column)) + 8u * (g / 2u);
            }
        }
        vector_scale_at = B128 ? 4u * column : 4u * column + g;
    }
};

#endif
