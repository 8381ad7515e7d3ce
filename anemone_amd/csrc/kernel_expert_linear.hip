/*
 * kernel_expert_linear.hip -- the routed experts of the original FP4 weights on gfx950: gate and up products with the
 * hidden step, the down product, and the row sum. Entry names, records, launch shapes and rounding points follow the
 * reference (source/kernel_expert_linear.cu:157-231, 403-419; include/anemone/linear_records.h:45-99, 231-305):
 *   - weights WEIGHT_FORMAT_E2M1_SCALED exactly as stored (lane order words [tile][load][lane][step], E8M0 scales
 *     [tile][load][g] behind them; include/anemone/weight_format_seam.h:26-34), vectors as the quantizer writes them
 *     (E4M3 codes in lane order, E8M0 exponents per 32);
 *   - a product is cut in S slices of whole loads; a slice is one chain over its blocks of 32 inputs in ascending
 *     order; the S chains are added from +0 in order and the sum is rounded once to bfloat16;
 *   - the hidden step: g = min(gate, L), u = clamp(up, +-L), bf16(((g / (1 + exp(-g))) u) route weight), gate and up
 *     rounded to bfloat16 first.
 * The arithmetic form is the block-scaled one (the reference's native form, include/anemone/linear_records.h:63-66):
 * one v_mfma_scale_f32_16x16x128_f8f6f4 takes 128 inputs = four blocks of 32 with both E8M0 scale codes inside the
 * instruction and adds their terms to the running chain; E2M1 weights by E4M3 vector codes, no conversion.
 *
 * Work mapping (this build's own). What bounds a streaming kernel on this card, besides memory itself, is the number
 * of memory instructions: a compute unit takes one wavefront-wide load every 16 cycles whatever its width, which at
 * full memory speed leaves room for about six a KB of weights, and in practice far fewer. So:
 *   - a block is one strip of tiles (64 outputs of 4-bit weights, 32 of one-byte weights) of one job; a wavefront is one slice of the inputs, for the
 *     gate AND the up matrix (their sums meet in one lane for the hidden step, no exchange);
 *   - a stage is one K step (128 inputs) of all the wavefront's tiles: 1,024 bytes a tile go from memory straight
 *     into the wavefront's LDS window with one 16-byte-a-lane load (no registers in between), the tiles' 64 scale
 *     bytes each with one more load for every four tiles; two or three stages are on their way while one is used;
 *   - the codes of the job's (at most eight) vectors for the step and their scale codes travel the same way, one load
 *     each a stage, and serve every tile of the wavefront; nothing of the loop passes through registers, so the
 *     compiler has no wait of its own to place and the waits are this file's constants;
 *   - lane (o, g) of the MFMA needs output row o of inputs block g, which the stored form spreads over four stored
 *     lanes (t = 0..3) as the even (o < 8) or odd (o >= 8) nibbles of two words each: four 8-byte LDS reads, and two
 *     shifts, a shift and a bit-field insert a register.
 *
 * MFMA operand layout on gfx950, as measured on the card: A (fp4) lane l: row l % 16, element e = 8 v + n (register v,
 * nibble n) is k = 32 (l / 16) + e; B (fp8) lane l: column l % 16, element e = 4 v + b is k = 64 (e / 16) +
 * 16 (l / 16) + e % 16; scale of lane l: row or column l % 16, inputs block l / 16; D lane l: column l % 16, rows
 * 4 (l / 16) + v.
 */
#include "kernel_registry.h"
#include "linear_device.cuh"
#include "quantize_device.cuh"

/* A wavefront's part of a strip: MATRICES matrices (gate and up, or down alone) x STRIP tiles, K steps [first, last).
 * LDS window of a wavefront: DEPTH stages; a stage: MATRICES x STRIP x 1,024 bytes of weights, MATRICES x 256 bytes
 * of their scales (a matrix's STRIP tiles x 64), 1,024 bytes of the vectors' codes (8 columns x 128) and 256 bytes
 * holding their scale words. */
template <uint32_t MATRICES, bool BYTES>
struct strip_chain {
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
            load_to_lds_4(scales[m] + (uint64_t)at * (BYTES ? 4u : 64u), scale_offset, base + SCALES_AT + m * 256u);
        }
        load_to_lds_16(codes + (uint64_t)at * 128u, codes_offset, base + VECTOR_AT);
        load_to_lds_4(exponents + (uint64_t)at * 4u, exponents_offset, base + VECTOR_SCALE_AT);
    }

    template <typename T>
    __device__ static __forceinline__ T lds_read(uint32_t address)
    {
        return *(const __attribute__((address_space(3))) T *)(uintptr_t)address;
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
        const uint32_t scale_b = lds_read<unsigned char>(base + VECTOR_SCALE_AT + vector_scale_at);
#pragma unroll
        for (uint32_t tile = 0; tile < TILES; tile++) {
            int8_vector a = {0, 0, 0, 0, 0, 0, 0, 0};
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
            const uint32_t scale_rows = (outputs + 31u) / 32u, row0 = tile0 / 2u;
#pragma unroll
            for (uint32_t m = 0; m < MATRICES; m++) {
                words[m] = matrices[m] + ((uint64_t)tile0 * steps + first) * STEP_BYTES;
                scales[m] = matrices[m] + (uint64_t)outputs * inputs + (uint64_t)row0 * (inputs / 32u) + 4u * first;
            }
            /* lane L of a load lands at slot L and asks for the piece L ^ (bits 3, 4 of L, as a number): the pieces
             * (group, G, t) of one t then lie in different banks for the readers */
            piece_offset = 16u * (lane ^ ((lane >> 3) & 3u));
            /* the scale words of the step: lane L asks for scale row row0 + min(L, rows left) */
            const uint32_t rows_left = scale_rows - 1u - row0;
            scale_offset = (lane < rows_left ? lane : rows_left) * (inputs / 32u);
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
            /* lane L of a 16-byte load lands at bytes 16 L of the tile's stage and asks for the piece
             * p = L ^ (2 bit4(L) + bit5(L)) of the step: the pieces of one T (p = 32 ld + 4 G + T) then lie in
             * different LDS banks for the readers, and every 16 lanes still read 256 contiguous bytes of memory */
            piece_offset = 16u * (lane ^ (2u * ((lane >> 4) & 1u) + ((lane >> 5) & 1u)));
            /* scales: uint32 [tile][load][G]; lane L of the 4-byte load: tile L / 16, word L % 16 = 8 ld + G */
            scale_offset = (lane / 16u) * (loads * 32u) + (lane % 16u) * 4u;
#pragma unroll
            for (uint32_t T = 0; T < 4u; T++) {
                read_at[T] = 16u * (32u * ld + 4u * G + (T ^ (2u * (G / 4u) + ld))) + 8u * q;
            }
#pragma unroll
            for (uint32_t n = 0; n < STRIP; n++) {
                scale_at[n] = n * 64u + (8u * ld + G) * 4u + 2u * q + parity;
            }
            shift = 4u * parity;
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
        vector_scale_at = 4u * column + g;
    }
};

/* gate and up: block = S wavefronts (slices of the inputs); grid (ceil(output_size / 64), jobs) */
template <uint32_t S, bool BYTES>
__device__ static __forceinline__ void expert_gate_up(const struct expert_gate_up_arguments &arguments,
                                                      unsigned char *arena, uint16_t *strip_hidden = nullptr)
{
    typedef strip_chain<2, BYTES> chain_type;
    constexpr uint32_t TILES = chain_type::TILES, STRIP = chain_type::STRIP;
    __shared__ __attribute__((aligned(16))) unsigned char window[S][chain_type::WINDOW_BYTES];
    static_assert(chain_type::WINDOW_BYTES >= TILES * WAVE * 16u, "a wavefront's sums fit its idle window");
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + arguments.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x % WAVE, slice = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t column = lane % 16u;
    const bool live = column < job->row_count; /* a job holds at most eight rows */
    const uint32_t pair = live ? job->pair_index[column] : 0u;
    uint32_t rows[8]; /* the vectors' rows; columns without a row read row 0, and are never stored */
#pragma unroll
    for (uint32_t c = 0; c < 8u; c++) {
        rows[c] = c < job->row_count ? job->pair_index[c] / arguments.pairs_per_row : 0u;
    }
    const uint32_t steps = arguments.input_size / 128u;
    const uint32_t first = steps * slice / S, last = steps * (slice + 1u) / S;
    chain_type chain_of;
    const unsigned char *const matrices[2] = {arena + job->gate_offset, arena + job->up_offset};
    chain_of.place(matrices, arguments.output_size, arguments.input_size, blockIdx.x, first, arena + arguments.codes_offset,
                   arena + arguments.exponents_offset, rows, (uint32_t)(uintptr_t)(lds_pointer)&window[slice][0], lane);
    float4_t chain[TILES];
#pragma unroll
    for (uint32_t tile = 0; tile < TILES; tile++) {
        chain[tile] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
    }
    chain_of.whole(last - first, chain);
    /* the S chains meet in the windows, idle now: [slice][tile][lane] float4 */
    float4_t *sums = (float4_t *)&window[slice][0];
#pragma unroll
    for (uint32_t tile = 0; tile < TILES; tile++) {
        sums[tile * WAVE + lane] = chain[tile];
    }
    __syncthreads();
    /* wavefront w finishes the tiles n = w, w + S, ..: the S chains from +0, in order, then the hidden step */
    const uint32_t tiles = arguments.output_size / 16u;
    const uint32_t tile0 = blockIdx.x * STRIP + STRIP <= tiles ? blockIdx.x * STRIP : tiles - STRIP;
    for (uint32_t n = slice; n < STRIP; n += S) {
        if (!live || tile0 + n < blockIdx.x * STRIP) { /* a tile the strip before this one stores */
            continue;
        }
        float gate[4] = {0.0f, 0.0f, 0.0f, 0.0f}, up[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (uint32_t part = 0; part < S; part++) {
            const float4_t g4 = ((const float4_t *)&window[part][0])[n * WAVE + lane];
            const float4_t u4 = ((const float4_t *)&window[part][0])[(STRIP + n) * WAVE + lane];
#pragma unroll
            for (uint32_t v = 0; v < 4u; v++) {
                gate[v] = __fadd_rn(gate[v], g4[v]);
                up[v] = __fadd_rn(up[v], u4[v]);
            }
        }
        const float limit = arguments.activation_limit, weight = job->route_weight[column];
        uint16_t hidden[4];
#pragma unroll
        for (uint32_t v = 0; v < 4u; v++) {
            const float g = bf16_to_float(float_to_bf16(gate[v])), u = bf16_to_float(float_to_bf16(up[v]));
            const float bounded_gate = fminf(g, limit);
            const float bounded_up = fminf(fmaxf(u, -limit), limit);
            const float value = __fmul_rn(__fmul_rn(__fdiv_rn(bounded_gate, __fadd_rn(1.0f, det_expf(-bounded_gate))), bounded_up), weight);
            hidden[v] = float_to_bf16(value);
        }
        uint16_t *out = (uint16_t *)(arena + arguments.hidden_offset) + (uint64_t)pair * arguments.output_size +
                        (tile0 + n) * 16u + 4u * (lane / 16u);
        *(uint2_t *)out = (uint2_t){(uint32_t)hidden[0] | ((uint32_t)hidden[1] << 16), (uint32_t)hidden[2] | ((uint32_t)hidden[3] << 16)};
        if (strip_hidden != nullptr) { /* the producer's copy: [column][the strip's outputs] */
            uint16_t *copy = strip_hidden + column * (STRIP * 16u) + n * 16u + 4u * (lane / 16u);
#pragma unroll
            for (uint32_t v = 0; v < 4u; v++) {
                copy[v] = hidden[v];
            }
        }
    }
}

/* The producer: gate with up, then the quantization of the strip's hidden values, in one launch. A block of the
 * quantization is 32 consecutive outputs and a strip holds whole blocks (64 outputs of 4-bit weights, 32 of one-byte
 * weights), so the second step needs nothing of another block: the hidden values pass through LDS. One more row of
 * blocks (blockIdx.y = the jobs' number) quantizes, from memory, the pairs that stand in no job, as the quantizer's
 * own launch does. Grid (ceil(output_size / strip), jobs + 1). */
template <uint32_t S, bool BYTES>
__device__ static __forceinline__ void expert_gate_up_quantize(const struct expert_gate_up_quantize_arguments &arguments,
                                                               unsigned char *arena)
{
    typedef strip_chain<2, BYTES> chain_type;
    constexpr uint32_t STRIP_OUTPUTS = chain_type::STRIP * 16u;
    __shared__ uint16_t strip_hidden[LINEAR_MAXIMUM_ROWS][STRIP_OUTPUTS];
    __shared__ uint32_t routed[EXPERT_PRODUCER_MOST_PAIRS / 32u];
    const uint32_t tiles = arguments.output_size / 16u;
    const uint32_t tile0 = blockIdx.x * chain_type::STRIP + chain_type::STRIP <= tiles ? blockIdx.x * chain_type::STRIP : tiles - chain_type::STRIP;
    const uint32_t lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t width = arguments.output_size;
    const uint32_t first_output = blockIdx.x * STRIP_OUTPUTS; /* a last strip that reaches past the matrix starts earlier */
    if (blockIdx.y + 1u == gridDim.y) {
        /* the pairs no job holds: a bit a pair from the job table (a job a pair at most), then the quantizer's work */
        const struct expert_job_record *jobs = (const struct expert_job_record *)(arena + arguments.jobs_offset);
        if (threadIdx.x < EXPERT_PRODUCER_MOST_PAIRS / 32u) {
            uint32_t bits = 0;
            for (uint32_t job = 0; job < arguments.pair_count; job++) {
                for (uint32_t column = 0; column < jobs[job].row_count; column++) {
                    const uint32_t pair = jobs[job].pair_index[column];
                    bits |= pair / 32u == threadIdx.x ? 1u << (pair % 32u) : 0u;
                }
            }
            routed[threadIdx.x] = bits;
        }
        __syncthreads();
        for (uint32_t pair = wave; pair < arguments.pair_count; pair += S) {
            if ((routed[pair / 32u] >> (pair % 32u)) & 1u) {
                continue;
            }
            for (uint32_t at = lane; at < STRIP_OUTPUTS; at += WAVE) {
                const uint32_t index = tile0 * 16u + at;
                if (index < first_output) { /* whole blocks of 32 that the strip before this one takes */
                    continue;
                }
                const uint32_t bits = ((const uint16_t *)(arena + arguments.hidden_offset))[(uint64_t)pair * width + index];
                quantize_value(bits, index, arena + arguments.hidden_codes_offset + (uint64_t)pair * width,
                               arena + arguments.hidden_exponents_offset + (uint64_t)pair * (width / 32u),
                               (uint16_t *)(arena + arguments.hidden_operands_offset) + (uint64_t)pair * width);
            }
        }
        return;
    }
    const struct expert_gate_up_arguments plain = {arguments.jobs_offset, arguments.codes_offset, arguments.exponents_offset,
                                                   arguments.operands_offset, arguments.hidden_offset, arguments.output_size,
                                                   arguments.input_size, arguments.pair_count, arguments.pairs_per_row,
                                                   arguments.activation_limit, 0u};
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + arguments.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    expert_gate_up<S, BYTES>(plain, arena, &strip_hidden[0][0]);
    __syncthreads();
    for (uint32_t column = wave; column < job->row_count; column += S) {
        const uint64_t pair = job->pair_index[column];
        for (uint32_t at = lane; at < STRIP_OUTPUTS; at += WAVE) {
            if (tile0 * 16u + at < first_output) {
                continue;
            }
            quantize_value(strip_hidden[column][at], tile0 * 16u + at, arena + arguments.hidden_codes_offset + pair * width,
                           arena + arguments.hidden_exponents_offset + pair * (width / 32u),
                           (uint16_t *)(arena + arguments.hidden_operands_offset) + pair * width);
        }
    }
}

/* down: block = S wavefronts; grid (ceil(output_size / 64), jobs) */
template <uint32_t S, bool BYTES>
__device__ static __forceinline__ void expert_down(const struct expert_down_arguments &arguments, unsigned char *arena)
{
    typedef strip_chain<1, BYTES> chain_type;
    constexpr uint32_t TILES = chain_type::TILES, STRIP = chain_type::STRIP;
    __shared__ __attribute__((aligned(16))) unsigned char window[S][chain_type::WINDOW_BYTES];
    static_assert(chain_type::WINDOW_BYTES >= TILES * WAVE * 16u, "a wavefront's sums fit its idle window");
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + arguments.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x % WAVE, slice = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), column = lane % 16u;
    const bool live = column < job->row_count;
    const uint64_t pair = live ? job->pair_index[column] : 0u;
    uint32_t rows[8]; /* the vectors are the pairs' hidden vectors */
#pragma unroll
    for (uint32_t c = 0; c < 8u; c++) {
        rows[c] = c < job->row_count ? job->pair_index[c] : 0u;
    }
    const uint32_t steps = arguments.input_size / 128u;
    const uint32_t first = steps * slice / S, last = steps * (slice + 1u) / S;
    chain_type chain_of;
    const unsigned char *const matrices[1] = {arena + job->down_offset};
    chain_of.place(matrices, arguments.output_size, arguments.input_size, blockIdx.x, first, arena + arguments.codes_offset,
                   arena + arguments.exponents_offset, rows, (uint32_t)(uintptr_t)(lds_pointer)&window[slice][0], lane);
    float4_t chain[TILES];
#pragma unroll
    for (uint32_t tile = 0; tile < TILES; tile++) {
        chain[tile] = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
    }
    chain_of.whole(last - first, chain);
    float4_t *sums = (float4_t *)&window[slice][0];
#pragma unroll
    for (uint32_t tile = 0; tile < TILES; tile++) {
        sums[tile * WAVE + lane] = chain[tile];
    }
    __syncthreads();
    const uint32_t tiles = arguments.output_size / 16u;
    const uint32_t tile0 = blockIdx.x * STRIP + STRIP <= tiles ? blockIdx.x * STRIP : tiles - STRIP;
    for (uint32_t n = slice; n < STRIP; n += S) {
        if (!live || tile0 + n < blockIdx.x * STRIP) {
            continue;
        }
        float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (uint32_t part = 0; part < S; part++) {
            const float4_t d4 = ((const float4_t *)&window[part][0])[n * WAVE + lane];
#pragma unroll
            for (uint32_t v = 0; v < 4u; v++) {
                sum[v] = __fadd_rn(sum[v], d4[v]);
            }
        }
        uint16_t *out = (uint16_t *)(arena + arguments.output_offset) + pair * arguments.output_size + (tile0 + n) * 16u + 4u * (lane / 16u);
        *(uint2_t *)out = (uint2_t){(uint32_t)float_to_bf16(sum[0]) | ((uint32_t)float_to_bf16(sum[1]) << 16),
                                    (uint32_t)float_to_bf16(sum[2]) | ((uint32_t)float_to_bf16(sum[3]) << 16)};
    }
}

/* expert_gate_up_<S>, expert_down_<S>: the reference's entries, of WEIGHT_FORMAT_E2M1_SCALED experts. The _e4m3_
 * entries take WEIGHT_FORMAT_E4M3_SCALED experts (a format the reference stores and lays out but multiplies in its
 * trunk alone: no counterpart among its expert kernels); same records, same rounding points. */
#define EXPERT_ENTRIES(S)                                                                                         \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_gate_up_##S(struct expert_gate_up_arguments arguments, unsigned char *arena)                      \
    {                                                                                                             \
        expert_gate_up<S, false>(arguments, arena);                                                               \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_##S, expert_gate_up_arguments);                      \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_down_##S(struct expert_down_arguments arguments, unsigned char *arena)                            \
    {                                                                                                             \
        expert_down<S, false>(arguments, arena);                                                                  \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_down_##S, expert_down_arguments);                            \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_gate_up_e4m3_##S(struct expert_gate_up_arguments arguments, unsigned char *arena)                 \
    {                                                                                                             \
        expert_gate_up<S, true>(arguments, arena);                                                                \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_e4m3_##S, expert_gate_up_arguments);                 \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_down_e4m3_##S(struct expert_down_arguments arguments, unsigned char *arena)                       \
    {                                                                                                             \
        expert_down<S, true>(arguments, arena);                                                                   \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_down_e4m3_##S, expert_down_arguments);                       \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_gate_up_quantize_##S(struct expert_gate_up_quantize_arguments arguments, unsigned char *arena)    \
    {                                                                                                             \
        expert_gate_up_quantize<S, false>(arguments, arena);                                                      \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_quantize_##S, expert_gate_up_quantize_arguments);    \
    extern "C" __global__ void __launch_bounds__(S * WAVE)                                                        \
        expert_gate_up_quantize_e4m3_##S(struct expert_gate_up_quantize_arguments arguments, unsigned char *arena) \
    {                                                                                                             \
        expert_gate_up_quantize<S, true>(arguments, arena);                                                       \
    }                                                                                                             \
    ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_gate_up_quantize_e4m3_##S, expert_gate_up_quantize_arguments)
EXPERT_ENTRIES(1);
EXPERT_ENTRIES(2);
EXPERT_ENTRIES(4);
EXPERT_ENTRIES(8);

/* float32 sum of a row's bfloat16 pair outputs from +0 in ascending slot order; a thread takes
 * EXPERT_ROW_SUM_CHANNELS consecutive outputs (one 16-byte load a slot); grid (ceil(width / (8 x 256)), rows) */
extern "C" __global__ void expert_row_sum_entry(struct expert_row_sum_arguments arguments, unsigned char *arena)
{
    const uint32_t channel = (blockIdx.x * blockDim.x + threadIdx.x) * EXPERT_ROW_SUM_CHANNELS;
    if (channel >= arguments.width) {
        return;
    }
    const uint64_t row = blockIdx.y;
    const uint16_t *pairs = (const uint16_t *)(arena + arguments.pair_output_offset) + row * arguments.pairs_per_row * arguments.width + channel;
    float *out = (float *)(arena + arguments.row_output_offset) + row * arguments.width + channel;
    float sum[EXPERT_ROW_SUM_CHANNELS];
#pragma unroll
    for (uint32_t i = 0; i < EXPERT_ROW_SUM_CHANNELS; i++) {
        sum[i] = 0.0f;
    }
    if (arguments.width % EXPERT_ROW_SUM_CHANNELS == 0u) {
        for (uint32_t slot = 0; slot < arguments.pairs_per_row; slot++) {
            const uint4_t eight = *(const uint4_t *)(pairs + (uint64_t)slot * arguments.width);
            const uint32_t words[4] = {eight.x, eight.y, eight.z, eight.w};
#pragma unroll
            for (uint32_t i = 0; i < EXPERT_ROW_SUM_CHANNELS; i++) {
                sum[i] = __fadd_rn(sum[i], __uint_as_float(i % 2u == 0u ? words[i / 2u] << 16 : words[i / 2u] & 0xFFFF0000u));
            }
        }
        *(float4_t *)out = (float4_t){sum[0], sum[1], sum[2], sum[3]};
        *(float4_t *)(out + 4) = (float4_t){sum[4], sum[5], sum[6], sum[7]};
        return;
    }
    for (uint32_t i = 0; i < EXPERT_ROW_SUM_CHANNELS && channel + i < arguments.width; i++) { /* a width that is no multiple of 8 */
        float one = 0.0f;
        for (uint32_t slot = 0; slot < arguments.pairs_per_row; slot++) {
            one = __fadd_rn(one, bf16_to_float(pairs[(uint64_t)slot * arguments.width + i]));
        }
        out[i] = one;
    }
}
ANEMONE_KERNEL(KERNEL_FILE_EXPERT_LINEAR, expert_row_sum_entry, expert_row_sum_arguments);
