/*
 * kernel_router.hip -- the router of one MoE layer on gfx950: score projection, affinity, top-k choice with route
 * weights, and the job table the routed experts read. Entry names and records follow the reference
 * (source/kernel_router.cu, source/kernel_router.cuh, include/anemone/router_records.h); the expert count, the
 * picks a row, the route scale and the affinity are run-time members of the record (a zero means the reference's
 * 384 / 6 / 1.5 / sqrt(softplus)).
 *
 * What a row's choice is (include/anemone/router_records.h:8-31): affinity a of every expert; the P experts of the
 * largest a + bias compared as the reference's top-k compares float32 (a not-a-number above every number, -0 below
 * +0, the lower expert first among equals); slots in ascending expert order; weights a / (t + 1e-20) * scale, each
 * operation one float32 rounding, t the sum of the P affinities from +0 in ascending expert order (or the
 * reference's tree order for six picks). The job table: a job for each chosen expert, ascending; a column for each
 * row that chose it, rows ascending; unused columns and empty jobs zero. No atomic operation; a row's choice
 * depends on that row alone.
 *
 * exp and log1p are fixed sequences of float32 operations (the same the CPU oracle runs), so that affinities, and
 * with them the expert ids, are the same bits on the card and on the host.
 */
#include "router_device.cuh"
#include "kernel_registry.h"
#include "sort_device.cuh"

#define PROJECTION_CHAINS 32u
#define PROJECTION_THREADS 128u

/* scores[row][expert] = sum_k w[expert][k] x[row][k]: 32 fma chains, chain c owning the inputs k = c mod 32 in
 * ascending order, then a halving fold 16, 8, 4, 2, 1 (source/kernel_official_router_projection.cu:33-57).
 * A block takes PROJECTION_EXPERTS experts and up to PROJECTION_ROWS rows: it stages the weights and the rows in
 * chunks of PROJECTION_CHUNK inputs through LDS with 16-byte coalesced loads (the next chunk in flight while this
 * one is consumed); a thread owns chains 2 j and 2 j + 1 of one expert for every row, so the fma order of a chain
 * is the definition's whatever the staging. grid (ceil(E / 8), ceil(rows / 4)), block 128; or, for a thin step, grid
 * (ceil(E / 8), rows): a row a block (the rows a block takes are what its grid leaves it, four or one), a quarter of
 * the fused multiply-adds a block and four times the blocks: the launch is a few round trips to memory either way. */
#define PROJECTION_MOST_ROWS 4u
#define PROJECTION_EXPERTS 8u
#define PROJECTION_CHUNK 1024u
#define PROJECTION_W_LOADS (PROJECTION_EXPERTS * PROJECTION_CHUNK * 2u / 16u / PROJECTION_THREADS)
template <uint32_t PROJECTION_ROWS>
__device__ static __forceinline__ void router_projection_block(const struct router_projection_arguments &arguments, unsigned char *arena)
{
    constexpr uint32_t PROJECTION_X_LOADS = PROJECTION_ROWS * PROJECTION_CHUNK * 2u / 16u / PROJECTION_THREADS;
    __shared__ __attribute__((aligned(16))) uint16_t w_tile[PROJECTION_EXPERTS][PROJECTION_CHUNK];
    __shared__ __attribute__((aligned(16))) uint16_t x_tile[PROJECTION_ROWS][PROJECTION_CHUNK];
    const uint32_t H = arguments.hidden, thread = threadIdx.x;
    const uint32_t first_expert = blockIdx.x * PROJECTION_EXPERTS, first_row = blockIdx.y * PROJECTION_ROWS;
    const uint16_t *weights = (const uint16_t *)(arena + arguments.weights_offset);
    const uint16_t *rows = (const uint16_t *)(arena + arguments.rows_offset);
    uint4_t w_next[PROJECTION_W_LOADS], x_next[PROJECTION_X_LOADS];
    /* piece p of a tile: 8 values of line p / (CHUNK / 8) at column 8 (p % (CHUNK / 8)); out of range reads zero */
    auto fetch = [&](uint32_t chunk) {
#pragma unroll
        for (uint32_t i = 0; i < PROJECTION_W_LOADS; i++) {
            const uint32_t piece = i * PROJECTION_THREADS + thread, line = piece / (PROJECTION_CHUNK / 8u);
            const uint32_t k = chunk + 8u * (piece % (PROJECTION_CHUNK / 8u)), expert = first_expert + line;
            w_next[i] = (uint4_t){0, 0, 0, 0};
            if (expert < arguments.expert_count && k < H) {
                w_next[i] = *(const uint4_t *)(weights + (uint64_t)expert * H + k);
            }
        }
#pragma unroll
        for (uint32_t i = 0; i < PROJECTION_X_LOADS; i++) {
            const uint32_t piece = i * PROJECTION_THREADS + thread, line = piece / (PROJECTION_CHUNK / 8u);
            const uint32_t k = chunk + 8u * (piece % (PROJECTION_CHUNK / 8u)), row = first_row + line;
            x_next[i] = (uint4_t){0, 0, 0, 0};
            if (row < arguments.row_count && k < H) {
                x_next[i] = *(const uint4_t *)(rows + (uint64_t)row * H + k);
            }
        }
    };
    const uint32_t expert_in_block = thread / 16u, pair = thread % 16u; /* chains 2 pair, 2 pair + 1 */
    float chain[PROJECTION_ROWS][2];
#pragma unroll
    for (uint32_t r = 0; r < PROJECTION_ROWS; r++) {
        chain[r][0] = chain[r][1] = 0.0f;
    }
    fetch(0u);
    for (uint32_t chunk = 0; chunk < H; chunk += PROJECTION_CHUNK) {
        __syncthreads(); /* the tile's readers of the chunk before are done */
#pragma unroll
        for (uint32_t i = 0; i < PROJECTION_W_LOADS; i++) {
            ((uint4_t *)&w_tile[0][0])[i * PROJECTION_THREADS + thread] = w_next[i];
        }
#pragma unroll
        for (uint32_t i = 0; i < PROJECTION_X_LOADS; i++) {
            ((uint4_t *)&x_tile[0][0])[i * PROJECTION_THREADS + thread] = x_next[i];
        }
        if (chunk + PROJECTION_CHUNK < H) {
            fetch(chunk + PROJECTION_CHUNK);
        }
        __syncthreads();
#pragma unroll 4
        for (uint32_t k = 0; k < PROJECTION_CHUNK; k += PROJECTION_CHAINS) {
            const uint32_t w = *(const uint32_t *)&w_tile[expert_in_block][k + 2u * pair];
            const float w0 = __uint_as_float(w << 16), w1 = __uint_as_float(w & 0xFFFF0000u);
#pragma unroll
            for (uint32_t r = 0; r < PROJECTION_ROWS; r++) {
                const uint32_t x = *(const uint32_t *)&x_tile[r][k + 2u * pair];
                chain[r][0] = __fmaf_rn(w0, __uint_as_float(x << 16), chain[r][0]);
                chain[r][1] = __fmaf_rn(w1, __uint_as_float(x & 0xFFFF0000u), chain[r][1]);
            }
        }
    }
    const uint32_t expert = first_expert + expert_in_block;
#pragma unroll
    for (uint32_t r = 0; r < PROJECTION_ROWS; r++) {
        float even = __fadd_rn(0.0f, chain[r][0]), odd = __fadd_rn(0.0f, chain[r][1]);
        /* chain c + distance lies distance / 2 threads on, for the distances 16, 8, 4, 2 */
#pragma unroll
        for (uint32_t distance = 8u; distance != 0u; distance >>= 1u) {
            even = __fadd_rn(even, __shfl_down(even, distance, 16));
            odd = __fadd_rn(odd, __shfl_down(odd, distance, 16));
        }
        const float sum = __fadd_rn(even, odd); /* distance 1: chain 0 + chain 1 */
        if (pair == 0u && expert < arguments.expert_count && first_row + r < arguments.row_count) {
            ((float *)(arena + arguments.output_offset))[(uint64_t)(first_row + r) * arguments.expert_count + expert] = __fadd_rn(0.0f, sum);
        }
    }
}

extern "C" __global__ void __launch_bounds__(PROJECTION_THREADS)
    router_projection(struct router_projection_arguments arguments, unsigned char *arena)
{
    if (gridDim.y >= arguments.row_count) { /* the same in every block: a row a block */
        router_projection_block<1u>(arguments, arena);
    } else {
        router_projection_block<PROJECTION_MOST_ROWS>(arguments, arena);
    }
}
ANEMONE_KERNEL(KERNEL_FILE_ROUTER, router_projection, router_projection_arguments);

/* The same scores on the matrix unit, for steps of many rows. v_mfma_f32_16x16x1_4b_f32 adds, to each of four 16 x 16
 * blocks of sums, one product a sum, each a fused multiply-add of float32 rounded once (compared bit for bit with
 * fmaf over wide exponent ranges, subnormal products and infinities): a block is a chain, its 16 x 16 sums the chains
 * of 16 experts by 16 rows, and the eight instructions of a group of 32 inputs advance the 32 chains by one input
 * each, in the definition's order. Instruction q takes the chains 8 b + q of the blocks b = 0 .. 3, so that lane
 * (b, n) needs the inputs 32 i + 8 b + {0 .. 7} of expert n (and of row n): one 16-byte piece each a group. The fold is
 * inside a lane. grid (E / 16, ceil(rows / 64)), block 256: a wavefront 16 rows.
 *
 * The pieces pass through LDS. Read by the lanes that use them they would be 64 bytes of each of sixteen rows an
 * instruction, rows a power of two apart: half-used lines that fall into the same few sets of the first-level cache, and
 * the wavefronts waited for them three quarters of their time. Instead a stage of PROJECTION_STAGE_INPUTS inputs of the
 * block's 16 experts and 64 rows (80 rows of 256 bytes) is brought by 20 loads of a wavefront that go from memory
 * straight into LDS, each 256 contiguous bytes of four rows; piece p of tile row R lies at slot p ^ (R % 16) of its row,
 * so that the eight lanes of a 16-byte read (eight rows, one piece) meet eight different bank groups. Two stages (40 KB:
 * three blocks a CU, which measured faster than three stages and two blocks): the next stage is asked for behind the
 * barrier that ends the stage before the current one. */
typedef __attribute__((ext_vector_type(16))) float float16_t;
#define PROJECTION_STAGE_ROW_BYTES (PROJECTION_STAGE_INPUTS * 2u)
#define PROJECTION_STAGE_ROWS (16u + PROJECTION_TILE_ROWS)
#define PROJECTION_STAGE_BYTES (PROJECTION_STAGE_ROWS * PROJECTION_STAGE_ROW_BYTES)
#define PROJECTION_STAGES 2u
#define PROJECTION_WAVE_LOADS (PROJECTION_STAGE_BYTES / 1024u / (PROJECTION_TILE_THREADS / WAVE)) /* 5 */

/* a group of 32 inputs: eight instructions, each one input further on the four chains it takes */
__device__ static __forceinline__ void projection_tile_group(const uint4_t &w_now, const uint4_t &x_now, float16_t (&chain)[8])
{
    const uint32_t w_words[4] = {w_now.x, w_now.y, w_now.z, w_now.w}, x_words[4] = {x_now.x, x_now.y, x_now.z, x_now.w};
#pragma unroll
    for (uint32_t q = 0; q < 8u; q++) {
        const float a = __uint_as_float(q % 2u == 0u ? w_words[q / 2u] << 16 : w_words[q / 2u] & 0xFFFF0000u);
        const float b = __uint_as_float(q % 2u == 0u ? x_words[q / 2u] << 16 : x_words[q / 2u] & 0xFFFF0000u);
        chain[q] = __builtin_amdgcn_mfma_f32_16x16x1f32(a, b, chain[q], 0, 0, 0);
    }
}

/* 16 bytes a lane from memory straight into LDS (lane L lands at lds_base + 16 L). Written as assembly: the compiler keeps
 * no book on it, so the waits for it are written out where a stage is needed. */
__device__ static __forceinline__ void projection_load_to_lds(const void *lane_address, uint32_t lds_base)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(lane_address), "s"(lds_base) : "memory", "m0");
}

extern "C" __global__ void __launch_bounds__(PROJECTION_TILE_THREADS, 3) /* three blocks a CU */
    router_projection_tiles(struct router_projection_arguments arguments, unsigned char *arena)
{
    __shared__ __attribute__((aligned(1024))) unsigned char window[PROJECTION_STAGES * PROJECTION_STAGE_BYTES];
    const uint32_t lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), block = lane / 16u, index = lane % 16u;
    const uint32_t H = arguments.hidden, groups = H / PROJECTION_CHAINS;
    const uint32_t stages = groups / 4u; /* whole stages: whoever prepares the launch holds the width to a multiple of PROJECTION_STAGE_INPUTS */
    const uint32_t first_expert = blockIdx.x * 16u, block_row = blockIdx.y * PROJECTION_TILE_ROWS, first_row = block_row + wave * 16u;
    const uint32_t window_address = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)window;
    /* what this wavefront brings of a stage: the loads wave, wave + 4, ...; load d is the tile rows 4 d .. 4 d + 3 (the
     * experts' rows first, then the block's rows; a row past the last repeats the last: its sums are not stored) */
    const unsigned char *source[PROJECTION_WAVE_LOADS];
    uint32_t piece_bytes[PROJECTION_WAVE_LOADS];
#pragma unroll
    for (uint32_t part = 0; part < PROJECTION_WAVE_LOADS; part++) {
        const uint32_t tile_row = 4u * (wave + 4u * part) + lane / 16u;
        piece_bytes[part] = 16u * ((lane % 16u) ^ (tile_row % 16u));
        if (tile_row < 16u) {
            source[part] = arena + arguments.weights_offset + (uint64_t)(first_expert + tile_row) * H * 2u;
        } else {
            const uint32_t row = block_row + tile_row - 16u;
            source[part] = arena + arguments.rows_offset + (uint64_t)(row < arguments.row_count ? row : arguments.row_count - 1u) * H * 2u;
        }
    }
    auto ask = [&](uint32_t stage) {
        const uint32_t base = window_address + (stage % PROJECTION_STAGES) * PROJECTION_STAGE_BYTES;
#pragma unroll
        for (uint32_t part = 0; part < PROJECTION_WAVE_LOADS; part++) {
            projection_load_to_lds(source[part] + stage * PROJECTION_STAGE_ROW_BYTES + piece_bytes[part], base + (wave + 4u * part) * 1024u);
        }
    };
    /* where lane (b, n) reads its pieces of group i of a stage: piece 4 i + b of expert n and of the wavefront's row n */
    uint32_t w_at[4], x_at[4];
#pragma unroll
    for (uint32_t i = 0; i < 4u; i++) {
        const uint32_t slot = 16u * ((4u * i + block) ^ index);
        w_at[i] = index * PROJECTION_STAGE_ROW_BYTES + slot;
        x_at[i] = (16u + 16u * wave + index) * PROJECTION_STAGE_ROW_BYTES + slot;
    }
    float16_t chain[8];
#pragma unroll
    for (uint32_t q = 0; q < 8u; q++) {
#pragma unroll
        for (uint32_t v = 0; v < 16u; v++) {
            chain[q][v] = 0.0f;
        }
    }
    ask(0u);
    for (uint32_t stage = 0; stage < stages; stage++) {
        /* this wavefront's loads of the stage have landed, then every wavefront's; behind the barrier every wavefront is
         * through the stage before, whose window the next stage takes */
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (stage + 1u < stages) {
            ask(stage + 1u);
        }
        const unsigned char *now = window + (stage % PROJECTION_STAGES) * PROJECTION_STAGE_BYTES;
        uint4_t w_now = *(const uint4_t *)(now + w_at[0]), x_now = *(const uint4_t *)(now + x_at[0]);
#pragma unroll
        for (uint32_t i = 0; i < 4u; i++) {
            const uint4_t w_use = w_now, x_use = x_now;
            if (i + 1u < 4u) { /* the next group's pieces are on their way behind this group's instructions */
                w_now = *(const uint4_t *)(now + w_at[i + 1u]);
                x_now = *(const uint4_t *)(now + x_at[i + 1u]);
                __builtin_amdgcn_sched_barrier(0); /* asked for here, not behind the group's instructions */
            }
            projection_tile_group(w_use, x_use, chain);
        }
    }
    /* register v = 4 b + r of chain[q] is chain 8 b + q of expert 4 (lane / 16) + r and row lane % 16. The fold, as the
     * definition orders it: + 0 first, then the distances 16 and 8 (blocks), 4, 2 and 1 (instructions) */
    float sums[8][8];
#pragma unroll
    for (uint32_t q = 0; q < 8u; q++) {
#pragma unroll
        for (uint32_t v = 0; v < 8u; v++) {
            sums[q][v] = __fadd_rn(__fadd_rn(0.0f, chain[q][v]), __fadd_rn(0.0f, chain[q][v + 8u]));
        }
#pragma unroll
        for (uint32_t r = 0; r < 4u; r++) {
            sums[q][r] = __fadd_rn(sums[q][r], sums[q][r + 4u]);
        }
    }
#pragma unroll
    for (uint32_t distance = 4u; distance != 0u; distance >>= 1u) {
#pragma unroll
        for (uint32_t q = 0; q < distance; q++) {
#pragma unroll
            for (uint32_t r = 0; r < 4u; r++) {
                sums[q][r] = __fadd_rn(sums[q][r], sums[q + distance][r]);
            }
        }
    }
    if (first_row + index < arguments.row_count) {
        float *out = (float *)(arena + arguments.output_offset) + (uint64_t)(first_row + index) * arguments.expert_count + first_expert + 4u * block;
        *(float4_t *)out = (float4_t){__fadd_rn(0.0f, sums[0][0]), __fadd_rn(0.0f, sums[0][1]), __fadd_rn(0.0f, sums[0][2]), __fadd_rn(0.0f, sums[0][3])};
    }
}
ANEMONE_KERNEL(KERNEL_FILE_ROUTER, router_projection_tiles, router_projection_arguments);

extern "C" __global__ void __launch_bounds__(SELECT_THREADS)
    router_select_entry(struct router_select_arguments arguments, unsigned char *arena)
{
    __shared__ struct router_select_lds lds;
    router_select_body(arguments, arena, threadIdx.x, blockDim.x, lds);
}
ANEMONE_KERNEL(KERNEL_FILE_ROUTER, router_select_entry, router_select_arguments);

/* ---- the wide select: rows of a prefill, sorted by expert ------------------------------------------------------
 * Four launches of one record, in this order (include/anemone/router_records.h:31-47 of the reference; the kernels
 * at source/kernel_router.cu:97-459 there): the picks of every live row; the pairs of each expert counted in blocks
 * of ROUTER_SORT_ROWS rows; every pair placed (a pair's place: the pairs of lower experts, and of its expert in
 * lower rows), the runs and the tiles of at most 64 pairs; the job table of at most 8 pairs a job. No atomic
 * operation: a thread owns an expert and walks the block's picks in row order. */
#define WIDE_SORT_THREADS 512u

__device__ static __forceinline__ uint32_t wide_live_rows(const struct router_wide_arguments &arguments, const unsigned char *arena)
{
    const uint32_t step_rows = ((const struct step_block *)(arena + arguments.step_offset))->row_count;
    return step_rows < arguments.row_count ? step_rows : arguments.row_count;
}

/* grid (ceil(row_count / 8)), a wavefront a row: its affinities, as the select writes them, and its picks by slot */
extern "C" __global__ void __launch_bounds__(SELECT_THREADS)
    router_wide_select(struct router_wide_arguments arguments, unsigned char *arena)
{
    __shared__ float affinities[LINEAR_MAXIMUM_ROWS * ROUTER_MOST_EXPERTS];
    const uint32_t experts = arguments.expert_count, picks = arguments.pick_count, places = experts / WAVE;
    const uint32_t wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const uint32_t row = blockIdx.x * LINEAR_MAXIMUM_ROWS + wave;
    /* asked for together: the step's rows, the lane's bias values and scores (the row is inside the scores' array or the
     * wavefront reads row 0's) */
    const uint32_t live_rows = wide_live_rows(arguments, arena);
    const uint64_t first = (uint64_t)(row < arguments.row_count ? row : 0u) * experts;
    float bias_of[ROUTER_PLACES], scores[ROUTER_PLACES];
#pragma unroll
    for (uint32_t place = 0; place < ROUTER_PLACES; place++) {
        bias_of[place] = place < places ? ((const float *)(arena + arguments.bias_offset))[lane + place * WAVE] : 0.0f;
        scores[place] = place < places ? ((const float *)(arena + arguments.scores_offset))[first + lane + place * WAVE] : 0.0f;
    }
    if (row >= live_rows) {
        return; /* no barrier in this kernel: a wavefront is a row */
    }
    struct router_pick my_pick;
    uint32_t my_slot;
    router_row_any(scores, bias_of, experts, affinities + wave * experts, (float *)(arena + arguments.affinities_offset) + first, lane,
                   arguments.affinity_kind, picks, arguments.reference_order, arguments.route_scale, my_pick.expert, my_slot, my_pick.route_weight);
    if (lane < picks) { /* lane p holds pick p */
        ((struct router_pick *)(arena + arguments.picks_offset))[(uint64_t)row * picks + my_slot] = my_pick;
    }
}
ANEMONE_KERNEL(KERNEL_FILE_ROUTER, router_wide_select, router_wide_arguments);

/* the picked experts of the live rows of block `block` of ROUTER_SORT_ROWS rows, into LDS; returns their number */
__device__ static __forceinline__ uint32_t wide_block_picks(const struct router_wide_arguments &arguments, const unsigned char *arena,
                                                            uint32_t block, uint32_t live_rows, uint32_t *experts_out)
{
    return sort_block_picks((const struct router_pick *)(arena + arguments.picks_offset), arguments.pick_count, block, live_rows, experts_out);
}

/* grid (ceil(row_count / ROUTER_SORT_ROWS)): counts [block][E] */
extern "C" __global__ void __launch_bounds__(WIDE_SORT_THREADS)
    router_wide_count(struct router_wide_arguments arguments, unsigned char *arena)
{
    __shared__ __attribute__((aligned(16))) uint32_t block_experts[ROUTER_SORT_ROWS * ROUTER_MOST_PICKS];
    const uint32_t live_rows = wide_live_rows(arguments, arena);
    const uint32_t pairs = wide_block_picks(arguments, arena, blockIdx.x, live_rows, block_experts);
    __syncthreads();
    if (pairs == 0u) {
        return; /* a block of no live row writes nothing; the place reads no count of it */
    }
    __shared__ uint32_t histogram[ROUTER_MOST_EXPERTS];
    sort_count_picks(block_experts, pairs, arguments.expert_count, histogram);
    uint32_t *counts = (uint32_t *)(arena + arguments.counts_offset) + (uint64_t)blockIdx.x * arguments.expert_count;
    for (uint32_t expert = threadIdx.x; expert < arguments.expert_count; expert += blockDim.x) {
        counts[expert] = histogram[expert];
    }
}
ANEMONE_KERNEL(KERNEL_FILE_ROUTER, router_wide_count, router_wide_arguments);

/* What a block of the place does once it holds, in LDS, its picks (block_experts, `pairs` of them) and of every expert
 * the pairs of all blocks (totals; starts a copy of them), those of the blocks before this one (before) and its
 * tiles (tile_starts): the sorted pairs of the block's rows; block 0 also the runs and every tile. The whole block
 * calls it after a barrier. */
__device__ static __forceinline__ void wide_place_block(const struct router_wide_arguments &arguments, unsigned char *arena, uint32_t block,
                                                        const uint32_t *block_experts, uint32_t *place_of, uint32_t pairs, uint32_t *totals,
                                                        uint32_t *starts, const uint32_t *before, uint32_t *tile_starts, uint32_t *scratch,
                                                        uint32_t *first_places, uint32_t *cursors)
{
    const uint32_t experts = arguments.expert_count, picks = arguments.pick_count;
    (void)block_exclusive_scan(starts, experts, scratch);
    const struct router_pick *all_picks = (const struct router_pick *)(arena + arguments.picks_offset);
    struct wide_pair *sorted = (struct wide_pair *)(arena + arguments.pairs_offset);
    const uint32_t first_pair = block * ROUTER_SORT_ROWS * picks;
    /* every pick's place into LDS; the pairs are written behind it, a thread a pick */
    for (uint32_t expert = threadIdx.x; expert < experts; expert += blockDim.x) {
        first_places[expert] = starts[expert] + before[expert];
    }
    __syncthreads();
    sort_place_picks(block_experts, pairs, experts, first_places, cursors, place_of);
    for (uint32_t index = threadIdx.x; index < pairs; index += blockDim.x) {
        sorted[place_of[index]] = (struct wide_pair){first_pair + index, all_picks[first_pair + index].route_weight};
    }
    if (block != 0u) {
        return;
    }
    struct wide_run *runs = (struct wide_run *)(arena + arguments.runs_offset);
    for (uint32_t expert = threadIdx.x; expert < experts; expert += blockDim.x) {
        runs[expert] = (struct wide_run){starts[expert], totals[expert]};
    }
    const uint32_t used_tiles = block_exclusive_scan(tile_starts, experts, scratch);
    if (threadIdx.x == 0u) {
        tile_starts[experts] = used_tiles;
    }
    __syncthreads();
    const uint32_t all_tiles = ROUTER_WIDE_TILES_OF(arguments.row_count, picks, experts);
    struct wide_expert_tile *tiles = (struct wide_expert_tile *)(arena + arguments.tiles_offset);
    const uint64_t *offsets = (const uint64_t *)(arena + arguments.expert_offsets_offset);
    for (uint32_t tile = threadIdx.x; tile < all_tiles; tile += blockDim.x) {
        struct wide_expert_tile value = {0, 0, 0, 0, 0};
        if (tile < used_tiles) {
            uint32_t low = 0, high = experts; /* the expert whose tiles hold this one: tile_starts[e] <= tile < [e + 1] */
            while (high - low > 1u) {
                const uint32_t middle = (low + high) / 2u;
                if (tile_starts[middle] <= tile) {
                    low = middle;
                } else {
                    high = middle;
                }
            }
            const uint32_t taken = (tile - tile_starts[low]) * WIDE_TILE_PAIRS, left = totals[low] - taken;
            value.gate_offset = offsets[(uint64_t)low * MODEL_EXPERT_MATRICES + 0u];
            value.up_offset = offsets[(uint64_t)low * MODEL_EXPERT_MATRICES + 1u];
            value.down_offset = offsets[(uint64_t)low * MODEL_EXPERT_MATRICES + 2u];
            value.first_pair = starts[low] + taken;
            value.pair_count = left < WIDE_TILE_PAIRS ? left : WIDE_TILE_PAIRS;
        }
        tiles[tile] = value;
    }
}

/* grid as the count's: the sorted pairs of the block's rows; block 0 also the runs and every tile */
extern "C" __global__ void __launch_bounds__(WIDE_SORT_THREADS)
    router_wide_place(struct router_wide_arguments arguments, unsigned char *arena)
{
    __shared__ __attribute__((aligned(16))) uint32_t block_experts[ROUTER_SORT_ROWS * ROUTER_MOST_PICKS];
    __shared__ uint32_t place_of[ROUTER_SORT_ROWS * ROUTER_MOST_PICKS];
    __shared__ uint32_t totals[ROUTER_MOST_EXPERTS], starts[ROUTER_MOST_EXPERTS], before[ROUTER_MOST_EXPERTS];
    __shared__ uint32_t tile_starts[ROUTER_MOST_EXPERTS + 1u], scratch[ROUTER_MOST_EXPERTS];
    __shared__ uint32_t first_places[ROUTER_MOST_EXPERTS], cursors[SORT_MOST_WAVES * ROUTER_MOST_EXPERTS];
    const uint32_t experts = arguments.expert_count;
    const uint32_t live_rows = wide_live_rows(arguments, arena);
    const uint32_t live_blocks = (live_rows + ROUTER_SORT_ROWS - 1u) / ROUTER_SORT_ROWS;
    const uint32_t pairs = wide_block_picks(arguments, arena, blockIdx.x, live_rows, block_experts);
    if (pairs == 0u && blockIdx.x != 0u) {
        return;
    }
    const uint32_t *counts = (const uint32_t *)(arena + arguments.counts_offset);
    for (uint32_t expert = threadIdx.x; expert < experts; expert += blockDim.x) {
        uint32_t total = 0, lower = 0;
        for (uint32_t block = 0; block < live_blocks; block++) {
            const uint32_t count = counts[(uint64_t)block * experts + expert];
            total += count;
            lower += block < blockIdx.x ? count : 0u;
        }
        totals[expert] = total;
        starts[expert] = total;
        before[expert] = lower;
        tile_starts[expert] = (total + WIDE_TILE_PAIRS - 1u) / WIDE_TILE_PAIRS;
    }
    __syncthreads();
    wide_place_block(arguments, arena, blockIdx.x, block_experts, place_of, pairs, totals, starts, before, tile_starts, scratch, first_places,
                     cursors);
}
ANEMONE_KERNEL(KERNEL_FILE_ROUTER, router_wide_place, router_wide_arguments);

/* The job table of the runs, a thread a job; job_starts holds every expert's jobs. The whole block calls it after a
 * barrier that follows the writing of the runs and the sorted pairs. */
__device__ static __forceinline__ void wide_jobs_block(const struct router_wide_arguments &arguments, unsigned char *arena,
                                                       uint32_t *job_starts, uint32_t *scratch)
{
    const uint32_t experts = arguments.expert_count, picks = arguments.pick_count;
    const struct wide_run *runs = (const struct wide_run *)(arena + arguments.runs_offset);
    const uint32_t used_jobs = block_exclusive_scan(job_starts, experts, scratch);
    if (threadIdx.x == 0u) {
        job_starts[experts] = used_jobs;
    }
    __syncthreads();
    const uint32_t all_jobs = ROUTER_WIDE_JOBS_OF(arguments.row_count, picks, experts);
    const struct wide_pair *sorted = (const struct wide_pair *)(arena + arguments.pairs_offset);
    const uint64_t *offsets = (const uint64_t *)(arena + arguments.expert_offsets_offset);
    struct expert_job_record *jobs = (struct expert_job_record *)(arena + arguments.jobs_offset);
    for (uint32_t job = threadIdx.x; job < all_jobs; job += blockDim.x) {
        struct expert_job_record value;
        uint32_t *words = (uint32_t *)&value;
#pragma unroll
        for (uint32_t word = 0; word < JOB_WORDS; word++) {
            words[word] = 0u;
        }
        if (job < used_jobs) {
            uint32_t low = 0, high = experts;
            while (high - low > 1u) {
                const uint32_t middle = (low + high) / 2u;
                if (job_starts[middle] <= job) {
                    low = middle;
                } else {
                    high = middle;
                }
            }
            const struct wide_run run = runs[low];
            const uint32_t taken = (job - job_starts[low]) * LINEAR_MAXIMUM_ROWS, left = run.pair_count - taken;
            value.gate_offset = offsets[(uint64_t)low * MODEL_EXPERT_MATRICES + 0u];
            value.up_offset = offsets[(uint64_t)low * MODEL_EXPERT_MATRICES + 1u];
            value.down_offset = offsets[(uint64_t)low * MODEL_EXPERT_MATRICES + 2u];
            value.row_count = left < LINEAR_MAXIMUM_ROWS ? left : LINEAR_MAXIMUM_ROWS;
            value.expert = low;
            for (uint32_t column = 0; column < value.row_count; column++) {
                const struct wide_pair pair = sorted[run.first_pair + taken + column];
                value.pair_index[column] = pair.pair_index;
                value.route_weight[column] = pair.route_weight;
            }
        }
        jobs[job] = value;
    }
}

/* grid (1): the job table of the runs, a thread a job */
extern "C" __global__ void __launch_bounds__(WIDE_SORT_THREADS)
    router_wide_jobs(struct router_wide_arguments arguments, unsigned char *arena)
{
    __shared__ uint32_t job_starts[ROUTER_MOST_EXPERTS + 1u], scratch[ROUTER_MOST_EXPERTS];
    const struct wide_run *runs = (const struct wide_run *)(arena + arguments.runs_offset);
    for (uint32_t expert = threadIdx.x; expert < arguments.expert_count; expert += blockDim.x) {
        job_starts[expert] = (runs[expert].pair_count + LINEAR_MAXIMUM_ROWS - 1u) / LINEAR_MAXIMUM_ROWS;
    }
    __syncthreads();
    wide_jobs_block(arguments, arena, job_starts, scratch);
}
ANEMONE_KERNEL(KERNEL_FILE_ROUTER, router_wide_jobs, router_wide_arguments);

/* grid (1): the count, the place and the jobs of at most ROUTER_SORT_ROWS rows in one block (the reference's
 * router_wide_small, source/kernel_router.cu there): the same pairs, runs, tiles and jobs; the counts scratch is
 * not written */
extern "C" __global__ void __launch_bounds__(WIDE_SORT_THREADS)
    router_wide_small(struct router_wide_arguments arguments, unsigned char *arena)
{
    __shared__ __attribute__((aligned(16))) uint32_t block_experts[ROUTER_SORT_ROWS * ROUTER_MOST_PICKS];
    __shared__ uint32_t place_of[ROUTER_SORT_ROWS * ROUTER_MOST_PICKS];
    __shared__ uint32_t totals[ROUTER_MOST_EXPERTS], starts[ROUTER_MOST_EXPERTS], before[ROUTER_MOST_EXPERTS];
    __shared__ uint32_t tile_starts[ROUTER_MOST_EXPERTS + 1u], scratch[ROUTER_MOST_EXPERTS], job_starts[ROUTER_MOST_EXPERTS + 1u];
    __shared__ uint32_t first_places[ROUTER_MOST_EXPERTS], cursors[SORT_MOST_WAVES * ROUTER_MOST_EXPERTS];
    const uint32_t experts = arguments.expert_count;
    const uint32_t live_rows = wide_live_rows(arguments, arena);
    const uint32_t pairs = wide_block_picks(arguments, arena, 0u, live_rows, block_experts);
    __syncthreads();
    sort_count_picks(block_experts, pairs, experts, totals);
    for (uint32_t expert = threadIdx.x; expert < experts; expert += blockDim.x) {
        const uint32_t count = totals[expert];
        starts[expert] = count;
        before[expert] = 0u;
        tile_starts[expert] = (count + WIDE_TILE_PAIRS - 1u) / WIDE_TILE_PAIRS;
        job_starts[expert] = (count + LINEAR_MAXIMUM_ROWS - 1u) / LINEAR_MAXIMUM_ROWS;
    }
    __syncthreads();
    wide_place_block(arguments, arena, 0u, block_experts, place_of, pairs, totals, starts, before, tile_starts, scratch, first_places, cursors);
    __threadfence_block();
    __syncthreads(); /* the runs and the sorted pairs, written by this block, are read by its jobs */
    wide_jobs_block(arguments, arena, job_starts, scratch);
}
ANEMONE_KERNEL(KERNEL_FILE_ROUTER, router_wide_small, router_wide_arguments);
