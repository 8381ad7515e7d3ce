/*
 * kernel_exl3_tcp.hip -- the routed experts of one EXL3 layer for a prefill-sized call on gfx950: the pairs sorted by
 * expert and the expert computation as a grouped GEMM on the matrix cores with the trellis decode fused into the
 * weight tile loads. The counterpart of the reference's prefill form (source/kernel_exl3_tcp.cuh:7-15,
 * include/anemone/exl3_tc_records.h:205-304): same record, same order of the work (route, operands, gate/up GEMM,
 * activation and down operands, down GEMM, combine in route order).
 *
 * Arithmetic: the chain's (kernel_exl3.hip): fp16 operands from a float32 Hadamard transform, exactly decoded fp16
 * weights, float32 MFMA sums over increasing k (one chain an output: the GEMM is not cut along k), SwiGLU in float32,
 * a row's weighted pair outputs added in slot order. A pair's result does not depend on the other pairs of the call.
 *
 * The GEMM block: 256 outputs (four wavefronts of four 16 x 16 tiles) by one chunk of at most EXL3_TCP_CHUNK_PAIRS (160)
 * pairs of one expert. A K step is 64 inputs: the chunk's operand columns (160 x 64 fp16, 20 KB) go from memory straight
 * into LDS once a block and serve all four wavefronts; each wavefront's codes go from memory into the registers of the
 * lanes that decode them, a decoded operand of eight weights a lane feeds up to five matrix instructions of 32 x 32
 * outputs, one for every 32 columns. Decoding is the vector unit's work (about 3.7 instructions a weight) and the
 * products the matrix unit's (32 cycles an instruction).
 */
#include "exl3_stream_device.cuh"
#include "kernel_registry.h"
#include "sort_device.cuh"

#define TCP_SORT_THREADS 512u
#define TCP_GEMM_WAVES 4u
#define TCP_GEMM_THREADS (TCP_GEMM_WAVES * WAVE)
#define TCP_WAVE_PAIRS 2u  /* pairs of adjacent output tiles of a wavefront: 64 outputs */
#define TCP_COLUMN_BLOCKS (EXL3_TCP_CHUNK_PAIRS / 16u) /* of sixteen columns: two a block of the matrix instruction's 32 */
#define TCP_STEP_INPUTS 64u
#define TCP_DIES 8u         /* the card's dies (XCDs), each with a level-2 cache of its own: blocks are dealt to them in turn */
#define TCP_BATCH 4u        /* columns the element-wise launches take at a time */
#define TCP_WAVE_BLOCKS 4u  /* blocks of 128 channels a wavefront of an element-wise launch takes: a row of sixteen lanes each */

struct tcp_shape {
    uint32_t hidden, intermediate, picks, pairs, experts;
    struct exl3_tcp_layout layout;
};

__device__ static __forceinline__ tcp_shape tcp_shape_of(const struct exl3_tcp_record &record)
{
    tcp_shape shape;
    shape.hidden = record.hidden;
    shape.intermediate = record.intermediate;
    shape.picks = record.pairs_per_row;
    shape.pairs = record.row_count * record.pairs_per_row;
    shape.experts = record.expert_count;
    shape.layout = exl3_tcp_layout_of(record.row_count, record.pairs_per_row, record.expert_count, record.hidden, record.intermediate);
    return shape;
}

__device__ static __forceinline__ uint32_t tcp_bits_x2(const struct exl3_tcp_record &record, const unsigned char *arena,
                                                       uint32_t expert, uint32_t matrix)
{
    if (record.widths_offset == 0u) {
        return record.bits_x2;
    }
    return exl3_bits_x2(exl3_width_of(((const uint32_t *)(arena + record.widths_offset))[expert], matrix));
}

__device__ static __forceinline__ uint64_t tcp_matrix_of(const struct exl3_tcp_record &record, const unsigned char *arena,
                                                         uint32_t expert, uint32_t matrix)
{
    return ((const uint64_t *)(arena + record.expert_offsets_offset))[(uint64_t)expert * MODEL_EXPERT_MATRICES + matrix];
}

/* launch 0: grid (ceil(row_count / ROUTER_SORT_ROWS)): counts [block][experts] */
extern "C" __global__ void __launch_bounds__(TCP_SORT_THREADS) exl3_tcp_count(struct exl3_tcp_record record, unsigned char *arena)
{
    __shared__ __attribute__((aligned(16))) uint32_t block_experts[ROUTER_SORT_ROWS * ROUTER_MOST_PICKS];
    const tcp_shape shape = tcp_shape_of(record);
    const uint32_t pairs = sort_block_picks((const struct router_pick *)(arena + record.picks_offset), shape.picks, blockIdx.x,
                                            record.row_count, block_experts);
    __syncthreads();
    __shared__ uint32_t histogram[ROUTER_MOST_EXPERTS];
    sort_count_picks(block_experts, pairs, shape.experts, histogram);
    uint32_t *counts = (uint32_t *)(arena + record.workspace_offset + shape.layout.counts) + (uint64_t)blockIdx.x * shape.experts;
    for (uint32_t expert = threadIdx.x; expert < shape.experts; expert += blockDim.x) {
        counts[expert] = histogram[expert];
    }
}
ANEMONE_KERNEL(EXL3_TCP_KERNEL_FILE, exl3_tcp_count, exl3_tcp_record);

/* launch 1: the same grid: the block's pairs placed (sorted [place] and place_of [pair]); block 0 also the runs, the
 * chunks and their number */
extern "C" __global__ void __launch_bounds__(TCP_SORT_THREADS) exl3_tcp_place(struct exl3_tcp_record record, unsigned char *arena)
{
    __shared__ __attribute__((aligned(16))) uint32_t block_experts[ROUTER_SORT_ROWS * ROUTER_MOST_PICKS];
    __shared__ uint32_t block_places[ROUTER_SORT_ROWS * ROUTER_MOST_PICKS];
    __shared__ uint32_t totals[ROUTER_MOST_EXPERTS], starts[ROUTER_MOST_EXPERTS], before[ROUTER_MOST_EXPERTS];
    __shared__ uint32_t chunk_starts[ROUTER_MOST_EXPERTS + 1u], scratch[ROUTER_MOST_EXPERTS];
    __shared__ uint32_t first_places[ROUTER_MOST_EXPERTS], cursors[SORT_MOST_WAVES * ROUTER_MOST_EXPERTS];
    const tcp_shape shape = tcp_shape_of(record);
    const uint32_t experts = shape.experts;
    const uint32_t blocks = (record.row_count + ROUTER_SORT_ROWS - 1u) / ROUTER_SORT_ROWS;
    unsigned char *workspace = arena + record.workspace_offset;
    const uint32_t pairs = sort_block_picks((const struct router_pick *)(arena + record.picks_offset), shape.picks, blockIdx.x,
                                            record.row_count, block_experts);
    const uint32_t *counts = (const uint32_t *)(workspace + shape.layout.counts);
    for (uint32_t expert = threadIdx.x; expert < experts; expert += blockDim.x) {
        uint32_t total = 0, lower = 0;
        for (uint32_t block = 0; block < blocks; block++) {
            const uint32_t count = counts[(uint64_t)block * experts + expert];
            total += count;
            lower += block < blockIdx.x ? count : 0u;
        }
        totals[expert] = total;
        starts[expert] = total;
        before[expert] = lower;
        chunk_starts[expert] = (total + EXL3_TCP_CHUNK_PAIRS - 1u) / EXL3_TCP_CHUNK_PAIRS;
    }
    __syncthreads();
    (void)block_exclusive_scan(starts, experts, scratch);
    uint32_t *sorted = (uint32_t *)(workspace + shape.layout.sorted), *place_of = (uint32_t *)(workspace + shape.layout.place_of);
    const uint32_t first_pair = blockIdx.x * ROUTER_SORT_ROWS * shape.picks;
    /* every pick's place into LDS; the two tables are written behind it, a thread a pick */
    for (uint32_t expert = threadIdx.x; expert < experts; expert += blockDim.x) {
        first_places[expert] = starts[expert] + before[expert];
    }
    __syncthreads();
    sort_place_picks(block_experts, pairs, experts, first_places, cursors, block_places);
    for (uint32_t index = threadIdx.x; index < pairs; index += blockDim.x) {
        const uint32_t place = block_places[index];
        sorted[place] = first_pair + index;
        place_of[first_pair + index] = place;
    }
    if (blockIdx.x != 0u) {
        return;
    }
    struct wide_run *runs = (struct wide_run *)(workspace + shape.layout.runs);
    for (uint32_t expert = threadIdx.x; expert < experts; expert += blockDim.x) {
        runs[expert] = (struct wide_run){starts[expert], totals[expert]};
    }
    const uint32_t used = block_exclusive_scan(chunk_starts, experts, scratch);
    if (threadIdx.x == 0u) {
        chunk_starts[experts] = used;
        uint32_t *header = (uint32_t *)(workspace + shape.layout.header);
        header[0] = used;
        header[1] = header[2] = header[3] = 0u;
    }
    __syncthreads();
    struct exl3_tcp_chunk *chunks = (struct exl3_tcp_chunk *)(workspace + shape.layout.chunks);
    for (uint32_t chunk = threadIdx.x; chunk < shape.layout.chunk_capacity; chunk += blockDim.x) {
        struct exl3_tcp_chunk value = {0, 0, 0, 0};
        if (chunk < used) {
            uint32_t low = 0, high = experts; /* the expert whose chunks hold this one */
            while (high - low > 1u) {
                const uint32_t middle = (low + high) / 2u;
                if (chunk_starts[middle] <= chunk) {
                    low = middle;
                } else {
                    high = middle;
                }
            }
            const uint32_t taken = (chunk - chunk_starts[low]) * EXL3_TCP_CHUNK_PAIRS, left = totals[low] - taken;
            value.expert = low;
            value.first_pair = starts[low] + taken;
            value.pair_count = left < EXL3_TCP_CHUNK_PAIRS ? left : EXL3_TCP_CHUNK_PAIRS;
        }
        chunks[chunk] = value;
    }
}
ANEMONE_KERNEL(EXL3_TCP_KERNEL_FILE, exl3_tcp_place, exl3_tcp_record);

__device__ static __forceinline__ struct exl3_tcp_chunk tcp_chunk_of(const tcp_shape &shape, const unsigned char *workspace, uint32_t index)
{
    const uint32_t used = ((const uint32_t *)(workspace + shape.layout.header))[0];
    struct exl3_tcp_chunk chunk = {0, 0, 0, 0};
    if (index < used) {
        chunk = ((const struct exl3_tcp_chunk *)(workspace + shape.layout.chunks))[index];
    }
    return chunk;
}

/* The element-wise launches take a block of 128 values in a row of sixteen lanes, eight consecutive values a lane
 * (one 16-byte load of bfloat16 or fp16, two of float32): a wavefront is four adjacent blocks of one vector, 1 KB of
 * bfloat16 a load. this lane's block of 128 channels and its first channel, or false past the width */
__device__ static __forceinline__ bool tcp_lane_channels(uint32_t width, uint32_t &channel)
{
    const uint32_t lane = threadIdx.x;
    channel = (blockIdx.x * TCP_WAVE_BLOCKS + lane / 16u) * EXL3_TRANSFORM + 8u * (lane % 16u);
    return channel < width;
}

/* launch 2: grid (ceil(hidden / 512), chunk capacity, EXL3_TCP_COLUMN_PARTS), block 64: the gate and the up operands of
 * a part of a chunk's pairs, by place: fp16(H128(x suh) / sqrt(128)); a row is read once for both */
extern "C" __global__ void exl3_tcp_operands(struct exl3_tcp_record record, unsigned char *arena)
{
    const tcp_shape shape = tcp_shape_of(record);
    unsigned char *workspace = arena + record.workspace_offset;
    const struct exl3_tcp_chunk chunk = tcp_chunk_of(shape, workspace, blockIdx.y);
    const uint32_t first_column = blockIdx.z * EXL3_TCP_PART_COLUMNS;
    uint32_t channel;
    if (first_column >= chunk.pair_count || !tcp_lane_channels(shape.hidden, channel)) {
        return;
    }
    const uint32_t lane = threadIdx.x;
    const uint32_t last_column = first_column + EXL3_TCP_PART_COLUMNS < chunk.pair_count ? first_column + EXL3_TCP_PART_COLUMNS : chunk.pair_count;
    float scale[2][8];
#pragma unroll
    for (uint32_t projection = 0; projection < 2u; projection++) {
        const uint64_t matrix = tcp_matrix_of(record, arena, chunk.expert, projection);
        const uint16_t *suh = (const uint16_t *)(arena + matrix + exl3_code_bytes(shape.hidden, shape.intermediate,
                                                                                   tcp_bits_x2(record, arena, chunk.expert, projection)));
        unpack_half8(*(const uint4_t *)(suh + channel), scale[projection]);
    }
    const uint16_t *rows = (const uint16_t *)(arena + record.hidden_offset);
    const uint32_t *sorted = (const uint32_t *)(workspace + shape.layout.sorted);
    uint16_t *operands = (uint16_t *)(workspace + shape.layout.operands);
    /* TCP_BATCH columns at a time: their loads are asked for together, so that one column's latency hides behind
     * the others' (a column past the part's last repeats it and is not stored) */
    for (uint32_t first = first_column; first < last_column; first += TCP_BATCH) {
        uint4_t loads[TCP_BATCH];
        uint32_t place[TCP_BATCH];
#pragma unroll
        for (uint32_t i = 0; i < TCP_BATCH; i++) {
            const uint32_t column = first + i < last_column ? first + i : last_column - 1u;
            place[i] = chunk.first_pair + column;
            const uint64_t row = sorted[place[i]] / shape.picks;
            loads[i] = *(const uint4_t *)(rows + row * shape.hidden + channel);
        }
#pragma unroll
        for (uint32_t i = 0; i < TCP_BATCH; i++) {
            float x[8];
            unpack_bf16x8(loads[i], x);
#pragma unroll
            for (uint32_t projection = 0; projection < 2u; projection++) {
                float v[8];
#pragma unroll
                for (uint32_t j = 0; j < 8u; j++) {
                    v[j] = __fmul_rn(x[j], scale[projection][j]);
                }
                row_hadamard128(v, lane);
#pragma unroll
                for (uint32_t j = 0; j < 8u; j++) {
                    v[j] = __fmul_rn(v[j], EXL3_NORMALIZATION);
                }
                if (first + i < last_column) {
                    *(uint4_t *)(operands + ((uint64_t)projection * shape.pairs + place[i]) * shape.hidden + channel) = pack_half8(v);
                }
            }
        }
    }
}
ANEMONE_KERNEL(EXL3_TCP_KERNEL_FILE, exl3_tcp_operands, exl3_tcp_record);

/*
 * The GEMM block: 256 outputs by one chunk of at most EXL3_TCP_CHUNK_PAIRS pairs of one expert, four wavefronts of 64
 * outputs each (two pairs of adjacent output tiles). A K step is 64 inputs (four K tiles).
 *
 * Weights: the codes go from memory straight into the registers of the lanes that decode them, by the stream product's
 * decode (exl3_stream_device.cuh) under the assignment of chunks to lanes that tcp_wave_gemm states; a decoded operand
 * of eight weights a lane (output half h, input half v) feeds one matrix instruction a block of 32 columns.
 * Operands: a stage holds the step's 64 inputs of every column of the chunk, 128 bytes a column, its eight 16-byte pieces
 * at the slots piece ^ ((column / 2) % 8) so that sixteen lanes of one read (sixteen columns, one piece) meet sixteen
 * different bank groups. Each wavefront brings a share of the stage by LDS DMA a step ahead, one barrier a step; the
 * reader of column block j takes piece 4 s + 2 (lane / 32) + v of column 32 j + lane % 32 as the instruction's B operand.
 */
/* 16 bytes a lane from memory straight into LDS (lane L lands at lds_base + 16 L), no register in between. Written as
 * assembly: the compiler keeps no book on it, so the wait that ends a step (every load of the wavefront, then the block's
 * barrier) is written out below. */
__device__ static __forceinline__ void tcp_load_to_lds(const void *lane_address, uint32_t lds_base)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(lane_address), "s"(lds_base) : "memory", "m0");
}

#define TCP_STAGE_COLUMN_BYTES (TCP_STEP_INPUTS * 2u)
#define TCP_STAGE_BYTES (EXL3_TCP_CHUNK_PAIRS * TCP_STAGE_COLUMN_BYTES)
#define TCP_STAGE_GROUPS (EXL3_TCP_CHUNK_PAIRS / 8u) /* groups of eight columns: one 16-byte-a-lane load of a wavefront each */
#define TCP_WAVE_GROUPS ((TCP_STAGE_GROUPS + TCP_GEMM_WAVES - 1u) / TCP_GEMM_WAVES)

/* A wavefront's product of 64 outputs by the chunk's columns on the matrix instruction of 32 x 32 outputs
 * (v_mfma_f32_32x32x16_f16: A lane l row l % 32, k = 8 (l / 32) + e; B lane l column l % 32, the same k; D lane l
 * column l % 32, register r row r % 4 + 8 (r / 4) + 4 (l / 32); measured on the card). Lane 16 g + i decodes chunk i % 8 of output tile i / 8 + 2 (g % 2) of the
 * wavefront's four and of K tile 2 s + g / 2 of the step's four (s = 0, 1: the step's halves), so the 32 rows of an
 * instruction (h, v) are output (i % 8) + 8 h of those four tiles and its sixteen k are inputs 8 v .. + 7 of the two K
 * tiles of half s: what a lane decodes, and how, is the stream product's; a decoded operand feeds LIVE instructions of
 * twice the work each. LIVE: blocks of 32 columns. */
typedef float float16v_t __attribute__((ext_vector_type(16)));

template <uint32_t bits_x2, uint32_t LIVE>
__device__ static __forceinline__ void
tcp_wave_gemm(const uint32_t *__restrict__ codes, uint32_t out_tiles, uint32_t strip_tile, uint32_t inputs,
                const half_t *__restrict__ columns, uint32_t column_count, uint32_t stages, uint32_t wave,
                uint32_t lane, bool strip_is_live, float16v_t (&accumulator)[2][LIVE])
{
    typedef exl3_chunk<bits_x2> C;
    constexpr uint32_t live_groups = 4u * LIVE; /* groups of eight columns that hold a pair */
    constexpr uint32_t wave_groups = (live_groups + TCP_GEMM_WAVES - 1u) / TCP_GEMM_WAVES;
    const uint32_t g = lane / 16u, i = lane % 16u, c = i % 8u, upper = lane / 32u, row = lane % 32u;
    const bool odd = (c & 1u) != 0u;
    uint32_t own, front;
    exl3_chunk_place<bits_x2>(c, own, front);
    const uint64_t step_stride = 4u * (uint64_t)out_tiles * C::tile_words, half_stride = 2u * (uint64_t)out_tiles * C::tile_words;
    /* a strip past the matrix reads the matrix's first strip (its sums are not stored): every wavefront runs the same loop */
    const uint32_t *tile = codes + ((uint64_t)(g / 2u) * out_tiles + (strip_is_live ? strip_tile : 0u) + i / 8u + 2u * (g % 2u)) * C::tile_words;
    /* the stage's groups this wavefront brings: wave, wave + 4, ...: lane L column 8 G + L / 8, slot L % 8 */
    const unsigned char *operand_source[wave_groups];
#pragma unroll
    for (uint32_t part = 0; part < wave_groups; part++) {
        const uint32_t group = wave + TCP_GEMM_WAVES * part, column = 8u * group + lane / 8u;
        const uint32_t piece = (lane % 8u) ^ ((column / 2u) % 8u);
        operand_source[part] = (const unsigned char *)(columns + (uint64_t)(column < column_count ? column : 0u) * inputs) + piece * 16u;
    }
    /* where this lane reads its B operand (half s, inputs v) of column block j: column 32 j + row, piece 4 s + 2 upper + v */
    uint32_t read_at[2][2];
#pragma unroll
    for (uint32_t s = 0; s < 2u; s++) {
#pragma unroll
        for (uint32_t v = 0; v < 2u; v++) {
            read_at[s][v] = row * TCP_STAGE_COLUMN_BYTES + (((4u * s + 2u * upper + v) ^ ((row / 2u) % 8u)) * 16u);
        }
    }
#pragma unroll
    for (uint32_t h = 0; h < 2u; h++) {
#pragma unroll
        for (uint32_t j = 0; j < LIVE; j++) {
#pragma unroll
            for (uint32_t r = 0; r < 16u; r++) {
                accumulator[h][j][r] = 0.0f;
            }
        }
    }
    const uint32_t steps = inputs / TCP_STEP_INPUTS;
    exl3_chunk_words<bits_x2> held[2][2];
#pragma unroll
    for (uint32_t s = 0; s < 2u; s++) {
        exl3_chunk_load<bits_x2>(tile + s * half_stride, own, front, held[0][s]);
    }
#pragma unroll
    for (uint32_t part = 0; part < wave_groups; part++) {
        if (wave + TCP_GEMM_WAVES * part < live_groups) {
            tcp_load_to_lds(operand_source[part], stages + (wave + TCP_GEMM_WAVES * part) * 1024u);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    auto one_step = [&](uint32_t step, exl3_chunk_words<bits_x2> (&now)[2], exl3_chunk_words<bits_x2> (&next)[2]) {
        const bool more = step + 1u < steps; /* the same in every lane */
        const uint32_t stage = stages + (step % 2u) * TCP_STAGE_BYTES, other = stages + ((step + 1u) % 2u) * TCP_STAGE_BYTES;
        if (more) {
            tile += step_stride;
#pragma unroll
            for (uint32_t s = 0; s < 2u; s++) {
                exl3_chunk_load<bits_x2>(tile + s * half_stride, own, front, next[s]);
            }
#pragma unroll
            for (uint32_t part = 0; part < wave_groups; part++) {
                if (wave + TCP_GEMM_WAVES * part < live_groups) {
                    tcp_load_to_lds(operand_source[part] + (uint64_t)(step + 1u) * TCP_STAGE_COLUMN_BYTES,
                                    other + (wave + TCP_GEMM_WAVES * part) * 1024u);
                }
            }
        }
#pragma unroll
        for (uint32_t s = 0; s < 2u; s++) {
            exl3_chunk_align<bits_x2>(now[s], odd);
        }
        /* Eight operands of eight weights a lane: k = 4 s + 2 v + h (the B operands of (s, v) serve both h and are read a
         * pair of operands ahead). An operand's LIVE matrix instructions are issued with the next operand's decoding
         * between them: the decoding runs in the products' shadow. */
        auto decode_weight = [&](uint32_t k, uint32_t w, uint32_t (&into)[4]) {
            const uint32_t s = k / 4u, v = k / 2u % 2u, h = k % 2u, t = w / 2u, m = 8u * t + 4u * h + 2u * v + w % 2u;
            uint32_t funnel[C::words];
#pragma unroll
            for (uint32_t word = 0; word < C::words; word++) {
                funnel[word] = __builtin_amdgcn_alignbit(now[s].z[word], now[s].z[word + 1u], 16u);
            }
            const uint32_t product = exl3_chunk_state<bits_x2>(now[s].z, funnel, m) * EXL3_MUL1_MULTIPLIER;
            if (w % 2u == 0u) {
                into[t] = __builtin_amdgcn_sad_u8(product, 0u, (uint32_t)EXL3_MUL1_BASE * 0x10001u);
            } else {
                const uint32_t sums = __builtin_amdgcn_sad_hi_u8(product, 0u, into[t]);
                const half2_t scale = __builtin_bit_cast(half2_t, (uint32_t)EXL3_MUL1_SCALE * 0x10001u);
                const half2_t bias = __builtin_bit_cast(half2_t, (uint32_t)EXL3_MUL1_BIAS * 0x10001u);
                into[t] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(half2_t, sums), scale, bias));
            }
        };
        half8_t operand_b[2][LIVE];
        uint32_t a[4], ahead[4];
        auto read_operands = [&](uint32_t k) { /* those of operands k and k + 1 */
#pragma unroll
            for (uint32_t j = 0; j < LIVE; j++) {
                operand_b[k / 2u % 2u][j] = __builtin_bit_cast(half8_t, *(const __attribute__((address_space(3))) uint4_t *)(uintptr_t)(stage + j * (32u * TCP_STAGE_COLUMN_BYTES) + read_at[k / 4u][k / 2u % 2u]));
            }
        };
        read_operands(0u); /* on their way while the first operand is decoded */
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (uint32_t w = 0; w < 8u; w++) {
            decode_weight(0u, w, a);
        }
#pragma unroll
        for (uint32_t k = 0; k < 8u; k++) {
            const uint32_t h = k % 2u;
            if (k % 2u == 0u && k + 2u < 8u) {
                read_operands(k + 2u);
            }
            const uint4_t packed = {a[0], a[1], a[2], a[3]};
            const half8_t weights = __builtin_bit_cast(half8_t, packed);
#pragma unroll
            for (uint32_t j = 0; j < LIVE; j++) {
                accumulator[h][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(weights, operand_b[k / 2u % 2u][j], accumulator[h][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (k + 1u < 8u) {
#pragma unroll
                    for (uint32_t w = 0; w < 8u; w++) {
                        if (w * LIVE / 8u == j) {
                            decode_weight(k + 1u, w, ahead);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (uint32_t t = 0; t < 4u; t++) {
                a[t] = ahead[t];
            }
        }
        /* every load of this wavefront has landed (the next step's stage among them), this step's stage is read */
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __syncthreads();
    };
    for (uint32_t step = 0; step < steps; step += 2u) {
        one_step(step, held[0], held[1]);
        if (step + 1u < steps) {
            one_step(step + 1u, held[1], held[0]);
        }
    }
}

/* launches 3 and 5: grid (ceil(outputs / 256), chunk capacity, projections), block 256.
 * pass EXL3_TCP_GATE_AND_UP: z = 0 gate, 1 up, products [z][place][intermediate]; pass EXL3_TCP_DOWN: down,
 * products [place][hidden]. */
extern "C" __global__ void __launch_bounds__(TCP_GEMM_THREADS, 2) exl3_tcp_gemm(struct exl3_tcp_record record, unsigned char *arena)
{
    __shared__ __attribute__((aligned(16))) unsigned char stages[2u * TCP_STAGE_BYTES];
    const tcp_shape shape = tcp_shape_of(record);
    unsigned char *workspace = arena + record.workspace_offset;
    /* Which (strip of 256 outputs, chunk, projection) this block takes. The card deals blocks to its eight dies in turn by
     * their number x + gx (y + gy z), so die c holds the blocks whose x % 8 is c. Every output strip of a chunk reads the
     * chunk's operand columns: the blocks of eight consecutive rows m = y + gy z of the grid are re-assigned so that those
     * a die holds among them are all the strips of one (chunk, projection), which then come from memory into that die's
     * level-2 cache once (a grid whose x is no multiple of eight, and the rows past the last whole eight, stay as dealt). */
    uint32_t strip = blockIdx.x, place = blockIdx.y + gridDim.y * blockIdx.z;
    const uint32_t places = gridDim.y * gridDim.z;
    if (gridDim.x % TCP_DIES == 0u && place < places / TCP_DIES * TCP_DIES) {
        strip = (place % TCP_DIES) * (gridDim.x / TCP_DIES) + blockIdx.x / TCP_DIES;
        place = place / TCP_DIES * TCP_DIES + blockIdx.x % TCP_DIES;
    }
    const struct exl3_tcp_chunk chunk = tcp_chunk_of(shape, workspace, place % gridDim.y);
    if (chunk.pair_count == 0u) {
        return;
    }
    const uint32_t lane = threadIdx.x % WAVE, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const bool down = record.pass == EXL3_TCP_DOWN;
    const uint32_t projection = down ? 2u : place / gridDim.y;
    const uint32_t inputs = down ? shape.intermediate : shape.hidden, outputs = down ? shape.hidden : shape.intermediate;
    const uint32_t bits_x2 = tcp_bits_x2(record, arena, chunk.expert, projection);
    const uint32_t *codes = (const uint32_t *)(arena + tcp_matrix_of(record, arena, chunk.expert, projection));
    const half_t *columns = (const half_t *)(workspace + shape.layout.operands) +
                            ((uint64_t)(down ? 0u : projection) * shape.pairs + chunk.first_pair) * inputs;
    float *products = down ? (float *)(workspace + shape.layout.down) + (uint64_t)chunk.first_pair * outputs
                           : (float *)(workspace + shape.layout.gate_up) + ((uint64_t)projection * shape.pairs + chunk.first_pair) * outputs;
    const uint32_t strip_tile = (strip * EXL3_TCP_BLOCK_OUTPUTS) / EXL3_TILE + wave * 2u * TCP_WAVE_PAIRS;
    const bool strip_is_live = strip_tile * EXL3_TILE < outputs;
    const uint32_t stage_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)stages;
    const uint32_t live_blocks = (chunk.pair_count + 15u) / 16u;
    /* one instance a width and a count of live blocks of 32 columns (1 to 5): the pairs' columns and nothing past them */
#define TCP_GEMM_OF(bits, live)                                                                                                   \
    do {                                                                                                                          \
        float16v_t accumulator[2][live];                                                                                          \
        tcp_wave_gemm<bits, live>(codes, outputs / EXL3_TILE, strip_tile, inputs, columns, chunk.pair_count, stage_base, wave, lane, \
                                    strip_is_live, accumulator);                                                                  \
        if (strip_is_live) {                                                                                                      \
            _Pragma("unroll") for (uint32_t j = 0; j < live; j++)                                                                 \
            {                                                                                                                     \
                const uint32_t column = 32u * j + lane % 32u;                                                                     \
                if (column < chunk.pair_count) {                                                                                  \
                    float *out = products + (uint64_t)column * outputs;                                                           \
                    _Pragma("unroll") for (uint32_t h = 0; h < 2u; h++)                                                           \
                    {                                                                                                             \
                        _Pragma("unroll") for (uint32_t q = 0; q < 4u; q++)                                                       \
                        {                                                                                                         \
                            const uint32_t first_row = 8u * q + 4u * (lane / 32u);                                                \
                            const uint32_t output = EXL3_TILE * (strip_tile + first_row % 16u / 8u + 2u * (first_row / 16u)) +    \
                                                    first_row % 8u + 8u * h;                                                      \
                            *(float4_t *)(out + output) = (float4_t){accumulator[h][j][4u * q], accumulator[h][j][4u * q + 1u],   \
                                                                     accumulator[h][j][4u * q + 2u], accumulator[h][j][4u * q + 3u]}; \
                        }                                                                                                         \
                    }                                                                                                             \
                }                                                                                                                 \
            }                                                                                                                     \
        }                                                                                                                         \
    } while (0)
#define TCP_GEMM_WIDTH(bits)                    \
    if (live_blocks <= 2u) {                    \
        TCP_GEMM_OF(bits, 1u);                  \
    } else if (live_blocks <= 4u) {             \
        TCP_GEMM_OF(bits, 2u);                  \
    } else if (live_blocks <= 6u) {             \
        TCP_GEMM_OF(bits, 3u);                  \
    } else if (live_blocks <= 8u) {             \
        TCP_GEMM_OF(bits, 4u);                  \
    } else {                                    \
        TCP_GEMM_OF(bits, TCP_COLUMN_BLOCKS / 2u); \
    }
    switch (bits_x2) {
    case 4u: TCP_GEMM_WIDTH(4u) break;
    case 5u: TCP_GEMM_WIDTH(5u) break;
    case 6u: TCP_GEMM_WIDTH(6u) break;
    case 8u: TCP_GEMM_WIDTH(8u) break;
    default: return; /* no width of the format: the prepare refuses such a record */
    }
#undef TCP_GEMM_WIDTH
#undef TCP_GEMM_OF
}
ANEMONE_KERNEL(EXL3_TCP_KERNEL_FILE, exl3_tcp_gemm, exl3_tcp_record);

/* launch 4: grid (ceil(intermediate / 512), chunk capacity, EXL3_TCP_COLUMN_PARTS), block 64: per pair of a part of the chunk, gate = H128(gate products) /
 * sqrt(128) x svh, up the same, the SwiGLU with its limit, x the down matrix's suh, H128 -> the fp16 down operand */
extern "C" __global__ void exl3_tcp_activate(struct exl3_tcp_record record, unsigned char *arena)
{
    const tcp_shape shape = tcp_shape_of(record);
    unsigned char *workspace = arena + record.workspace_offset;
    const struct exl3_tcp_chunk chunk = tcp_chunk_of(shape, workspace, blockIdx.y);
    const uint32_t first_column = blockIdx.z * EXL3_TCP_PART_COLUMNS;
    uint32_t channel;
    if (first_column >= chunk.pair_count || !tcp_lane_channels(shape.intermediate, channel)) {
        return;
    }
    const uint32_t lane = threadIdx.x;
    const uint32_t last_column = first_column + EXL3_TCP_PART_COLUMNS < chunk.pair_count ? first_column + EXL3_TCP_PART_COLUMNS : chunk.pair_count;
    const uint32_t H = shape.hidden, I = shape.intermediate, e = chunk.expert;
    const uint16_t *gate_svh = (const uint16_t *)(arena + tcp_matrix_of(record, arena, e, 0u) + exl3_code_bytes(H, I, tcp_bits_x2(record, arena, e, 0u))) + H;
    const uint16_t *up_svh = (const uint16_t *)(arena + tcp_matrix_of(record, arena, e, 1u) + exl3_code_bytes(H, I, tcp_bits_x2(record, arena, e, 1u))) + H;
    const uint16_t *down_suh = (const uint16_t *)(arena + tcp_matrix_of(record, arena, e, 2u) + exl3_code_bytes(I, H, tcp_bits_x2(record, arena, e, 2u)));
    float gs[8], us[8], ds[8];
    unpack_half8(*(const uint4_t *)(gate_svh + channel), gs);
    unpack_half8(*(const uint4_t *)(up_svh + channel), us);
    unpack_half8(*(const uint4_t *)(down_suh + channel), ds);
    const float limit = record.activation_limit;
    const float *gate_products = (const float *)(workspace + shape.layout.gate_up);
    const float *up_products = gate_products + (uint64_t)shape.pairs * I;
    uint16_t *operands = (uint16_t *)(workspace + shape.layout.operands);
    constexpr uint32_t BATCH = 2u; /* two columns' eight loads together */
    for (uint32_t first = first_column; first < last_column; first += BATCH) {
        float4_t loads[BATCH][4];
        uint64_t place[BATCH];
#pragma unroll
        for (uint32_t i = 0; i < BATCH; i++) {
            const uint32_t column = first + i < last_column ? first + i : last_column - 1u;
            place[i] = chunk.first_pair + column;
            const float4_t *gate = (const float4_t *)(gate_products + place[i] * I + channel), *up = (const float4_t *)(up_products + place[i] * I + channel);
            loads[i][0] = gate[0];
            loads[i][1] = gate[1];
            loads[i][2] = up[0];
            loads[i][3] = up[1];
        }
#pragma unroll
        for (uint32_t i = 0; i < BATCH; i++) {
            float g[8], u[8], v[8];
#pragma unroll
            for (uint32_t j = 0; j < 8u; j++) {
                g[j] = loads[i][j / 4u][j % 4u];
                u[j] = loads[i][2u + j / 4u][j % 4u];
            }
            row_hadamard128(g, lane);
            row_hadamard128(u, lane);
#pragma unroll
            for (uint32_t j = 0; j < 8u; j++) {
                const float gate = __fmul_rn(__fmul_rn(g[j], EXL3_NORMALIZATION), gs[j]);
                const float up = __fmul_rn(__fmul_rn(u[j], EXL3_NORMALIZATION), us[j]);
                const float bounded_gate = limit > 0.0f ? fminf(gate, limit) : gate;
                const float bounded_up = limit > 0.0f ? fminf(fmaxf(up, -limit), limit) : up;
                const float hidden = __fmul_rn(det_silu(bounded_gate), bounded_up);
                v[j] = __fmul_rn(hidden, ds[j]);
            }
            row_hadamard128(v, lane);
#pragma unroll
            for (uint32_t j = 0; j < 8u; j++) {
                v[j] = __fmul_rn(v[j], EXL3_NORMALIZATION);
            }
            if (first + i < last_column) {
                *(uint4_t *)(operands + place[i] * I + channel) = pack_half8(v);
            }
        }
    }
}
ANEMONE_KERNEL(EXL3_TCP_KERNEL_FILE, exl3_tcp_activate, exl3_tcp_record);

/* launch 6: grid (ceil(hidden / 512), row_count), block 64: a row's pairs in slot order */
extern "C" __global__ void exl3_tcp_combine(struct exl3_tcp_record record, unsigned char *arena)
{
    const tcp_shape shape = tcp_shape_of(record);
    const unsigned char *workspace = arena + record.workspace_offset;
    uint32_t channel;
    if (!tcp_lane_channels(shape.hidden, channel)) {
        return;
    }
    const uint32_t lane = threadIdx.x, row = blockIdx.y;
    const uint32_t H = shape.hidden, I = shape.intermediate;
    const struct router_pick *picks = (const struct router_pick *)(arena + record.picks_offset) + (uint64_t)row * shape.picks;
    const uint32_t *place_of = (const uint32_t *)(workspace + shape.layout.place_of);
    const float *down = (const float *)(workspace + shape.layout.down);
    float sum[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t slot = 0; slot < shape.picks; slot++) {
        const struct router_pick pick = picks[slot];
        const uint64_t place = place_of[row * shape.picks + slot];
        const uint16_t *svh = (const uint16_t *)(arena + tcp_matrix_of(record, arena, pick.expert, 2u) +
                                                 exl3_code_bytes(I, H, tcp_bits_x2(record, arena, pick.expert, 2u))) + I;
        const float4_t *products = (const float4_t *)(down + place * H + channel);
        const float4_t low = products[0], high = products[1];
        float v[8] = {low[0], low[1], low[2], low[3], high[0], high[1], high[2], high[3]}, scale[8];
        unpack_half8(*(const uint4_t *)(svh + channel), scale);
        row_hadamard128(v, lane);
#pragma unroll
        for (uint32_t j = 0; j < 8u; j++) {
            sum[j] = __fadd_rn(sum[j], __fmul_rn(__fmul_rn(__fmul_rn(v[j], EXL3_NORMALIZATION), scale[j]), pick.route_weight));
        }
    }
    float4_t *out = (float4_t *)((float *)(arena + record.output_offset) + (uint64_t)row * H + channel);
    out[0] = (float4_t){sum[0], sum[1], sum[2], sum[3]};
    out[1] = (float4_t){sum[4], sum[5], sum[6], sum[7]};
}
ANEMONE_KERNEL(EXL3_TCP_KERNEL_FILE, exl3_tcp_combine, exl3_tcp_record);
