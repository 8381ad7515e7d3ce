/*
 * anemone_records.h -- the by-value records of every kernel of the routed-expert path, and the arrays they name.
 * Compiles as C11 (the host's prepare functions) and as HIP C++ (the kernels).
 *
 * The kernel ABI is the reference's (include/anemone/backend_seam.h:60-69): every kernel is
 *     extern "C" __global__ void <name>(struct <record> record, unsigned char *arena)
 * and a record names memory by BYTE OFFSETS into the card's one arena, never by address. Records are fixed-size,
 * little-endian, without padding, at most LAUNCH_ARGUMENT_BYTES (192).
 *
 * Layout compatibility. Each struct below keeps the reference's members in the reference's order, so a caller that
 * fills a record by member name fills the same leading bytes:
 *     expert_job_record                 include/anemone/linear_records.h:245-253       (96 B)
 *     router_pick, wide_pair/run/tile   include/anemone/router_records.h:112-115, wide_linear_records.h:62-78
 *     step_block                        include/anemone/step_records.h:111-115         (16 B)
 *     exl3_reconstruct_record           include/anemone/exl3_records.h:123-130         (32 B)
 *     expert_row_sum_arguments          include/anemone/linear_records.h:300-305       (24 B)
 *     activation_quantize_arguments     include/anemone/linear_records.h:222-229       (40 B)
 *     expert_gate_up_arguments          include/anemone/linear_records.h:263-275       (64 B)
 *     expert_down_arguments             include/anemone/linear_records.h:283-293       (56 B)
 * Four records carry a TRAILING EXTENSION the reference does not have, because the reference fixes one model's
 * shape at compile time (384 experts, 6 picks, hidden 5120, one width per layer) and this build takes them at run
 * time. A zero extension means "the reference's behaviour":
 *     router_select_arguments  80 B  (router_records.h:98-110)   + expert_count, pick_count, affinity_kind, route_scale
 *     router_wide_arguments    120 B (router_records.h:117-134)  + the same four
 *     exl3_expert_record       80 B  (exl3_records.h:144-159)    + widths_offset
 *     exl3_tc_record           72 B  (exl3_tc_records.h:40-58)   + widths_offset, hidden, pairs_per_row, expert_count
 *     exl3_tcp_record          88 B  (exl3_tc_records.h:244-262) + widths_offset, hidden, pairs_per_row, expert_count
 * widths_offset: 0, or the arena offset of uint32 [expert_count], entry e = gate | up << 8 | down << 16, the stored
 * widths of expert e's three matrices (per-matrix widths: one layer mixes K = 2, 3, 4). When it is 0 every matrix
 * has the record's one width, as in the reference.
 */
#ifndef ANEMONE_RECORDS_H
#define ANEMONE_RECORDS_H

#include <stdint.h>

#ifdef __cplusplus
#define ANEMONE_RECORD_HAS(record, bytes) static_assert(sizeof(struct record) == (bytes), #record " ABI")
#else
#define ANEMONE_RECORD_HAS(record, bytes) _Static_assert(sizeof(struct record) == (bytes), #record " ABI")
#endif

/* ---- shared geometry ---- */
#define LINEAR_MAXIMUM_ROWS 8u          /* columns of one job; rows of one thin trunk launch, a group of a wide one */
#define LINEAR_OUTPUTS_PER_TILE 16u
#define LINEAR_VALUES_PER_BLOCK 32u     /* values that share one scale exponent */
#define LINEAR_VALUES_PER_LOAD 64u
#define LINEAR_OFFSET_ALIGNMENT_BYTES 16u
#define LINEAR_ELEMENT_THREADS 256u
#define WIDE_TILE_PAIRS 64u
#define MODEL_EXPERT_MATRICES 3u        /* gate, up, down */
#define ROUTER_DEFAULT_EXPERTS 384u     /* what a zero extension stands for */
#define ROUTER_DEFAULT_PICKS 6u
#define ROUTER_DEFAULT_SCALE 1.5f
#define ROUTER_MOST_EXPERTS 512u
#define ROUTER_MOST_PICKS 8u
#define ROUTER_AFFINITY_SQRT_SOFTPLUS 0u
#define ROUTER_AFFINITY_SIGMOID 1u

/* ---- step ---- */
struct step_block {
    uint64_t sequence;
    uint32_t row_count; /* the live rows of the step: the routers read it, not their record's */
    uint32_t flags;
};
ANEMONE_RECORD_HAS(step_block, 16);

/* ---- job table and the wide select's arrays ---- */
struct expert_job_record {
    uint64_t gate_offset;
    uint64_t up_offset;
    uint64_t down_offset;
    uint32_t row_count; /* 0 .. 8; an empty job is read no further */
    uint32_t expert;
    uint32_t pair_index[LINEAR_MAXIMUM_ROWS]; /* row * pairs_per_row + slot */
    float route_weight[LINEAR_MAXIMUM_ROWS];
};
ANEMONE_RECORD_HAS(expert_job_record, 96);

struct router_pick {
    uint32_t expert;
    float route_weight;
};
struct wide_pair {
    uint32_t pair_index;
    float route_weight;
};
struct wide_run {
    uint32_t first_pair;
    uint32_t pair_count;
};
struct wide_expert_tile {
    uint64_t gate_offset;
    uint64_t up_offset;
    uint64_t down_offset;
    uint32_t first_pair;
    uint32_t pair_count; /* at most WIDE_TILE_PAIRS */
};
ANEMONE_RECORD_HAS(router_pick, 8);
ANEMONE_RECORD_HAS(wide_pair, 8);
ANEMONE_RECORD_HAS(wide_run, 8);
ANEMONE_RECORD_HAS(wide_expert_tile, 32);

/* ---- router ---- */
#define KERNEL_FILE_ROUTER "kernel_router"
#define KERNEL_ROUTER_PROJECTION "router_projection"
#define KERNEL_ROUTER_PROJECTION_TILES "router_projection_tiles" /* the same scores on the matrix unit: steps of many rows */
#define PROJECTION_TILE_THREADS 256u
#define PROJECTION_TILE_ROWS 64u   /* rows of a block of router_projection_tiles: 16 a wavefront */
#define PROJECTION_TILE_LEAST_ROWS 257u /* fewer rows take router_projection: its blocks are smaller and more */
#define PROJECTION_STAGE_INPUTS 128u     /* inputs of a stage of router_projection_tiles: the width is a whole number of them */
#define KERNEL_ROUTER_SELECT "router_select_entry"
#define KERNEL_ROUTER_WIDE_SELECT "router_wide_select"
#define KERNEL_ROUTER_WIDE_COUNT "router_wide_count"
#define KERNEL_ROUTER_WIDE_PLACE "router_wide_place"
#define KERNEL_ROUTER_WIDE_JOBS "router_wide_jobs"
#define KERNEL_ROUTER_WIDE_SMALL "router_wide_small"
#define ROUTER_THREADS 256u
#define ROUTER_SORT_ROWS 384u
#define ROUTER_WIDE_MOST_ROWS 65536u /* rows of one wide select */

struct router_projection_arguments { /* scores [rows][experts] = W x, bfloat16 in, float32 out */
    uint64_t weights_offset;         /* read: bfloat16 [expert_count][hidden] */
    uint64_t rows_offset;            /* read: bfloat16 [row_count][hidden] */
    uint64_t output_offset;          /* written: float32 [row_count][expert_count] */
    uint32_t row_count;
    uint32_t hidden;
    uint32_t expert_count;
    uint32_t reserved_zero;
};
ANEMONE_RECORD_HAS(router_projection_arguments, 40);

struct router_select_arguments {
    uint64_t step_offset;            /* read: struct step_block */
    uint64_t scores_offset;          /* read: float32 [row_count][E] */
    uint64_t bias_offset;            /* read: float32 [E] */
    uint64_t expert_offsets_offset;  /* read: uint64 [E][3] */
    uint64_t affinities_offset;      /* written: float32 [row_count][E], live rows */
    uint64_t jobs_offset;            /* written: struct expert_job_record [P row_count], every byte */
    uint64_t weights_offset;         /* the experts' range: its first byte, */
    uint64_t gate_up_last_offset;    /* the last a gate or up matrix may begin at, */
    uint64_t down_last_offset;       /* the last a down matrix may begin at */
    uint32_t row_count;              /* 1 .. LINEAR_MAXIMUM_ROWS */
    uint32_t reference_order;        /* 0 or 1 (1: six picks alone) */
    /* extension */
    uint32_t expert_count;           /* 0: 384 */
    uint32_t pick_count;             /* 0: 6 */
    uint32_t affinity_kind;          /* ROUTER_AFFINITY_* */
    float route_scale;               /* 0: 1.5 */
};
ANEMONE_RECORD_HAS(router_select_arguments, 96);

struct router_wide_arguments {
    uint64_t step_offset;
    uint64_t scores_offset;
    uint64_t bias_offset;
    uint64_t expert_offsets_offset;
    uint64_t affinities_offset;      /* written: float32 [row_count][E] */
    uint64_t picks_offset;           /* scratch: struct router_pick [row_count][P] */
    uint64_t counts_offset;          /* scratch: uint32 [ceil(row_count / ROUTER_SORT_ROWS)][E] */
    uint64_t pairs_offset;           /* written: struct wide_pair [P row_count] */
    uint64_t runs_offset;            /* written: struct wide_run [E] */
    uint64_t tiles_offset;           /* written: struct wide_expert_tile [tiles of row_count] */
    uint64_t jobs_offset;            /* written: struct expert_job_record [jobs of row_count] */
    uint64_t weights_offset;
    uint64_t gate_up_last_offset;
    uint64_t down_last_offset;
    uint32_t row_count;
    uint32_t reference_order;
    /* extension */
    uint32_t expert_count;
    uint32_t pick_count;
    uint32_t affinity_kind;
    float route_scale;
};
ANEMONE_RECORD_HAS(router_wide_arguments, 136);

/* tiles / jobs of a wide select: each run cut in 64s (8s), the last ragged */
#define ROUTER_WIDE_TILES_OF(row_count, picks, experts) \
    (((row_count) * (picks) + WIDE_TILE_PAIRS - 1u) / WIDE_TILE_PAIRS + (experts))
#define ROUTER_WIDE_JOB_BOUND_OF(row_count, picks, experts) \
    (((row_count) * (picks) + (LINEAR_MAXIMUM_ROWS - 1u) * (experts)) / LINEAR_MAXIMUM_ROWS)
#define ROUTER_WIDE_JOBS_OF(row_count, picks, experts)                                             \
    ((row_count) * (picks) < ROUTER_WIDE_JOB_BOUND_OF(row_count, picks, experts) ? (row_count) * (picks) \
                                                                                  : ROUTER_WIDE_JOB_BOUND_OF(row_count, picks, experts))

/* ---- EXL3 ---- */
#define EXL3_KERNEL_FILE "kernel_exl3"
#define EXL3_RECONSTRUCT "exl3_reconstruct"
#define EXL3_ROW_SUM "exl3_row_sum"
#define EXL3_TILE 16u
#define EXL3_TILE_VALUES 256u
#define EXL3_TRANSFORM 128u
#define EXL3_K2 2u   /* stored widths: K for a whole K, 16 K for a half K */
#define EXL3_K2_5 40u
#define EXL3_K3 3u
#define EXL3_K4 4u
#define EXL3_MUL1_MULTIPLIER 0x83DCD12Du
#define EXL3_MUL1_BASE 0x6400u
#define EXL3_MUL1_SCALE 0x1EEEu
#define EXL3_MUL1_BIAS 0xC931u
#define EXL3_NORMALIZATION 0.08838834764831845f
#define EXL3_EXPERT_LAUNCHES 5u
#define EXL3_PRODUCT_SLICES 4u
#define EXL3_STRIP_TILES 8u      /* output tiles of a block of the chain's product launches: 128 outputs */
#define EXL3_THIN_STRIP_TILES 1u /* of the _thin instances, which a launch of fewer than EXL3_THIN_BELOW_BLOCKS blocks takes */
#define EXL3_THIN_BELOW_BLOCKS 256u

#ifdef __cplusplus
#define ANEMONE_INLINE __host__ __device__ static constexpr inline
#else
#define ANEMONE_INLINE static inline
#endif

/* bits_x2 = 2 K of a stored width; 0 for a value that is no width (whole 1-8, half 1.5-7.5) */
ANEMONE_INLINE uint32_t exl3_bits_x2(uint32_t stored_width)
{
    return stored_width >= 1u && stored_width <= 8u ? 2u * stored_width
           : stored_width % 16u == 8u && stored_width < 128u ? stored_width / 8u
                                                             : 0u;
}
/* the widths this build has kernels for */
ANEMONE_INLINE int exl3_width_supported(uint32_t stored_width)
{
    return stored_width == EXL3_K2 || stored_width == EXL3_K3 || stored_width == EXL3_K4 || stored_width == EXL3_K2_5;
}
/* S(i): ring bit where the window of position i ends */
ANEMONE_INLINE uint32_t exl3_window_end(uint32_t position, uint32_t bits_x2)
{
    return (position + 1u) * bits_x2 / 2u;
}
ANEMONE_INLINE uint64_t exl3_code_bytes(uint64_t inputs, uint64_t outputs, uint32_t bits_x2)
{
    return inputs * outputs / 16u * bits_x2;
}
/* an expert's packed widths entry -> the stored width of matrix m (0 gate, 1 up, 2 down) */
ANEMONE_INLINE uint32_t exl3_width_of(uint32_t packed, uint32_t matrix)
{
    return (packed >> (8u * matrix)) & 255u;
}

struct exl3_reconstruct_record {
    uint64_t matrix_offset;
    uint64_t output_offset; /* written: fp16 [input][output], before either transform or scale */
    uint32_t input_size;
    uint32_t output_size;
    uint32_t bits_per_weight; /* stored width */
    uint32_t reserved_zero;
};
ANEMONE_RECORD_HAS(exl3_reconstruct_record, 32);

/* The five-launch chain of one layer: input, gate/up products, activate, down products, finish (then exl3_row_sum).
 * operands fp16 [2][pairs][input_size]; products float32 [2][pairs][inner_size], later [pairs][input_size];
 * hidden bf16 [pairs][inner_size]; output float32 [pairs][input_size] == products (in place). */
struct exl3_expert_record {
    uint64_t jobs_offset;
    uint64_t input_offset;    /* read: bf16 [rows][input_size] */
    uint64_t operands_offset;
    uint64_t products_offset;
    uint64_t hidden_offset;
    uint64_t output_offset;   /* == products_offset */
    uint32_t input_size;
    uint32_t inner_size;
    uint32_t pair_count;
    uint32_t pairs_per_row;
    uint32_t job_count;
    uint32_t bits_per_weight; /* the one stored width, unless widths_offset names per-matrix widths */
    float activation_limit;
    uint32_t reserved_zero;
    /* extension */
    uint64_t widths_offset;
};
ANEMONE_RECORD_HAS(exl3_expert_record, 88);

#define EXPERT_ROW_SUM_CHANNELS 8u /* consecutive outputs a thread of expert_row_sum_entry sums */
struct expert_row_sum_arguments {
    uint64_t pair_output_offset;
    uint64_t row_output_offset;
    uint32_t width;
    uint32_t pairs_per_row;
};
ANEMONE_RECORD_HAS(expert_row_sum_arguments, 24);

/* ---- EXL3 fused decode (at most EXL3_TC_MOST_ROWS rows) ---- */
#define EXL3_TC_KERNEL_FILE "kernel_exl3_tc"
#define EXL3_TC_LAUNCHES 5u
#define EXL3_TC_MOST_ROWS 64u
#define EXL3_TC_DEFAULT_HIDDEN 5120u
#define EXL3_TC_DEFAULT_PAIRS_PER_ROW 6u
#define EXL3_TC_GATE_UP_SLICES 4u /* K slices of a gate/up product: partial sums kept apart, added in order */
#define EXL3_TC_DOWN_SLICES 4u
#define EXL3_TC_STRIP_OUTPUTS 64u /* outputs of one wavefront item of the products launches */

struct exl3_tc_record {
    uint64_t jobs_offset;      /* read: struct expert_job_record [job_capacity], empty ones anywhere */
    uint64_t hidden_offset;    /* read: bf16 [row_count][hidden] */
    uint64_t workspace_offset; /* scratch: exl3_tc_workspace_bytes(...), 256-aligned */
    uint64_t output_offset;    /* written: float32 [row_count][hidden], each row's route-weighted expert sum */
    uint32_t row_count;
    uint32_t job_capacity;
    uint32_t intermediate;
    uint32_t bits_x2;          /* the one width as 2 K, unless widths_offset names per-matrix widths */
    float activation_limit;    /* the SwiGLU limit; 0: none */
    uint32_t pass;             /* the products launches: 0 gate and up, 1 down; the others 0 */
    uint32_t rotation;         /* must be 0: a tensor-parallel feature, not built */
    uint32_t shared_sum;       /* 0: each row's sum float32 at output_offset; 1: added to the shared expert's rows, in place */
    uint64_t shared_offset;    /* shared_sum 1: read and written: bfloat16 [row_count][hidden], bfloat16(sum + row) */
    /* extension */
    uint64_t widths_offset;
    uint32_t hidden;           /* 0: 5120 */
    uint32_t pairs_per_row;    /* 0: 6 */
    uint32_t expert_count;     /* entries of the table at widths_offset (needed with it; else 0): a job of an expert beyond it adds nothing */
    uint32_t reserved_zero;
};
ANEMONE_RECORD_HAS(exl3_tc_record, 96);

/* workspace of the fused decode: fp16 operands [2][pairs][hidden] (later [pairs][intermediate]), float32 gate/up
 * partial products [GATE_UP_SLICES][2][pairs][intermediate], float32 down partials [DOWN_SLICES][pairs][hidden] */
ANEMONE_INLINE uint64_t exl3_tc_operand_bytes(uint64_t pairs, uint64_t hidden)
{
    return (2u * pairs * hidden * 2u + 255u) / 256u * 256u;
}
ANEMONE_INLINE uint64_t exl3_tc_gate_up_bytes(uint64_t pairs, uint64_t intermediate)
{
    return (EXL3_TC_GATE_UP_SLICES * 2u * pairs * intermediate * 4u + 255u) / 256u * 256u;
}
ANEMONE_INLINE uint64_t exl3_tc_down_bytes(uint64_t pairs, uint64_t hidden)
{
    return (EXL3_TC_DOWN_SLICES * pairs * hidden * 4u + 255u) / 256u * 256u;
}
ANEMONE_INLINE uint64_t exl3_tc_workspace_bytes(uint64_t pairs, uint64_t hidden, uint64_t intermediate)
{
    return exl3_tc_operand_bytes(pairs, hidden) + exl3_tc_gate_up_bytes(pairs, intermediate) +
           exl3_tc_down_bytes(pairs, hidden);
}

/* ---- EXL3 prefill: the routed experts as a grouped GEMM (include/anemone/exl3_tc_records.h:205-304 of the
 * reference: struct exl3_tcp_record and its workspace) ----
 * Seven launches of one record: the pairs of each expert counted in blocks of ROUTER_SORT_ROWS rows; every pair placed
 * (sorted by expert, rows ascending), the runs and the chunks of at most EXL3_TCP_CHUNK_PAIRS pairs of one expert; the
 * gate and up operands of every placed pair; the gate/up GEMM; the activation and the down operands; the down GEMM;
 * the combine of a row's pairs in slot order. */
#define EXL3_TCP_KERNEL_FILE "kernel_exl3_tcp"
#define EXL3_TCP_CHUNK_PAIRS 160u  /* columns of one GEMM block: pairs of one expert (ten MFMA column blocks) */
#define EXL3_TCP_PART_COLUMNS 16u /* pairs of a chunk a block of the element-wise launches (operands, activate) takes */
#define EXL3_TCP_COLUMN_PARTS ((EXL3_TCP_CHUNK_PAIRS + EXL3_TCP_PART_COLUMNS - 1u) / EXL3_TCP_PART_COLUMNS)
#define EXL3_TCP_BLOCK_OUTPUTS 256u /* outputs of one GEMM block: four wavefronts of four tiles */
#define EXL3_TCP_LAUNCHES 7u
#define EXL3_TCP_MOST_LAUNCHES 8u  /* the reference's bound of its own forms */
#define EXL3_TCP_MOST_ROWS 16384u
enum exl3_tcp_pass { EXL3_TCP_GATE_AND_UP = 0, EXL3_TCP_GATE = 1, EXL3_TCP_UP = 2, EXL3_TCP_DOWN = 3 };
enum exl3_tcp_launch {
    EXL3_TCP_COUNT_LAUNCH = 0,
    EXL3_TCP_PLACE_LAUNCH = 1,
    EXL3_TCP_OPERANDS_LAUNCH = 2,
    EXL3_TCP_GATE_UP_LAUNCH = 3,
    EXL3_TCP_ACTIVATE_LAUNCH = 4,
    EXL3_TCP_DOWN_LAUNCH = 5,
    EXL3_TCP_COMBINE_LAUNCH = 6
};

struct exl3_tcp_record {
    uint64_t picks_offset;          /* read: struct router_pick [row_count][pairs_per_row] */
    uint64_t expert_offsets_offset; /* read: uint64 [expert_count][3] */
    uint64_t hidden_offset;         /* read: bf16 [row_count][hidden] */
    uint64_t workspace_offset;      /* scratch: exl3_tcp_layout_of(...).total bytes, 256-aligned */
    uint64_t output_offset;         /* written: float32 [row_count][hidden] */
    uint32_t row_count;
    uint32_t intermediate;
    uint32_t bits_x2;               /* the one width as 2 K, unless widths_offset names per-matrix widths */
    uint32_t pass;                  /* the GEMM launches: enum exl3_tcp_pass; the others 0 */
    float activation_limit;
    uint32_t rotation;              /* must be 0: tensor-parallel features of the reference, not built */
    uint32_t half_rows;             /* must be 0 */
    uint32_t part;                  /* must be 0 */
    uint64_t step_offset;           /* unused (cone layers are outside this path) */
    uint32_t cone_layer;            /* must be 0 */
    uint32_t two_blocks;            /* must be 0 */
    /* extension */
    uint64_t widths_offset;
    uint32_t hidden;
    uint32_t pairs_per_row;
    uint32_t expert_count;
    uint32_t reserved_zero;
};
ANEMONE_RECORD_HAS(exl3_tcp_record, 112);

struct exl3_tcp_chunk {
    uint32_t expert;
    uint32_t first_pair; /* place of its first pair among the sorted pairs */
    uint32_t pair_count; /* 1 to EXL3_TCP_CHUNK_PAIRS */
    uint32_t reserved_zero;
};
ANEMONE_RECORD_HAS(exl3_tcp_chunk, 16);

/* The workspace, byte offsets from its start, every part 256-aligned: uint32 counts [blocks][experts]; struct wide_run
 * runs [experts]; a header of four uint32 (the chunks in use first); struct exl3_tcp_chunk chunks [capacity]; uint32
 * sorted [pairs] (the pair at each place); uint32 place_of [pairs]; fp16 operands [2][pairs][hidden], by place (later
 * the down operands [pairs][intermediate]); float32 gate and up products [2][pairs][intermediate]; float32 down
 * products [pairs][hidden]. */
struct exl3_tcp_layout {
    uint64_t counts, runs, header, chunks, sorted, place_of, operands, gate_up, down, total;
    uint32_t chunk_capacity, reserved;
};
ANEMONE_INLINE uint64_t exl3_tcp_rounded(uint64_t bytes)
{
    return (bytes + 255u) / 256u * 256u;
}
ANEMONE_INLINE struct exl3_tcp_layout exl3_tcp_layout_of(uint64_t rows, uint64_t picks, uint64_t experts, uint64_t hidden,
                                                         uint64_t intermediate)
{
    struct exl3_tcp_layout layout = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const uint64_t pairs = rows * picks, blocks = (rows + ROUTER_SORT_ROWS - 1u) / ROUTER_SORT_ROWS;
    layout.chunk_capacity = (uint32_t)(pairs / EXL3_TCP_CHUNK_PAIRS + experts);
    layout.counts = 0;
    layout.runs = layout.counts + exl3_tcp_rounded(blocks * experts * 4u);
    layout.header = layout.runs + exl3_tcp_rounded(experts * 8u);
    layout.chunks = layout.header + 256u;
    layout.sorted = layout.chunks + exl3_tcp_rounded((uint64_t)layout.chunk_capacity * 16u);
    layout.place_of = layout.sorted + exl3_tcp_rounded(pairs * 4u);
    layout.operands = layout.place_of + exl3_tcp_rounded(pairs * 4u);
    layout.gate_up = layout.operands + exl3_tcp_rounded(2u * pairs * hidden * 2u);
    layout.down = layout.gate_up + exl3_tcp_rounded(2u * pairs * intermediate * 4u);
    layout.total = layout.down + exl3_tcp_rounded(pairs * hidden * 4u);
    return layout;
}

/* ---- FP4 / FP8 expert linears ---- */
#define KERNEL_FILE_ACTIVATION_QUANTIZE "kernel_activation_quantize"
#define KERNEL_FILE_EXPERT_LINEAR "kernel_expert_linear"
#define KERNEL_ACTIVATION_QUANTIZE "activation_quantize_entry"
#define KERNEL_ACTIVATION_QUANTIZE_128 "activation_quantize_128_entry" /* no counterpart in the reference: 128 values a float32 scale */
#define KERNEL_EXPERT_GATE_UP_STEM "expert_gate_up_"
#define KERNEL_EXPERT_DOWN_STEM "expert_down_"
#define KERNEL_EXPERT_ROW_SUM "expert_row_sum_entry"

struct activation_quantize_arguments {
    uint64_t values_offset;    /* read: bf16 [V][width] */
    uint64_t codes_offset;     /* written: E4M3 codes [V][width], lane order */
    uint64_t exponents_offset; /* written: E8M0 [V][width / 32] */
    uint64_t operands_offset;  /* written: bf16 x 2^100 [V][width], operand order */
    uint32_t width;
    uint32_t reserved_zero;
};
ANEMONE_RECORD_HAS(activation_quantize_arguments, 40);

struct expert_gate_up_arguments {
    uint64_t jobs_offset;
    uint64_t codes_offset;     /* read: codes [R][input_size] */
    uint64_t exponents_offset;
    uint64_t operands_offset;
    uint64_t hidden_offset;    /* written: bf16 [pair][output_size] */
    uint32_t output_size;
    uint32_t input_size;
    uint32_t pair_count;
    uint32_t pairs_per_row;
    float activation_limit;
    uint32_t reserved_zero;
};
ANEMONE_RECORD_HAS(expert_gate_up_arguments, 64);

/* expert_gate_up_quantize_<S> (include/anemone/expert_fused_records.h:87-103 of the reference): gate with up and the
 * quantization of the hidden vectors in one launch */
#define KERNEL_EXPERT_GATE_UP_QUANTIZE_STEM "expert_gate_up_quantize_"
#define EXPERT_PRODUCER_MOST_PAIRS (LINEAR_MAXIMUM_ROWS * ROUTER_MOST_PICKS)
struct expert_gate_up_quantize_arguments {
    uint64_t jobs_offset;
    uint64_t codes_offset;            /* the rows' quantized input: as expert_gate_up_arguments */
    uint64_t exponents_offset;
    uint64_t operands_offset;
    uint64_t hidden_offset;           /* written (pairs that stand in a job); read (the others) */
    uint64_t hidden_codes_offset;     /* written, of every pair */
    uint64_t hidden_exponents_offset; /* written */
    uint64_t hidden_operands_offset;  /* written */
    uint64_t arrivals_offset;         /* uint32 [jobs][output_size / 32], zeros: not touched by this build's kernels */
    uint32_t output_size;
    uint32_t input_size;
    uint32_t pair_count;
    uint32_t pairs_per_row;
    float activation_limit;
    uint32_t reserved_zero;
};
ANEMONE_RECORD_HAS(expert_gate_up_quantize_arguments, 96);

/* ---- the wide products of the routed experts (include/anemone/wide_linear_records.h:80-118 of the reference) ---- */
#define KERNEL_FILE_WIDE_LINEAR "kernel_wide_linear"
#define KERNEL_WIDE_EXPERT_GATE_UP_STEM "wide_expert_gate_up_"
#define KERNEL_WIDE_EXPERT_DOWN_STEM "wide_expert_down_"
#define WIDE_BLOCK_THREADS 256u          /* four wavefronts: four strips of one tile of pairs */
#define WIDE_GATE_UP_BLOCK_OUTPUTS 128u   /* of gate and of up: a wavefront takes 32 of each */
#define WIDE_GATE_UP_WINDOW_BYTES 53760u  /* dynamic LDS of wide_expert_gate_up_<S>: two stages; three blocks fit a CU */
#define WIDE_GATE_UP_E4M3_BLOCK_OUTPUTS 64u /* of wide_expert_gate_up_e4m3_<S>: a wavefront takes 16 of gate and of up */
#define WIDE_GATE_UP_E4M3_WINDOW_BYTES 53760u /* of wide_expert_gate_up_e4m3_<S>: two stages */
#define WIDE_DOWN_WINDOW_BYTES 51712u     /* of wide_expert_down_<S>: two stages */
#define WIDE_DOWN_E4M3_WINDOW_BYTES 51712u /* of wide_expert_down_e4m3_<S>: two stages */
/* the kernels of the same launches for experts of WEIGHT_FORMAT_E2M1_GFX950 / _E4M3_GFX950: the same records */
#define KERNEL_FILE_NATIVE_LINEAR "kernel_native_linear"
#define KERNEL_NATIVE_EXPERT_GATE_UP_STEM "native_expert_gate_up_"
#define KERNEL_NATIVE_EXPERT_DOWN_STEM "native_expert_down_"
#define NATIVE_E2M1_COLUMN_BLOCKS 4u /* a block of the E2M1_GFX950 launches: one tile of the wide select (64 pairs) */
#define NATIVE_E4M3_COLUMN_BLOCKS 8u /* of the E4M3_GFX950 launches: two tiles of one expert (128 pairs), read once */
#define NATIVE_E2M1_STAGES 2u /* stages of columns in LDS: a K step in use, the next on its way */
#define NATIVE_E4M3_STAGES 3u
/* dynamic LDS: the stages of a K step of the block's columns (128 bytes of codes a column, 4 of scale codes) */
#define NATIVE_WINDOW_BYTES(column_blocks, stages) ((stages) * ((column_blocks) * 2048u + (column_blocks) * 64u))
struct wide_expert_gate_up_arguments {
    uint64_t tiles_offset;            /* read: struct wide_expert_tile [tile_count] */
    uint64_t pairs_offset;            /* read: struct wide_pair [pair_count] */
    uint64_t codes_offset;            /* read: the rows' quantized input [row][input_size] */
    uint64_t exponents_offset;
    uint64_t operands_offset;
    uint64_t hidden_codes_offset;     /* written [pair][output_size], of the tiles' pairs only */
    uint64_t hidden_exponents_offset; /* written [pair][output_size / 32] */
    uint64_t hidden_operands_offset;  /* written [pair][output_size] */
    uint32_t output_size;
    uint32_t input_size;
    uint32_t tile_count;
    uint32_t pairs_per_row;
    float activation_limit;
    uint32_t pair_count;
};
ANEMONE_RECORD_HAS(wide_expert_gate_up_arguments, 88);

struct wide_expert_down_arguments {
    uint64_t tiles_offset;
    uint64_t pairs_offset;
    uint64_t codes_offset;     /* read: the pairs' quantized hidden [pair][input_size] */
    uint64_t exponents_offset;
    uint64_t operands_offset;
    uint64_t output_offset;    /* written: bf16 [pair][output_size], of the tiles' pairs only */
    uint32_t output_size;
    uint32_t input_size;
    uint32_t tile_count;
    uint32_t pair_count;
};
ANEMONE_RECORD_HAS(wide_expert_down_arguments, 64);

struct expert_down_arguments {
    uint64_t jobs_offset;
    uint64_t codes_offset;     /* read: codes [pair][input_size] */
    uint64_t exponents_offset;
    uint64_t operands_offset;
    uint64_t output_offset;    /* written: bf16 [pair][output_size] */
    uint32_t output_size;
    uint32_t input_size;
    uint32_t pair_count;
    uint32_t reserved_zero;
};
ANEMONE_RECORD_HAS(expert_down_arguments, 56);

/* ---- the shared expert and the FFN site's join: the step behind the routed experts ----
 * Records of the reference member for member (include/anemone/linear_records.h:307-356,
 * include/anemone/expert_fused_records.h:100-131, include/anemone/hyper_connection_records.h:79-89). The reference
 * fixes the streams' width at its model's 5,120; here a join's width is what its grid covers: grid[0] x block[0]
 * threads of HYPER_VALUES_PER_THREAD values each. */
#define KERNEL_FILE_TRUNK_LINEAR "kernel_trunk_linear"
#define KERNEL_TRUNK_LINEAR_QUANTIZED_STEM "trunk_linear_quantized_"
#define KERNEL_TRUNK_LINEAR_QUANTIZED_WIDE_STEM "trunk_linear_quantized_wide_"
#define KERNEL_TRUNK_LINEAR_QUANTIZED_INTERLEAVED "trunk_linear_quantized_interleaved_1"
#define KERNEL_TRUNK_HIDDEN "trunk_hidden_entry"
#define KERNEL_EXPERT_SHARED_JOIN_STEM "expert_shared_join_"
#define KERNEL_FILE_HYPER_CONNECTION "kernel_hyper_connection"
#define KERNEL_HYPER_POST "hyper_post_entry"
#define KERNEL_EXPERT_JOIN "expert_join"
#define LINEAR_MERGED_MATRICES 2u /* the most matrices one trunk launch reads */
#define TRUNK_STRIP_OUTPUTS 32u   /* outputs of a block of the thin and the wide trunk kernels: two tiles of one-byte weights */
#define TRUNK_INTERLEAVED_ROWS 64u          /* rows of a block of the interleaved instance: one tile of vectors */
#define TRUNK_INTERLEAVED_BLOCK_OUTPUTS 128u /* its outputs: four wavefronts' strips of two tiles */
#define TRUNK_INTERLEAVED_WINDOW_BYTES 51712u
#define MODEL_STREAMS 4u
#define HYPER_VALUES_PER_THREAD 8u /* one 16-byte load of bfloat16 */
#define HYPER_PIECE_THREADS 128u
#define EXPERT_JOIN_NO_ROW_SUMS UINT64_MAX /* in place of row_sums_offset: the sums are not stored */

struct trunk_linear_quantized_arguments {
    uint64_t weights_offset[LINEAR_MERGED_MATRICES]; /* read: WEIGHT_FORMAT_E4M3_SCALED matrices of one input_size */
    uint64_t output_offset[LINEAR_MERGED_MATRICES];  /* written: bf16 [row_count][output_size[m]] */
    uint64_t codes_offset;                           /* read: the rows' codes, exponents, operands */
    uint64_t exponents_offset;
    uint64_t operands_offset;
    uint32_t output_size[LINEAR_MERGED_MATRICES];    /* [1] is 0 where there is one matrix */
    uint32_t input_size;
    uint32_t row_count;
};
ANEMONE_RECORD_HAS(trunk_linear_quantized_arguments, 72);

struct trunk_hidden_arguments { /* the hidden step alone, route weight 1; grid[1] vectors */
    uint64_t gate_offset;   /* read: bf16 [V][width] */
    uint64_t up_offset;
    uint64_t hidden_offset; /* written: bf16 [V][width] */
    uint32_t width;
    float activation_limit;
};
ANEMONE_RECORD_HAS(trunk_hidden_arguments, 32);

struct hyper_post_arguments {
    uint64_t streams_offset; /* read and written: bf16 [row][4][width] */
    uint64_t post_offset;    /* read: float32 [row][4] */
    uint64_t comb_offset;    /* read: float32 [row][4 sources][4 targets] */
    uint64_t output_offset;  /* read: bf16 [row][width], the sublayer's or the shared expert's */
    uint64_t sums_offset;    /* read with the combine alone: float32 [row][width] */
    uint32_t is_combined;
    uint32_t reserved_zero;
};
ANEMONE_RECORD_HAS(hyper_post_arguments, 48);

struct expert_join_arguments {
    uint64_t pair_output_offset;   /* read: bf16 [row * pairs_per_row + slot][width] */
    uint64_t shared_output_offset; /* read: bf16 [row][width] */
    uint64_t streams_offset;       /* read and written */
    uint64_t post_offset;
    uint64_t comb_offset;
    uint64_t row_sums_offset;      /* written: float32 [row][width], or EXPERT_JOIN_NO_ROW_SUMS */
    uint32_t pairs_per_row;
    uint32_t reserved_zero;
};
ANEMONE_RECORD_HAS(expert_join_arguments, 56);

struct expert_shared_join_arguments {
    uint64_t weights_offset;     /* the shared expert's down: E4M3_SCALED, the streams' width by input_size */
    uint64_t codes_offset;       /* its quantized input, as trunk_linear_quantized_arguments */
    uint64_t exponents_offset;
    uint64_t operands_offset;
    uint64_t output_offset;      /* written: the shared expert's output, bf16 [row][width] */
    uint64_t pair_output_offset; /* the join's, as expert_join_arguments */
    uint64_t streams_offset;
    uint64_t post_offset;
    uint64_t comb_offset;
    uint64_t row_sums_offset;
    uint32_t input_size;
    uint32_t row_count;
    uint32_t pairs_per_row;
    uint32_t reserved_zero;      /* extension: the streams' width (the down matrix's outputs); 0 stands for 5,120 */
};
ANEMONE_RECORD_HAS(expert_shared_join_arguments, 96);

/* ---- the launches a site front stands for: the mix finish and the dense product ----
 * include/anemone/hyper_connection_records.h:46-84 and include/anemone/dense_linear_records.h:56-148 of the reference. */
#define KERNEL_HYPER_MIX_FINISH "hyper_mix_finish"
#define MODEL_MIXES 24u                 /* (2 + streams) x streams: pre, post, comb */
#define MODEL_HYPER_EPSILON 1e-6f
#define MODEL_NORM_EPSILON 1e-20f
#define MODEL_SINKHORN_ITERATIONS 20u
#define HYPER_SCALES 3u                 /* pre, post, comb */
#define HYPER_FINISH_MOST_THREADS 1024u /* a row's values over 8: the widths 256 .. 8192 in whole groups of 32 threads */

/* Launch: grid (1, rows), block width / 8: a thread eight values of the row; the width is what the block covers (the
 * reference fixes 5,120 and adds a group of 32 threads for Sinkhorn: here the first sixteen threads do it behind the
 * barrier). */
struct hyper_finish_arguments {
    uint64_t streams_offset; /* read: bf16 [row][4][width] */
    uint64_t pre_offset;     /* float32 [row][4]: the carried pre, read; then the site's, written */
    uint64_t mixes_offset;   /* read: float32 [row][24] */
    uint64_t scale_offset;   /* read: float32 [3] */
    uint64_t base_offset;    /* read: float32 [24] */
    uint64_t post_offset;    /* written: float32 [row][4] */
    uint64_t comb_offset;    /* written: float32 [row][4][4] */
    uint64_t weight_offset;  /* read: the norm's, bf16 [width] */
    uint64_t hidden_offset;  /* written: bf16 [row][width] */
};
ANEMONE_RECORD_HAS(hyper_finish_arguments, 72);

#define KERNEL_FILE_DENSE_LINEAR "kernel_dense_linear"
#define KERNEL_DENSE_LINEAR_STEM "dense_linear_"
#define DENSE_OUTPUTS_PER_BLOCK 4u
#define DENSE_NARROW_BELOW_BLOCKS 256u /* fewer blocks than this: a block owns one output, so that more units read */
#define DENSE_CHUNK_INPUTS 8u
#define DENSE_THREADS_VALUE 256u
#define DENSE_ROW_SCALE 0x1u
#define DENSE_STEP_ROWS 0x2u /* not built: the head's */
#define DENSE_CONE_ROWS 0x4u /* not built: the prefill cone's */
#define DENSE_FLAGS (DENSE_ROW_SCALE | DENSE_STEP_ROWS | DENSE_CONE_ROWS)
enum dense_type_code { DENSE_BFLOAT16 = 0, DENSE_FLOAT32 = 1, DENSE_TYPE_COUNT = 2 };
#define DENSE_FORMS 2u          /* four outputs a block, then one (narrow) */
#define DENSE_INSTANCES 8u      /* forms by types by row counts: [form][type][one row, 8] */
#define DENSE_FORM_INSTANCES 4u
#define DENSE_ROW_INSTANCES 2u
#define DENSE_WIDE_OUTPUTS 8u /* outputs of a block of dense_linear_<type>_8_wide: steps of more than 8 rows, groups of 8 on grid[1] */
#define DENSE_MOST_ROWS 65535u

/* Launch: function dense_linear_<type>_<R>[_narrow], R 1 for one row and 8 for 2 to 8; grid (output_size / outputs of
 * a block, 1), block 256. */
struct dense_linear_arguments {
    uint64_t weights_offset; /* read: [output_size][input_size] of the instance's type */
    uint64_t rows_offset;    /* read: bf16 [row_count][input_size] */
    uint64_t output_offset;  /* written: [row_count][output_size] of output_type */
    uint64_t step_offset;    /* not read (DENSE_STEP_ROWS and _CONE_ROWS are not built) */
    uint32_t output_size;
    uint32_t input_size;
    uint32_t row_count;
    uint32_t output_type;    /* enum dense_type_code */
    uint32_t flags;          /* DENSE_ROW_SCALE or 0 */
    float output_scale;
    float epsilon;           /* of DENSE_ROW_SCALE */
    uint32_t cone_layer;     /* 0 */
};
ANEMONE_RECORD_HAS(dense_linear_arguments, 64);

/* ---- the fused fronts of a block's sites (include/anemone/site_front_records.h of the reference): a site's mix project,
 * its mix finish and the quantization of the sublayer's input in ONE launch (site_front_<R>); the FFN front also the
 * router's scores, in the dense product's order, and its select between the finish and the quantization
 * (ffn_front_<R>). R = 1 for one row, 8 for 2 to 8 rows. Every output has the bits of the launches the front stands for.
 *
 * A front is a grid of blocks of width / 8 threads that take tickets from the scratch's first counter and their parts in
 * the tickets' order: the rows' blocks first (a row's input from its streams and the carried pre, and its quantization:
 * they wait for nothing), then the mix project's blocks (the last of them to publish its mixes waits for the rows' blocks,
 * which read the pre it writes, and forms every row's post, comb and pre), then the scores' blocks (they wait for the
 * rows' inputs; the last of them to publish its scores runs the select). A block waits only for blocks of lower tickets,
 * which are running and wait for nothing: the grid ends whatever part of it the card holds at once. No floating-point
 * result depends on the tickets. The last block to leave puts every counter back to zero. The input front
 * (the rows' blocks: a row a block, no counter) and then the coefficient front (the mix project's blocks; the last to
 * publish forms post, comb and pre and clears that counter) are the site front in two launches of one stream.
 *
 * The record is the reference's, 192 bytes: its router_select_arguments (80 bytes there) first, then the fourteen
 * offsets. What this build's select takes beside the reference's members (expert count, picks a row, affinity kind, route
 * scale) rides in the word of reference_order: bit 0 reference_order, bits 1-10 the expert count (0: 384), bits 11-14 the
 * picks (0: 6), bit 15 the affinity kind, bits 16-31 the route scale as fp16 (0: 1.5): all zero is the reference's model. */
#define KERNEL_FILE_SITE_FRONT "kernel_site_front"
#define KERNEL_SITE_FRONT_STEM "site_front_"
#define KERNEL_FFN_FRONT_STEM "ffn_front_"
#define SITE_FRONT_ARGUMENT_BYTES 192u
#define SITE_FRONT_SCRATCH_BYTES 7184u
#define SITE_FRONT_MOST_WIDTH 5120u /* blocks of width / 8 threads whose 8-row dense products need 168 registers */
#define SITE_FRONT_SCORE_OUTPUTS 4u /* experts of a block's quarter (256 threads: the dense product's block) */
#define SITE_FRONT_MIX_OUTPUTS 2u   /* mixes of a block's quarter */
#define SITE_FRONT_WAIT_POLLS (1u << 20) /* of a counter, some 100 ns apart; then the block gives up (scratch.gave_up) and leaves */
enum site_front_kind {
    SITE_FRONT_KIND_SITE = 0,
    SITE_FRONT_KIND_FFN = 1,
    SITE_FRONT_KIND_INPUT = 2,        /* the site front's first half: hidden, codes, exponents, operands */
    SITE_FRONT_KIND_COEFFICIENTS = 3, /* its second half: the mixes, post, comb, the site's pre */
    SITE_FRONT_KINDS = 4
};
#define SITE_FRONT_ROW_FORMS 2u /* one row, 8 */
#define SITE_FRONT_INSTANCES (SITE_FRONT_KINDS * SITE_FRONT_ROW_FORMS)

struct site_front_select {
    uint64_t step_offset;
    uint64_t scores_offset;          /* the FFN front: written, then read */
    uint64_t bias_offset;
    uint64_t expert_offsets_offset;
    uint64_t affinities_offset;
    uint64_t jobs_offset;
    uint64_t weights_offset;
    uint64_t gate_up_last_offset;
    uint64_t down_last_offset;
    uint32_t row_count;              /* the site front reads nothing else of the select */
    uint32_t reference_order_and_shape;
};
ANEMONE_RECORD_HAS(site_front_select, 80);

ANEMONE_INLINE uint32_t site_front_shape_word(uint32_t reference_order, uint32_t expert_count, uint32_t pick_count, uint32_t affinity_kind,
                                              uint32_t route_scale_fp16)
{
    return (reference_order & 1u) | ((expert_count & 1023u) << 1) | ((pick_count & 15u) << 11) | ((affinity_kind & 1u) << 15) |
           (route_scale_fp16 << 16);
}

/* the blocks of a front of blocks of width / 8 threads: a quarter (256 threads) takes SITE_FRONT_MIX_OUTPUTS mixes or
 * SITE_FRONT_SCORE_OUTPUTS experts, a block as many quarters as it holds whole */
ANEMONE_INLINE uint32_t site_front_mix_blocks(uint32_t width)
{
    return (MODEL_MIXES / SITE_FRONT_MIX_OUTPUTS + width / 2048u - 1u) / (width / 2048u);
}
ANEMONE_INLINE uint32_t site_front_score_blocks(uint32_t width, uint32_t expert_count)
{
    return (expert_count / SITE_FRONT_SCORE_OUTPUTS + width / 2048u - 1u) / (width / 2048u);
}

struct site_front_arguments {
    struct site_front_select select;
    uint64_t streams_offset;        /* read: bf16 [row][4][width] */
    uint64_t pre_offset;            /* read, then written: the carried pre, then the site's */
    uint64_t scale_offset;          /* read: float32 [3] */
    uint64_t base_offset;           /* read: float32 [24] */
    uint64_t post_offset;           /* written */
    uint64_t comb_offset;           /* written */
    uint64_t norm_weight_offset;    /* read: bf16 [width] */
    uint64_t hidden_offset;         /* written (and read by the FFN front's scores) */
    uint64_t mix_weights_offset;    /* read: float32 [24][4 width] */
    uint64_t codes_offset;          /* written: codes [row_count][width] */
    uint64_t exponents_offset;      /* written: exponents [row_count][width / 32] */
    uint64_t operands_offset;       /* written: operands [row_count][width] */
    uint64_t scratch_offset;        /* struct site_front_scratch: its mixes written, its counters zero again */
    uint64_t router_weights_offset; /* read by the FFN front: bf16 [experts][width] */
};
ANEMONE_RECORD_HAS(site_front_arguments, SITE_FRONT_ARGUMENT_BYTES);

struct site_front_scratch {
    uint32_t tickets, arrived, rows_ready, scored; /* zero before a launch and after it */
    float mixes[LINEAR_MAXIMUM_ROWS][MODEL_MIXES]; /* the launch's rows' */
    uint32_t departed;                             /* zero before a launch and after it */
    uint32_t gave_up;                              /* blocks that waited SITE_FRONT_WAIT_POLLS polls in vain: zero on a sound card */
    uint32_t reserved[62 + MODEL_MIXES * 8u * LINEAR_MAXIMUM_ROWS]; /* where the reference's blocks leave their partial sums */
};
ANEMONE_RECORD_HAS(site_front_scratch, SITE_FRONT_SCRATCH_BYTES);

#endif
