/*
 * anemone_ops.h -- the host-side operator entry points of the routed-expert path: load-time "prepare" functions
 * that check a description and fill immutable `struct kernel_launch` tables. C11, no device code, no allocation.
 *
 * Each function keeps the name, the argument meaning and the refusal rules of the reference function it replaces:
 *   weight_format_operations_of          include/anemone/weight_format_seam.h:93-94   (source/weight_format.c)
 *   exl3_*                               include/anemone/exl3.h:11-61                  (source/exl3.c)
 *   exl3_row_sum_prepare                 include/anemone/exl3_tp.h:77-80 (bb_exl3_row_sum_prepare; source/exl3_tp.c:250-290)
 *   exl3_tc_prepare, exl3_tcp_prepare    include/anemone/exl3_tc.h:22-59               (source/exl3_tc.c)
 *   router_*                             include/anemone/router.h:50-124               (source/router.c)
 *   linear_*                             include/anemone/linear.h:117-411              (source/linear.c, routed part)
 *   expert_producer_prepare              include/anemone/expert_fused.h:51-101         (source/expert_fused.c)
 * Contract of every prepare function (include/anemone/linear.h:17-48): arithmetic on a description, the arena is a
 * number; pure and reentrant; a refusal is a status with one error line on stderr and the launch table untouched.
 * What differs from the reference: shapes (experts, picks, hidden, widths) are run-time members instead of one
 * model's compile-time constants, and the arithmetic class accepted is ARITHMETIC_CLASS_GFX950.
 */
#ifndef ANEMONE_OPS_H
#define ANEMONE_OPS_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#include "anemone_backend.h"
#include "anemone_records.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- ranges, shapes, formats ---- */
struct linear_range {
    uint64_t byte_offset;
    uint64_t byte_count;
};
struct matrix_shape_record {
    uint32_t output_size;
    uint32_t input_size;
    uint32_t bits_per_weight; /* EXL3: a stored width; a format of one width checks its figure */
    uint32_t reserved_must_be_zero;
};
struct weight_format_operations {
    const char *name;
    MUST_CHECK result_status (*stored_byte_count)(const struct matrix_shape_record *shape, uint64_t *byte_count_out);
};
const struct weight_format_operations *weight_format_operations_of(enum weight_format_code format);
extern const struct weight_format_operations exl3_weight_operations;

/* Load-time re-lay-out between the reference's lane order and gfx950's (host only: bytes move, no weight or scale code
 * changes; no allocation). A matrix [outputs][inputs], outputs a multiple of 64 (32 for E4M3), inputs of 128, is tiles of
 * 16 outputs by K steps of 128 inputs. In a GFX950 format the tiles follow each other, a tile's K steps follow each
 * other, and a K step is the 64 lanes' A operand of v_mfma_scale_f32_16x16x128_f8f6f4, lane 16 g + o holding output o:
 *   E2M1_GFX950  16 bytes a lane: nibble n (0: low) of byte b of word T is input 32 g + 16 n + 2 T + {0, 8, 1, 9}[b] of
 *                the step; behind all tiles the scale codes, the tiles in groups of four (outputs a multiple of 64): a
 *                group's K step is a word a lane ([group][step][lane][4]), byte n the E8M0 code of output o of the
 *                group's tile n, inputs 32 g .. 32 g + 31: a wavefront's strip of two or four tiles takes its codes with
 *                one load and the matrix instruction picks the byte. Bytes: outputs inputs / 2 + outputs inputs / 32.
 *   E4M3_GFX950  32 bytes a lane as two halves of 1,024 bytes a step ([half][lane][16]): byte c of word v (0 .. 7; half
 *                v / 4) is input 64 (v / 4) + 16 g + 8 (c % 2) + 2 (v % 4) + c / 2; behind all tiles the scale codes as
 *                E4M3_SCALED stores them (a row of inputs / 32 for every 32 outputs). Bytes: E4M3_SCALED's.
 *   E4M3_BLOCK128_GFX950  E4M3_GFX950's bytes of codes; behind them E4M3_BLOCK128's float32 scales [outputs / 128][inputs /
 *                128] (outputs and inputs multiples of 128). Bytes: E4M3_BLOCK128's.
 * The byte a lane's register holds is the byte the reference-format kernels of this library form there from the
 * reference's lay-out, so both formats' kernels run the same sums. pack: from E2M1_SCALED to E2M1_GFX950, from
 * E4M3_SCALED to E4M3_GFX950 or from E4M3_BLOCK128 to E4M3_BLOCK128_GFX950 (`format` names the GFX950 format); unpack: back. The two byte counts must be the
 * formats' stored_byte_count of the shape and the buffers apart; else STATUS_INVALID_ARGUMENT and nothing is written. */
MUST_CHECK result_status weight_format_gfx950_pack(enum weight_format_code format, const struct matrix_shape_record *shape,
                                                   const void *reference_bytes, uint64_t reference_byte_count, void *packed_out,
                                                   uint64_t packed_byte_count);
MUST_CHECK result_status weight_format_gfx950_unpack(enum weight_format_code format, const struct matrix_shape_record *shape,
                                                     const void *packed_bytes, uint64_t packed_byte_count, void *reference_out,
                                                     uint64_t reference_byte_count);

enum linear_order_code { LINEAR_ORDER_FIXED = 0, LINEAR_ORDER_REFERENCE = 1 };

/* ---- EXL3 chain ---- */
const char *exl3_width_name(uint32_t bits_x2); /* "k2", "k2_5", "k3", "k4"; NULL for a width without entries */
MUST_CHECK result_status exl3_reconstruct_prepare(const struct exl3_reconstruct_record *record,
                                                  uint64_t arena_byte_count, uint32_t kernel,
                                                  struct kernel_launch *launch_out);
uint64_t exl3_scratch_byte_count(uint32_t pair_count, uint32_t input_size);
/* launches_out: EXL3_EXPERT_LAUNCHES launches (input, gate/up, activate, down, finish) */
MUST_CHECK result_status exl3_experts_prepare(const struct exl3_expert_record *record, uint64_t arena_byte_count,
                                              const struct backend_operations *backend, struct device_card *card,
                                              uint32_t arithmetic_class, struct kernel_launch *launches_out);
/* the reference's alternative work mappings of the same words; on gfx950 there is one mapping, so fast == retained */
MUST_CHECK result_status exl3_experts_fast_prepare(const struct exl3_expert_record *record,
                                                   uint64_t arena_byte_count,
                                                   const struct backend_operations *backend,
                                                   struct device_card *card, uint32_t arithmetic_class,
                                                   struct kernel_launch *launches_out);
/* another association of the float32 sums, the CMP cards' own: STATUS_UNSUPPORTED on any other class, so here */
MUST_CHECK result_status exl3_experts_relaxed_prepare(const struct exl3_expert_record *record,
                                                      uint64_t arena_byte_count,
                                                      const struct backend_operations *backend,
                                                      struct device_card *card, uint32_t arithmetic_class,
                                                      struct kernel_launch *launches_out);
MUST_CHECK result_status exl3_row_sum_prepare(const struct expert_row_sum_arguments *record, uint32_t rows,
                                              uint64_t arena_bytes, const struct backend_operations *backend,
                                              struct device_card *card, struct kernel_launch *launch_out);

/* ---- EXL3 fused decode (1 .. EXL3_TC_MOST_ROWS rows): EXL3_TC_LAUNCHES launches ---- */
MUST_CHECK result_status exl3_tc_prepare(const struct exl3_tc_record *record, uint64_t arena_byte_count,
                                         const struct backend_operations *backend, struct device_card *card,
                                         struct kernel_launch launches_out[EXL3_TC_LAUNCHES]);
/* the reference's row-count-independent and paired forms: on gfx950 exl3_tc_prepare already is row-count
 * independent (a row's bits do not depend on the other rows), so both are the same launches */
MUST_CHECK result_status exl3_tc_prepare_short(const struct exl3_tc_record *record, uint64_t arena_byte_count,
                                               const struct backend_operations *backend, struct device_card *card,
                                               struct kernel_launch launches_out[EXL3_TC_LAUNCHES]);
MUST_CHECK result_status exl3_tc_prepare_paired(const struct exl3_tc_record *record, uint64_t arena_byte_count,
                                                const struct backend_operations *backend, struct device_card *card,
                                                struct kernel_launch launches_out[EXL3_TC_LAUNCHES]);

/* exl3_tc_prepare's launches for a workspace that is not a range of the arena (its offset is checked for alignment only);
 * what exl3_tc_run_static builds its launches with */
MUST_CHECK result_status exl3_tc_prepare_detached(const struct exl3_tc_record *record, uint64_t arena_byte_count,
                                                  const struct backend_operations *backend, struct device_card *card,
                                                  struct kernel_launch launches_out[EXL3_TC_LAUNCHES]);

/* No counterpart in the reference. For callers that cannot allocate device memory (code under graph capture, serving
 * loops and harnesses that forbid it): the fused decode of exl3_tc_prepare + launch_run, its five launches queued on
 * `stream` (a hipStream_t; NULL: the default stream) of the current device, with the workspace in an array of
 * EXL3_TC_STATIC_SCRATCH_BYTES that the library holds on every device it has run on, in place of a range of the arena.
 * `arena_device` is the device address the record's offsets count from and `arena_byte_count` the bytes behind it that
 * the record's ranges must lie in; record->workspace_offset is ignored. Allocates nothing and does not wait: the array's
 * address on a device is found when card_open opens that device (which loads the library's code there); on a device no
 * card was opened on, the first call finds it itself, and that one call may load code and must not be made under
 * capture. A step
 * whose workspace (exl3_tc_workspace_bytes) is larger than the array is refused with STATUS_INVALID_ARGUMENT. Calls on
 * one device share that device's array: two calls whose launches overlap in time race. */
#define EXL3_TC_STATIC_SCRATCH_BYTES (16u << 20)
MUST_CHECK result_status exl3_tc_run_static(const struct exl3_tc_record *record, void *arena_device,
                                            uint64_t arena_byte_count, void *stream);

/* The prefill form (include/anemone/exl3_tc.h:40-59 of the reference): fills launches_out and *launch_count_out
 * (EXL3_TCP_LAUNCHES here). The reference's _base and _hybrid choose between two GEMM forms of the same bits; this
 * library has one form behind all three names. */
MUST_CHECK result_status exl3_tcp_prepare(const struct exl3_tcp_record *record, uint64_t arena_byte_count,
                                          const struct backend_operations *backend, struct device_card *card,
                                          struct kernel_launch launches_out[EXL3_TCP_MOST_LAUNCHES],
                                          uint32_t *launch_count_out);
MUST_CHECK result_status exl3_tcp_prepare_base(const struct exl3_tcp_record *record, uint64_t arena_byte_count,
                                               const struct backend_operations *backend, struct device_card *card,
                                               struct kernel_launch launches_out[EXL3_TCP_MOST_LAUNCHES],
                                               uint32_t *launch_count_out);
MUST_CHECK result_status exl3_tcp_prepare_hybrid(const struct exl3_tcp_record *record, uint64_t arena_byte_count,
                                                 const struct backend_operations *backend, struct device_card *card,
                                                 struct kernel_launch launches_out[EXL3_TCP_MOST_LAUNCHES],
                                                 uint32_t *launch_count_out);

/* ---- router ---- */
struct router_kernels_record {
    uint32_t select;
    uint32_t wide_select;
    uint32_t wide_count;
    uint32_t wide_place;
    uint32_t wide_jobs;
    uint32_t wide_small;
    uint32_t select_draft; /* BACKEND_NO_KERNEL: the draft's router is outside this path */
    uint32_t projection;   /* no counterpart: the router's score projection as its own launch */
    uint32_t projection_tiles; /* no counterpart: the same scores for steps of 257 rows and more, on the matrix unit */
};
MUST_CHECK result_status router_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                                struct router_kernels_record *kernels_out);

/* the subset of the reference's linear_routed_experts_description the router checks its table against */
struct linear_routed_experts_description {
    struct linear_range jobs;           /* struct expert_job_record [job_count] */
    struct linear_range expert_weights; /* holds every matrix a job names */
    struct linear_range codes, exponents, operands;
    struct linear_range hidden, hidden_codes, hidden_exponents, hidden_operands;
    struct linear_range pair_output, row_output;
    struct matrix_shape_record gate_up_shape;
    struct matrix_shape_record down_shape;
    enum weight_format_code weight_format; /* E2M1_SCALED, E4M3_SCALED or EXL3 */
    uint32_t job_count;
    uint32_t row_count;
    uint32_t pairs_per_row;
    uint32_t gate_up_slice_count;
    uint32_t down_slice_count;
    float activation_limit;
    uint32_t reserved_zero;
};

struct router_description {
    const struct linear_routed_experts_description *experts;
    const uint64_t *expert_offsets; /* [E][3]: what the arena holds at offsets */
    const uint32_t *expert_widths;  /* EXL3 with per-matrix widths: [E] packed as in the arena; else NULL */
    struct linear_range step, scores, bias, offsets, affinities;
    enum linear_order_code order;
    uint32_t expert_count; /* 1 .. ROUTER_MOST_EXPERTS, a multiple of 64 */
    uint32_t pick_count;   /* 1 .. ROUTER_MOST_PICKS */
    uint32_t affinity_kind;
    float route_scale;
};
MUST_CHECK result_status router_select_prepare(const struct router_description *description,
                                               uint64_t arena_byte_count,
                                               const struct router_kernels_record *kernels,
                                               struct kernel_launch *launch_out);

struct router_projection_description {
    struct linear_range weights, rows, output;
    uint32_t row_count, hidden, expert_count, reserved_zero;
};
MUST_CHECK result_status router_projection_prepare(const struct router_projection_description *description,
                                                   uint64_t arena_byte_count,
                                                   const struct router_kernels_record *kernels,
                                                   struct kernel_launch *launch_out);

enum router_wide_launch {
    ROUTER_WIDE_SELECT_LAUNCH = 0,
    ROUTER_WIDE_COUNT_LAUNCH = 1,
    ROUTER_WIDE_PLACE_LAUNCH = 2,
    ROUTER_WIDE_JOBS_LAUNCH = 3,
    ROUTER_WIDE_LAUNCH_COUNT = 4
};
struct router_wide_description {
    const uint64_t *expert_offsets;
    const uint32_t *expert_widths;
    struct linear_range step, scores, bias, offsets, expert_weights, affinities;
    struct linear_range picks, counts, pairs, runs, tiles, jobs;
    struct matrix_shape_record gate_up_shape, down_shape;
    enum weight_format_code weight_format;
    enum linear_order_code order;
    uint32_t row_count;
    uint32_t reserved_zero;
    uint32_t expert_count, pick_count, affinity_kind;
    float route_scale;
};
MUST_CHECK result_status router_wide_prepare(const struct router_wide_description *description,
                                             uint64_t arena_byte_count,
                                             const struct router_kernels_record *kernels,
                                             struct kernel_launch *launches_out);
/* include/anemone/router.h:117-124 of the reference: the same of at most ROUTER_SORT_ROWS rows in two launches, the
 * select and router_wide_small (the count, the place and the jobs in one block: the same picks, affinities, pairs,
 * runs, tiles and jobs; the counts scratch unwritten). More rows: STATUS_INVALID_ARGUMENT. */
#define ROUTER_WIDE_SMALL_LAUNCH_COUNT 2u
MUST_CHECK result_status router_wide_small_prepare(const struct router_wide_description *description,
                                                   uint64_t arena_byte_count,
                                                   const struct router_kernels_record *kernels,
                                                   struct kernel_launch *launches_out);

/* ---- the fused fronts of a block's sites (include/anemone/site_front.h:38-40, 42-75 of the reference) ---- */
struct site_front_kernels {
    uint32_t fronts[SITE_FRONT_INSTANCES]; /* site_front_1, _8, ffn_front_1, _8, input_front_1, _8, coefficient_front_1, _8 */
};
MUST_CHECK result_status site_front_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                                    struct site_front_kernels *kernels_out);
struct site_front_description {
    struct linear_range streams;     /* read: bf16 [row][4][width] */
    struct linear_range carried_pre; /* read, then written */
    struct linear_range mix_weights; /* read: float32 [24][4 width], exactly */
    struct linear_range scale;       /* read: float32 [3], exactly */
    struct linear_range base;        /* read: float32 [24], exactly */
    struct linear_range norm_weight; /* read: bf16 [width], exactly */
    struct linear_range post;        /* written */
    struct linear_range comb;        /* written */
    struct linear_range hidden;      /* written: the sublayer's input */
    struct linear_range codes;       /* written: [row_count][width] */
    struct linear_range exponents;   /* written: [row_count][width / 32] */
    struct linear_range operands;    /* written: [row_count][width] */
    struct linear_range scratch;     /* struct site_front_scratch, its counters zero */
    const struct router_description *router; /* the FFN front's select (its scores written too), or NULL */
    struct linear_range router_weights;      /* read by the FFN front: bf16 [experts][width], exactly */
    uint32_t kind;                   /* enum site_front_kind; FFN exactly where router is given */
    uint32_t row_count;
    uint32_t reserved_zero;          /* the width; 0: 5,120 (the reference's model) */
};
/* fills ONE launch: a whole front, or one of the two the site front is cut in (SITE_FRONT_KIND_INPUT, then _COEFFICIENTS) */
MUST_CHECK result_status site_front_prepare(const struct site_front_description *description, uint64_t arena_byte_count,
                                            const struct router_kernels_record *router_kernels,
                                            const struct site_front_kernels *kernels, struct kernel_launch *launch_out);
/* A fused front's blocks wait for each other a bounded number of polls (SITE_FRONT_WAIT_POLLS); one that waits in vain
 * counts itself in the scratch's gave_up, skips its part and leaves, and the launch still ends like any other. The count is
 * the caller's to read: this call brings it back from the card (behind every launch queued before it; staging: 8
 * page-locked bytes), writes it to gave_up_out (may be NULL) and, where it is not zero, clears it on the card and answers
 * STATUS_DEVICE_ERROR: what that launch wrote is not whole and the step must not go on. STATUS_OK: every block ran its
 * part. No counterpart in the reference, whose fronts wait without a bound (source/kernel_site_front.cu). */
MUST_CHECK result_status site_front_check(const struct backend_operations *backend, struct device_card *card,
                                          struct linear_range scratch, void *staging, uint64_t wait_limit_nanoseconds,
                                          uint32_t *gave_up_out);

/* ---- host experts: a step's expert pauses (include/anemone/model_seam.h:193-214, source/step_experts.c:27-168 of the
 * reference). Behind a layer's router, whose job table names a host expert i of the layer by three offsets equal to
 * slots_offset + 16 i, each such expert is put into one of the card's slots (slot k at slots_offset + k
 * slot_byte_count; uploaded unless a slot holds it already) and the job's offsets are pointed there; any other job keeps
 * its offsets, all below slots_offset. ---- */
#define EXPERT_PAUSE_MATRICES 3u
struct expert_pause { /* model_seam.h:202-214, member for member */
    uint64_t jobs_offset;
    uint64_t slots_offset;
    uint64_t slot_byte_count;
    uint64_t expert_byte_count; /* at most slot_byte_count */
    uint64_t matrix_offsets[EXPERT_PAUSE_MATRICES]; /* of gate, up, down inside an expert's bytes */
    uint32_t first_host_expert;
    uint32_t host_expert_count;
    uint32_t jobs_per_row;
    uint32_t slot_count; /* at least jobs_per_row times the most rows of a step */
    uint32_t card;
    uint32_t after_segment;
};
/* what the reference's step driver keeps of a card's slots between pauses (source/step_driver.h:17, 73): the caller's here */
#define EXPERT_SLOT_FIELDS 2u
struct expert_slots {
    uint64_t *fields;    /* [slot_count][2]: the host expert the slot holds + 1 (0: none), the mark of the pause that took it last */
    uint64_t pause_mark; /* of the last pause */
    uint32_t slot_count;
    uint32_t next_slot;  /* the slot the next upload tries first */
};
struct expert_pause_upload {
    uint32_t slot;
    uint32_t host_expert; /* of the pause's: 0 .. host_expert_count - 1 */
};
/* The walk over a job table in host memory: the jobs' offsets pointed into slots, the slots' state moved on, the uploads
 * the pause owes listed in their order (uploads_out: job_count places). STATUS_DEVICE_ERROR for a job that names neither
 * an expert on the card nor a host expert of the pause (a tag off the tags' step, beyond the layer's, matrices apart,
 * partly a tag), as the reference answers. */
MUST_CHECK result_status expert_pause_plan(const struct expert_pause *pause, struct expert_job_record *jobs, uint64_t job_count,
                                           struct expert_slots *slots, struct expert_pause_upload *uploads_out,
                                           uint32_t *upload_count_out, uint32_t *tag_count_out);
/* The pause on a card: the job table back into jobs_staging (page-locked, jobs_per_row row_count records), the walk, the
 * experts up from expert_copies (page-locked: the pause's host experts, expert_byte_count apart), the job table up again
 * where a tag was in it; every copy is finished when the call returns. */
MUST_CHECK result_status expert_pause_run(const struct backend_operations *backend, struct device_card *card,
                                          const struct expert_pause *pause, uint32_t row_count, struct expert_slots *slots,
                                          void *jobs_staging, const unsigned char *expert_copies, uint64_t wait_limit_nanoseconds,
                                          uint32_t *upload_count_out);

/* The page-locked copies the pauses of one card upload from: what the reference's step driver makes when host experts are
 * attached to it (include/anemone/step.h:55, 189; source/step_experts.c:170-240 of the reference: every host expert the
 * pauses name is copied once out of the host arena into memory from the backend's staging_allocate, a pause's experts
 * side by side, expert_byte_count apart). Here the block also holds, behind the experts and on a multiple of 256,
 * table_staging_bytes for the job table expert_pause_run brings back. pause_offsets_out[p] is where pause p's copies
 * begin: expert_pause_run takes block + pause_offsets_out[p] as expert_copies and block + table_staging_offset as
 * jobs_staging. host_expert_offsets [host_expert_count] are byte offsets into host_arena (host_byte_count bytes).
 * STATUS_INVALID_ARGUMENT: a pause without host experts, experts beyond the table or the arena; STATUS_OUT_OF_MEMORY:
 * more than most_bytes in all, or the backend's answer. A refusal allocates nothing and leaves both outputs untouched. */
struct expert_host_copies {
    unsigned char *block;          /* page-locked; NULL: nothing attached */
    uint64_t byte_count;           /* of the block */
    uint64_t table_staging_offset; /* in the block */
};
MUST_CHECK result_status expert_host_copies_attach(const struct backend_operations *backend, const struct expert_pause *pauses,
                                                   uint32_t pause_count, const uint64_t *host_expert_offsets,
                                                   uint64_t host_expert_count, const void *host_arena, uint64_t host_byte_count,
                                                   uint64_t table_staging_bytes, uint64_t most_bytes,
                                                   struct expert_host_copies *copies_out, uint64_t *pause_offsets_out);
/* gives the block back to the backend (when every upload from it has retired) and clears the record */
void expert_host_copies_detach(const struct backend_operations *backend, struct expert_host_copies *copies);

/* ---- FP4 / FP8 expert linears of the original weights (the routed part of the reference's linear.h) ---- */
#define LINEAR_SLICE_INSTANCES 5u /* product kernels are stamped for 1, 2, 4, 8, 16 slices; gfx950 holds 1, 2, 4, 8 */
#define LINEAR_MAXIMUM_SLICES 16u
struct linear_kernels_record { /* include/anemone/linear.h:121-132 of the reference, member for member */
    uint32_t activation_quantize;
    uint32_t expert_gate_up[LINEAR_SLICE_INSTANCES];
    uint32_t expert_down[LINEAR_SLICE_INSTANCES];
    uint32_t expert_row_sum;
    uint32_t trunk_linear_quantized[LINEAR_SLICE_INSTANCES]; /* the shared expert's products: 1, 2, 4, 8 slices */
    uint32_t trunk_linear_bfloat16[LINEAR_SLICE_INSTANCES];  /* rows that are not quantized: outside this path, BACKEND_NO_KERNEL */
    uint32_t trunk_hidden;
    uint32_t trunk_linear_quantized_wide[LINEAR_SLICE_INSTANCES]; /* prepared by linear_kernels_prepare too (the reference prepares them apart) */
    uint32_t trunk_linear_bfloat16_wide[LINEAR_SLICE_INSTANCES];  /* BACKEND_NO_KERNEL */
    uint32_t trunk_linear_quantized_interleaved;
    /* extension (no counterpart in the reference, whose expert kernels take E2M1 alone): the same two families
     * for experts of WEIGHT_FORMAT_E4M3_SCALED */
    uint32_t expert_gate_up_e4m3[LINEAR_SLICE_INSTANCES];
    uint32_t expert_down_e4m3[LINEAR_SLICE_INSTANCES];
    /* extension: experts of WEIGHT_FORMAT_E4M3_BLOCK128 and the quantizer of their vectors (128 values a float32 scale) */
    uint32_t expert_gate_up_b128[LINEAR_SLICE_INSTANCES];
    uint32_t expert_down_b128[LINEAR_SLICE_INSTANCES];
    uint32_t activation_quantize_128;
    /* extension: experts stored in gfx950's lane order, WEIGHT_FORMAT_E2M1_GFX950 and WEIGHT_FORMAT_E4M3_GFX950 */
    uint32_t expert_gate_up_gfx950[LINEAR_SLICE_INSTANCES];
    uint32_t expert_down_gfx950[LINEAR_SLICE_INSTANCES];
    uint32_t expert_gate_up_e4m3_gfx950[LINEAR_SLICE_INSTANCES];
    uint32_t expert_down_e4m3_gfx950[LINEAR_SLICE_INSTANCES];
    uint32_t expert_gate_up_b128_gfx950[LINEAR_SLICE_INSTANCES]; /* WEIGHT_FORMAT_E4M3_BLOCK128_GFX950 */
    uint32_t expert_down_b128_gfx950[LINEAR_SLICE_INSTANCES];
};
MUST_CHECK result_status linear_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                                uint32_t arithmetic_class, struct linear_kernels_record *kernels_out);

enum linear_profile_code { LINEAR_PROFILE_PRECISION = 0, LINEAR_PROFILE_SPEED = 1 };
enum linear_family_code {
    LINEAR_FAMILY_EXPERT_GATE_UP = 0,
    LINEAR_FAMILY_EXPERT_DOWN = 1,
    LINEAR_FAMILY_TRUNK_QUANTIZED = 2,
    LINEAR_FAMILY_TRUNK_BFLOAT16 = 3
};
/* the slice count of a product: 1 in the reference order; else gfx950's fixed counts (gate/up 4, down 2), never
 * chosen by row count or timing */
MUST_CHECK result_status linear_default_slice_count(enum linear_profile_code profile, enum linear_order_code order,
                                                    enum linear_family_code family,
                                                    const struct matrix_shape_record *shape,
                                                    uint32_t arithmetic_class, uint32_t *slice_count_out);

struct linear_quantize_description {
    struct linear_range values;    /* read: bfloat16 [row_count][width] */
    struct linear_range codes;     /* written: codes [row_count][width] */
    struct linear_range exponents; /* written: exponents [row_count][width / 32] */
    struct linear_range operands;  /* written: operands [row_count][width] */
    uint32_t width;
    uint32_t row_count;
};
MUST_CHECK result_status linear_quantize_prepare(const struct linear_quantize_description *description,
                                                 uint64_t arena_byte_count,
                                                 const struct linear_kernels_record *kernels,
                                                 struct kernel_launch *launch_out);

/* The same for the vectors of WEIGHT_FORMAT_E4M3_BLOCK128 matrices (no counterpart in the reference): one launch of
 * activation_quantize_128_entry. `exponents` receives the float32 scales [row_count][width / 128] (the same bytes);
 * `operands` is not written and may be empty; width a multiple of 128. */
MUST_CHECK result_status linear_quantize_128_prepare(const struct linear_quantize_description *description,
                                                     uint64_t arena_byte_count,
                                                     const struct linear_kernels_record *kernels,
                                                     struct kernel_launch *launch_out);

enum linear_routed_experts_launch {
    LINEAR_ROUTED_EXPERTS_GATE_UP = 0,  /* expert_gate_up_<S>: jobs and the rows' arrays to hidden */
    LINEAR_ROUTED_EXPERTS_QUANTIZE = 1, /* activation_quantize_entry: hidden of every pair to its arrays */
    LINEAR_ROUTED_EXPERTS_DOWN = 2,     /* expert_down_<S>: jobs and the hidden arrays to pair_output */
    LINEAR_ROUTED_EXPERTS_ROW_SUM = 3,  /* expert_row_sum_entry: pair_output to row_output */
    LINEAR_ROUTED_EXPERTS_LAUNCH_COUNT = 4
};
/* launches_out: LINEAR_ROUTED_EXPERTS_LAUNCH_COUNT launches; weight_format E2M1_SCALED, or (extensions) E4M3_SCALED,
 * E4M3_BLOCK128 (its exponent ranges hold float32 scales of 128 values (the same bytes), its quantizer launch is
 * activation_quantize_128_entry, its shapes are multiples of 128), E2M1_GFX950, E4M3_GFX950 or E4M3_BLOCK128_GFX950 (the
 * outputs of the same matrices stored as E2M1_SCALED, E4M3_SCALED or E4M3_BLOCK128, bit for bit) */
MUST_CHECK result_status linear_routed_experts_prepare(const struct linear_routed_experts_description *description,
                                                       uint64_t arena_byte_count,
                                                       const struct linear_kernels_record *kernels,
                                                       struct kernel_launch *launches_out);

/* ---- the shared expert (include/anemone/linear.h:161-262, 323-367 of the reference): trunk products of quantized
 * rows by WEIGHT_FORMAT_E4M3_SCALED matrices ---- */
/* The form of a trunk launch of more than LINEAR_MAXIMUM_ROWS rows. Every form gives the thin instance's bits.
 * Here: GROUP_BLOCKS the wide instance with a block for each group of 8 rows of each strip, TILE_BLOCKS one block a
 * strip that takes the groups in turn; both INTERLEAVED forms the interleaved instance of one slice (a block a tile of
 * 64 rows by 128 outputs, the card's grouped-GEMM form: what a step of many rows takes). */
enum linear_wide_form {
    LINEAR_WIDE_GROUP_BLOCKS = 0,
    LINEAR_WIDE_TILE_BLOCKS = 1,
    LINEAR_INTERLEAVED_CHUNK_BLOCKS = 2,
    LINEAR_INTERLEAVED_TILE_BLOCKS = 3,
    LINEAR_WIDE_FORM_COUNT = 4
};
struct linear_matrix {
    struct linear_range stored; /* read: exactly the bytes its format stores for its shape */
    struct matrix_shape_record shape;
    enum weight_format_code weight_format;
    uint32_t slice_count;
    enum linear_wide_form wide_form;
    uint32_t reserved_zero;
};
#define LINEAR_TRUNK_MOST_ROWS 16384u /* rows of one trunk launch (the reference: 1,024, a wide step's chunk) */
/* y = W x for quantized rows, of one matrix or of two that read the same rows (gate and up of the shared expert):
 * one launch of trunk_linear_quantized_<S>, of its wide instance or of the interleaved one. Refused: a format other
 * than E4M3_SCALED, a shape it does not store, inputs no multiple of 128, fewer than 32 outputs or no multiple of 16,
 * a slice count no kernel is built for or above inputs / 128, two matrices that differ in input_size, slice_count or
 * wide form, an interleaved form of more than one slice, 0 rows or more than LINEAR_TRUNK_MOST_ROWS, a bad range. */
struct linear_trunk_quantized_description {
    struct linear_matrix matrices[LINEAR_MERGED_MATRICES];
    struct linear_range codes;     /* read: codes [row_count][input_size] */
    struct linear_range exponents; /* read: exponents [row_count][input_size / 32] */
    struct linear_range operands;  /* read: operands [row_count][input_size] */
    struct linear_range outputs[LINEAR_MERGED_MATRICES]; /* written: bf16 [row_count][output_size] */
    uint32_t matrix_count; /* 1 or 2 */
    uint32_t row_count;
};
MUST_CHECK result_status linear_trunk_quantized_prepare(const struct linear_trunk_quantized_description *description,
                                                        uint64_t arena_byte_count, const struct linear_kernels_record *kernels,
                                                        struct kernel_launch *launch_out);

enum linear_shared_expert_launch {
    LINEAR_SHARED_EXPERT_GATE_UP = 0,  /* trunk_linear_quantized, two matrices: to gate_output and up_output */
    LINEAR_SHARED_EXPERT_HIDDEN = 1,   /* trunk_hidden_entry: gate_output and up_output to hidden */
    LINEAR_SHARED_EXPERT_QUANTIZE = 2, /* activation_quantize_entry: hidden to its arrays */
    LINEAR_SHARED_EXPERT_DOWN = 3,     /* trunk_linear_quantized: the hidden arrays to output */
    LINEAR_SHARED_EXPERT_LAUNCH_COUNT = 4
};
struct linear_shared_expert_description {
    struct linear_matrix gate, up, down; /* E4M3_SCALED; gate and up of one shape, slice_count and wide form */
    struct linear_range codes, exponents, operands;                     /* read: the rows' arrays, [row_count][gate.input_size] */
    struct linear_range gate_output, up_output, hidden;                 /* scratch: bf16 [row_count][gate.output_size] each */
    struct linear_range hidden_codes, hidden_exponents, hidden_operands; /* scratch: the hidden vectors' arrays */
    struct linear_range output;                                         /* written: bf16 [row_count][down.output_size] */
    uint32_t row_count;
    float activation_limit;
};
/* launches_out: LINEAR_SHARED_EXPERT_LAUNCH_COUNT launches */
MUST_CHECK result_status linear_shared_expert_prepare(const struct linear_shared_expert_description *description,
                                                      uint64_t arena_byte_count, const struct linear_kernels_record *kernels,
                                                      struct kernel_launch *launches_out);

/* ---- the producer, the join and the shared join (include/anemone/expert_fused.h:37-101 of the reference): the
 * routed experts' phase in fewer launches ---- */
struct expert_fused_kernels {
    uint32_t gate_up_quantize[LINEAR_SLICE_INSTANCES];
    uint32_t shared_join[LINEAR_SLICE_INSTANCES];
    uint32_t join;
    uint32_t gate_up_quantize_e4m3[LINEAR_SLICE_INSTANCES]; /* extension: experts of WEIGHT_FORMAT_E4M3_SCALED */
    uint32_t post;                                          /* extension: hyper_post_entry, the join's second half alone */
};
MUST_CHECK result_status expert_fused_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                                      uint32_t arithmetic_class, struct expert_fused_kernels *kernels_out);
/* One launch of expert_gate_up_quantize_<gate_up_slice_count>: it stands for launches LINEAR_ROUTED_EXPERTS_GATE_UP and
 * _QUANTIZE of linear_routed_experts_prepare and writes what they write, byte for byte. arrivals: uint32
 * [job_count][gate_up_shape.output_size / 32], holding zeros (left so). Refused besides what the routed experts'
 * prepare refuses: more than LINEAR_MAXIMUM_ROWS rows, more than EXPERT_PRODUCER_MOST_PAIRS pairs, an output size
 * that is no multiple of 32, an arrivals range that is too small or shares a byte with another range. */
MUST_CHECK result_status expert_producer_prepare(const struct linear_routed_experts_description *description,
                                                 struct linear_range arrivals, uint64_t arena_byte_count,
                                                 const struct linear_kernels_record *linear_kernels,
                                                 const struct expert_fused_kernels *kernels, struct kernel_launch *launch_out);

/* A layer's FFN join: a row's routed sum (as expert_row_sum_entry), the shared expert's output added to it, and the
 * post of the four residual streams, one launch of expert_join. The reference takes 1 to LINEAR_MAXIMUM_ROWS rows (a
 * thin step, or a slab of a wide one) of its model's width; here 1 to 65535 rows of `width` values, a multiple of
 * HYPER_VALUES_PER_THREAD x HYPER_PIECE_THREADS = 1,024 (0 stands for the reference's 5,120). */
struct expert_join_description {
    struct linear_range pair_output;   /* read: bf16 [row_count * pairs_per_row][width] */
    struct linear_range shared_output; /* read: bf16 [row_count][width] */
    struct linear_range streams;       /* read and written: bf16 [row_count][4][width] */
    struct linear_range post;          /* read: float32 [row_count][4] */
    struct linear_range comb;          /* read: float32 [row_count][4][4] */
    struct linear_range row_sums;      /* written: float32 [row_count][width], or no bytes */
    uint32_t pairs_per_row;
    uint32_t row_count;
    uint32_t width;                    /* extension */
};
MUST_CHECK result_status expert_join_prepare(const struct expert_join_description *description, uint64_t arena_byte_count,
                                             const struct expert_fused_kernels *kernels, struct kernel_launch *launch_out);
/* The post alone (hyper_post_entry with the combine: the sums read from join.row_sums, which must have bytes, the
 * output from join.shared_output): the second of the two launches an expert_join stands for, behind
 * expert_row_sum_entry. kernel: a handle of KERNEL_HYPER_POST. */
MUST_CHECK result_status expert_post_prepare(const struct expert_join_description *join, uint64_t arena_byte_count,
                                             uint32_t kernel, struct kernel_launch *launch_out);

/* The same join behind the shared expert's down, one launch of expert_shared_join_<down.slice_count>: at most
 * LINEAR_MAXIMUM_ROWS rows; down's outputs are the join's width; its output is written to join.shared_output. */
struct expert_shared_join_description {
    struct linear_matrix down;
    struct linear_range codes, exponents, operands; /* read: the hidden vectors' arrays, [row_count][down.input_size] */
    struct expert_join_description join;
};
MUST_CHECK result_status expert_shared_join_prepare(const struct expert_shared_join_description *description,
                                                    uint64_t arena_byte_count, const struct linear_kernels_record *linear_kernels,
                                                    const struct expert_fused_kernels *kernels, struct kernel_launch *launch_out);

/* ---- the wide form of the routed experts: a grouped GEMM over the tiles of a wide select ----
 * The reference prepares its wide products from a description of the routed experts plus the tiles and sorted pairs
 * of the router's wide select (struct expert_relaxed_description, include/anemone/expert_relaxed.h:79-99, for its
 * class-80 order; the kernels of the reference order are source/kernel_wide_linear.cu). Here: the same description,
 * three launches: wide_expert_gate_up_1 (gate with up, hidden step, quantization), wide_expert_down_1,
 * expert_row_sum_entry. Slice counts must be 1 (the only instance built); the outputs are those of the job-table
 * kernels of one slice, bit for bit. */
struct linear_wide_kernels_record {
    uint32_t wide_expert_gate_up; /* of one slice */
    uint32_t wide_expert_down;
    uint32_t wide_expert_gate_up_e4m3; /* extension: experts of WEIGHT_FORMAT_E4M3_SCALED */
    uint32_t wide_expert_down_e4m3;
    uint32_t wide_expert_gate_up_b128; /* extension: experts of WEIGHT_FORMAT_E4M3_BLOCK128 */
    uint32_t wide_expert_down_b128;
};
MUST_CHECK result_status linear_wide_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                                     uint32_t arithmetic_class, struct linear_wide_kernels_record *kernels_out);
enum linear_wide_experts_launch {
    LINEAR_WIDE_EXPERTS_GATE_UP = 0,
    LINEAR_WIDE_EXPERTS_DOWN = 1,
    LINEAR_WIDE_EXPERTS_ROW_SUM = 2,
    LINEAR_WIDE_EXPERTS_LAUNCH_COUNT = 3
};
struct linear_wide_experts_description {
    struct linear_routed_experts_description experts; /* the chain's arrays; jobs is not read (its range may be empty) */
    struct linear_range tiles;                        /* read: struct wide_expert_tile [tile_count] */
    struct linear_range pairs;                        /* read: struct wide_pair [row_count * pairs_per_row] */
    uint32_t tile_count;                              /* grid[1] of the two products */
    uint32_t reserved_zero;
};
MUST_CHECK result_status linear_wide_experts_prepare(const struct linear_wide_experts_description *description,
                                                     uint64_t arena_byte_count, const struct linear_kernels_record *linear_kernels,
                                                     const struct linear_wide_kernels_record *kernels,
                                                     struct kernel_launch *launches_out);

/* The wide form of WEIGHT_FORMAT_E4M3_BLOCK128 experts (no counterpart in the reference): four launches, the gate/up
 * product (which leaves the hidden VALUES where hidden_operands names: the same bytes), activation_quantize_128_entry of
 * them (codes and float32 scales), the down product, the row sum. Refusals as linear_wide_experts_prepare's, which
 * refuses this format as this function refuses the others. */
enum { LINEAR_WIDE_EXPERTS_BLOCK128_LAUNCH_COUNT = 4 };
MUST_CHECK result_status linear_wide_experts_block128_prepare(const struct linear_wide_experts_description *description,
                                                              uint64_t arena_byte_count, const struct linear_kernels_record *linear_kernels,
                                                              const struct linear_wide_kernels_record *kernels,
                                                              struct kernel_launch *launches_out);

/* The wide form of experts stored in gfx950's lane order (WEIGHT_FORMAT_E2M1_GFX950, _E4M3_GFX950, _E4M3_BLOCK128_GFX950; no
 * counterpart in the reference): linear_wide_experts_prepare's description, three launches (E4M3_BLOCK128_GFX950: the four
 * of linear_wide_experts_block128_prepare, LINEAR_WIDE_EXPERTS_BLOCK128_LAUNCH_COUNT) and outputs -- bit for bit those of
 * the same matrices in the reference's lay-out -- by the kernels of kernel_native_linear.hip, whose weights go from
 * memory into the matrix instruction's registers. */
struct linear_native_kernels_record {
    uint32_t native_expert_gate_up; /* E2M1_GFX950, one slice */
    uint32_t native_expert_down;
    uint32_t native_expert_gate_up_e4m3; /* E4M3_GFX950 */
    uint32_t native_expert_down_e4m3;
    uint32_t native_expert_gate_up_b128; /* E4M3_BLOCK128_GFX950 */
    uint32_t native_expert_down_b128;
};
MUST_CHECK result_status linear_native_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                                       uint32_t arithmetic_class, struct linear_native_kernels_record *kernels_out);
MUST_CHECK result_status linear_native_experts_prepare(const struct linear_wide_experts_description *description,
                                                       uint64_t arena_byte_count, const struct linear_kernels_record *linear_kernels,
                                                       const struct linear_native_kernels_record *kernels,
                                                       struct kernel_launch *launches_out);

uint64_t linear_values_byte_count(uint64_t vector_count, uint64_t width);    /* bfloat16 [vector][width] */
uint64_t linear_codes_byte_count(uint64_t vector_count, uint64_t width);     /* E4M3 [vector][width] */
uint64_t linear_exponents_byte_count(uint64_t vector_count, uint64_t width); /* E8M0 [vector][width / 32] */
uint64_t linear_sums_byte_count(uint64_t row_count, uint64_t width);         /* float32 [row][width] */
uint64_t linear_jobs_byte_count(uint64_t job_count);                         /* struct expert_job_record */

#ifdef __cplusplus
}
#endif

/* ---- the launches a block's site front stands for (the step ahead of the routed experts) ----
 * The reference merges a site's mix project, its mix finish, the router's scores, the select and the quantization of
 * the sublayer's input into one launch (include/anemone/site_front.h:2-20, site_front_records.h:10-37), which writes
 * "the same bits: only launches merge". Built here: the launches themselves, each the reference's own entry point --
 * the dense product (include/anemone/dense_linear.h:27-99, source/dense_linear.c) and the site's mix finish and post
 * (include/anemone/hyper_connection.h:25-71, source/hyper_connection.c); the select and the quantizer are router.h's
 * and linear.h's above. */
struct dense_linear_kernels {
    uint32_t products[DENSE_INSTANCES]; /* [form][type][one row, 8]: dense_linear_<type>_<R>, then _narrow */
    uint32_t wide_products[DENSE_TYPE_COUNT]; /* dense_linear_<type>_8_wide: more than 8 rows, 8 outputs a block */
};
MUST_CHECK result_status dense_linear_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                                      struct dense_linear_kernels *kernels_out);

/* include/anemone/dense_linear.h:70-99 of the reference. Refused with STATUS_INVALID_ARGUMENT: a NULL argument, a
 * type outside the enumeration, a flag outside DENSE_FLAGS, an output_size that is no multiple of
 * DENSE_OUTPUTS_PER_BLOCK or an input_size that is no multiple of DENSE_CHUNK_INPUTS, 0 rows, a range that breaks the
 * range rules, more than DENSE_MOST_ROWS rows; with STATUS_UNSUPPORTED: DENSE_STEP_ROWS and DENSE_CONE_ROWS. More than
 * LINEAR_MAXIMUM_ROWS rows: a wide launch, groups of 8 rows on grid[1], every output's bits those of its group's launch. */
struct dense_linear_description {
    struct linear_range weights; /* read: [output_size][input_size] of weight_type, exactly */
    struct linear_range rows;    /* read: bf16 [row_count][input_size] */
    struct linear_range output;  /* written: [row_count][output_size] of output_type */
    struct linear_range step;    /* no bytes */
    uint32_t output_size;
    uint32_t input_size;
    uint32_t row_count;
    uint32_t weight_type; /* enum dense_type_code */
    uint32_t output_type;
    uint32_t flags;       /* DENSE_ROW_SCALE or 0 */
    float output_scale;   /* 1 for none */
    float epsilon;        /* of DENSE_ROW_SCALE */
    uint32_t cone_layer;  /* 0 */
};
MUST_CHECK result_status dense_linear_prepare(const struct dense_linear_description *description, uint64_t arena_byte_count,
                                              const struct dense_linear_kernels *kernels, struct kernel_launch *launch_out);

/* include/anemone/hyper_connection.h:25-38: the handles of kernel_hyper_connection; the final collapse, the embedding
 * and the draft's two are not built and stay BACKEND_NO_KERNEL. */
struct hyper_kernels_record {
    uint32_t mix_finish;
    uint32_t final_collapse;
    uint32_t post;
    uint32_t embed;
    uint32_t draft_inputs;
    uint32_t final_kept;
};
MUST_CHECK result_status hyper_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                               struct hyper_kernels_record *kernels_out);

/* A site of a block (include/anemone/hyper_connection.h:40-71): its mix finish, between its mix project and its
 * sublayer, and its post after the sublayer, with the combine where routed_sums has bytes (the FFN site). 1 to
 * 65535 rows (a thin step's, or a prefill chunk's: a row's bits are its own). */
enum hyper_site_launch { HYPER_SITE_MIX_FINISH = 0, HYPER_SITE_POST = 1, HYPER_SITE_LAUNCH_COUNT = 2 };
struct hyper_site_description {
    struct linear_range streams;     /* read and written: bf16 [row_count][4][width] */
    struct linear_range carried_pre; /* read and written: float32 [row_count][4] */
    struct linear_range mixes;       /* read: float32 [row_count][24] */
    struct linear_range scale;       /* read: float32 [3], exactly */
    struct linear_range base;        /* read: float32 [24], exactly */
    struct linear_range norm_weight; /* read: bf16 [width], exactly */
    struct linear_range post;        /* written, then read: float32 [row_count][4] */
    struct linear_range comb;        /* written, then read: float32 [row_count][4][4] */
    struct linear_range hidden;      /* written: bf16 [row_count][width], the sublayer's input */
    struct linear_range output;      /* read: bf16 [row_count][width], the sublayer's output or the shared expert's */
    struct linear_range routed_sums; /* read: float32 [row_count][width], or no bytes */
    uint32_t row_count;
    uint32_t reserved_zero;          /* extension: the streams' width, a multiple of 1,024 up to 8,192; 0 stands for 5,120 */
};
MUST_CHECK result_status hyper_site_prepare(const struct hyper_site_description *description, uint64_t arena_byte_count,
                                            const struct hyper_kernels_record *kernels, struct kernel_launch *launches_out);

/* ---- load-time EXL3 slices (include/anemone/exl3_layout.h:15-103, source/exl3_layout.c of the reference) ----
 * A stored EXL3 matrix is [input / 16][output / 16][16 K] uint16 of codes, then suh[input], svh[output]. A slice keeps
 * whole transforms of 128 channels on either side, so a sliced matrix is a stored EXL3 matrix of the slice's shape: its
 * codes the code rows of the input range cut to the output range, its suh and svh the ranges' own. Nothing is decoded
 * and no arithmetic touches a weight: the kernels of this library give, for a slice of outputs with the whole of the
 * inputs, the bits they give for those outputs of the whole matrix (tested on the card), which is what lets a card
 * take a share of a layer's columns. Host-only code; no device or step-loop dependency. */
#define BB_EXL3_TP_RANKS 4u
struct bb_exl3_matrix_slice {
    uint32_t input_size, output_size;   /* of the whole matrix */
    uint32_t input_begin, input_count;  /* whole transforms of 128 */
    uint32_t output_begin, output_count;
    uint32_t bits_per_weight;           /* a stored width this build decodes */
    uint32_t reserved_zero;
};
struct bb_exl3_slice_sizes {
    uint64_t source_bytes; /* of the whole matrix as stored */
    uint64_t packed_bytes; /* of the slice as stored */
};
/* STATUS_INVALID_ARGUMENT (sizes_out unchanged) for a NULL argument, a reserved field that is not zero, a count of
 * zero, a size, origin or count that is no multiple of 128, a range past its dimension, a width this build has no
 * kernels for. */
MUST_CHECK result_status bb_exl3_matrix_slice_prepare(const struct bb_exl3_matrix_slice *slice, struct bb_exl3_slice_sizes *sizes_out);
/* The lossless copy at load. The source holds the whole matrix (source_bytes at least its stored bytes), the
 * destination at least the slice's; the two may not overlap. Refused before a byte is written. */
MUST_CHECK result_status bb_exl3_matrix_slice_copy(const struct bb_exl3_matrix_slice *slice, const void *source, size_t source_bytes,
                                                   void *destination, size_t destination_bytes);

enum bb_exl3_product_order { BB_EXL3_REFERENCE_ORDER = 0, BB_EXL3_EIGHT_PART_ORDER = 1 };
/* What one of rank_count cards (1 or BB_EXL3_TP_RANKS) takes of an expert: gate and up its share of the intermediate
 * outputs with all the inputs, down its share of the outer outputs with all the intermediate inputs: every product
 * keeps its whole K dimension, so its K slices and their order are the whole matrix's. Metadata only: nothing here
 * allocates, launches or moves data between cards. */
struct bb_exl3_output_shard_plan {
    struct bb_exl3_matrix_slice gate_up;
    struct bb_exl3_matrix_slice down;
    uint32_t rank_count;
    uint32_t rank;
    uint32_t product_slices;
    enum bb_exl3_product_order order;
};
MUST_CHECK result_status bb_exl3_output_shard_prepare(uint32_t outer_size, uint32_t inner_size, uint32_t bits_per_weight, uint32_t rank_count,
                                                      uint32_t rank, enum bb_exl3_product_order order,
                                                      struct bb_exl3_output_shard_plan *plan_out);

#endif
