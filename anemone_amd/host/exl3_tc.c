/*
 * exl3_tc.c -- load-time preparation of the fused EXL3 decode of one layer's routed experts (1 to 64 rows): five
 * launches from the router's job table. Entry points follow the reference's source/exl3_tc.c:120-268 and
 * include/anemone/exl3_tc.h:22-43; hidden size, picks a row and per-matrix widths are members of the record.
 *
 *   launch      kernel              grid                                            block
 *   operands    exl3_tc_operands    (hidden / 128, job_capacity, 2)                 64
 *   gate/up     exl3_tc_products    (intermediate / 64, job_capacity, 2 S_gu / 4)   256   pass 0
 *   activate    exl3_tc_activate    (intermediate / 128, job_capacity, 1)           64
 *   down        exl3_tc_products    (hidden / 64, job_capacity, S_d / 4)            256   pass 1
 *   combine     exl3_tc_combine     (hidden / 128, row_count, 1)                    512   a wavefront a slot of the row
 * S_gu = EXL3_TC_GATE_UP_SLICES and S_d = EXL3_TC_DOWN_SLICES K slices; every slice is a whole number of steps of four
 * K tiles (64 inputs): slice s takes the steps [steps s / S, steps (s + 1) / S). Hidden and intermediate: multiples of 128.
 */
#include <math.h>
#include <string.h>

#include "prepare_common.h"

#define WAVE_THREADS 64u
#define PRODUCT_THREADS 256u
#define PRODUCT_WAVES 4u
#define MOST_GRID_ROWS 65535u

/* a block's four wavefronts take four items: of one strip (its matrices x slices a multiple of four: z blocks a strip)
 * or of adjacent strips (a divisor of four: that many strips a block) */
enum { GATE_UP_ITEMS = 2u * EXL3_TC_GATE_UP_SLICES, DOWN_ITEMS = EXL3_TC_DOWN_SLICES };
_Static_assert((GATE_UP_ITEMS % PRODUCT_WAVES == 0 || PRODUCT_WAVES % GATE_UP_ITEMS == 0) &&
               (DOWN_ITEMS % PRODUCT_WAVES == 0 || PRODUCT_WAVES % DOWN_ITEMS == 0), "a block's four wavefronts take four whole items");
#define GATE_UP_STRIPS (GATE_UP_ITEMS >= PRODUCT_WAVES ? 1u : PRODUCT_WAVES / GATE_UP_ITEMS)
#define DOWN_STRIPS (DOWN_ITEMS >= PRODUCT_WAVES ? 1u : PRODUCT_WAVES / DOWN_ITEMS)

/* why the fused decode's launches do not take a layer of these sizes (the prefill launches take every layer they take,
 * and an intermediate size up to twice the hidden); NULL when they do */
const char *exl3_tc_geometry_refusal(uint32_t hidden, uint32_t intermediate)
{
    if (hidden == 0 || intermediate == 0 || intermediate % EXL3_TRANSFORM != 0 || hidden % EXL3_TRANSFORM != 0) {
        return "the sizes are multiples of 128";
    }
    if (intermediate > hidden) {
        return "the intermediate size is at most the hidden size";
    }
    if (intermediate % (EXL3_TC_STRIP_OUTPUTS * GATE_UP_STRIPS) != 0 || hidden % (EXL3_TC_STRIP_OUTPUTS * DOWN_STRIPS) != 0) {
        return "the sizes are whole numbers of the products' blocks";
    }
    return NULL;
}

/* detached_workspace: the workspace is not a range of the arena (exl3_tc_run_static names it by an offset of its own) */
static result_status tc_prepare(const struct exl3_tc_record *record, uint64_t arena_byte_count,
                                const struct backend_operations *backend, struct device_card *card,
                                struct kernel_launch launches_out[EXL3_TC_LAUNCHES], bool detached_workspace)
{
    static const char what[] = "EXL3 fused decode";
    if (record == NULL || backend == NULL || backend->kernel_prepare == NULL || card == NULL || launches_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t hidden = record->hidden != 0 ? record->hidden : EXL3_TC_DEFAULT_HIDDEN;
    const uint32_t picks = record->pairs_per_row != 0 ? record->pairs_per_row : EXL3_TC_DEFAULT_PAIRS_PER_ROW;
    const uint32_t I = record->intermediate;
    if (record->row_count == 0 || record->row_count > EXL3_TC_MOST_ROWS || record->job_capacity == 0 ||
        record->job_capacity > MOST_GRID_ROWS || record->pass != 0 || picks > ROUTER_MOST_PICKS ||
        !(record->activation_limit >= 0.0f) || !isfinite(record->activation_limit)) {
        REFUSE("%s: 1 to %u rows, 1 to %u jobs, pass 0, an activation limit of zero (none) or above", what,
               EXL3_TC_MOST_ROWS, MOST_GRID_ROWS);
        return STATUS_INVALID_ARGUMENT;
    }
    if (record->shared_sum > 1u) {
        REFUSE("%s: shared_sum %u: 0 (the sums to output_offset) or 1 (added to the shared expert's rows in place)", what, record->shared_sum);
        return STATUS_INVALID_ARGUMENT;
    }
    if (record->rotation != 0) {
        REFUSE("%s: expert rotation is a tensor-parallel form this library does not build", what);
        return STATUS_UNSUPPORTED;
    }
    if (I == 0 || I % EXL3_TRANSFORM != 0 || hidden % EXL3_TRANSFORM != 0 || I > hidden) {
        REFUSE("%s: hidden %u and intermediate %u: multiples of 128, the intermediate size at most the hidden", what, hidden, I);
        return STATUS_UNSUPPORTED;
    }
    const bool mixed = record->widths_offset != 0;
    if (!mixed && (record->bits_x2 != 4u && record->bits_x2 != 5u && record->bits_x2 != 6u && record->bits_x2 != 8u)) {
        REFUSE("%s: bits_x2 %u: this build decodes 4, 5, 6 and 8", what, record->bits_x2);
        return exl3_width_name(record->bits_x2) == NULL && (record->bits_x2 == 0 || record->bits_x2 > 16u)
                   ? STATUS_INVALID_ARGUMENT
                   : STATUS_UNSUPPORTED;
    }
    const uint64_t pairs = (uint64_t)record->row_count * picks;
    const uint64_t workspace = exl3_tc_workspace_bytes(pairs, hidden, I);
    /* the table of per-matrix widths, where one is named: uint32 an expert, expert_count of them, inside the arena and
     * clear of what the launches write; the kernels read no entry beyond it */
    if (record->reserved_zero != 0 || (mixed ? record->expert_count == 0 : record->expert_count != 0)) {
        REFUSE("%s: a widths table needs its expert count (%u), a record without one names none, and the reserved word is zero", what,
               record->expert_count);
        return STATUS_INVALID_ARGUMENT;
    }
    struct checked_range ranges[6] = {
        {"the jobs", {record->jobs_offset, (uint64_t)record->job_capacity * sizeof(struct expert_job_record)},
         (uint64_t)record->job_capacity * sizeof(struct expert_job_record), false},
        {"the rows", {record->hidden_offset, (uint64_t)record->row_count * hidden * 2u}, (uint64_t)record->row_count * hidden * 2u, false},
        {"the output", {record->output_offset, (uint64_t)record->row_count * hidden * 4u}, (uint64_t)record->row_count * hidden * 4u, false},
        {"the workspace", {record->workspace_offset, workspace}, workspace, false},
        {"the shared expert's rows", {record->shared_offset, (uint64_t)record->row_count * hidden * 2u}, (uint64_t)record->row_count * hidden * 2u, false},
    };
    uint32_t range_count = 5u;
    if (record->shared_sum == 0u) {
        range_count = 4u;
    }
    if (detached_workspace) { /* the ranges of the arena alone */
        ranges[3] = ranges[4];
        range_count -= 1u;
    }
    if (mixed) {
        const uint64_t table_bytes = (uint64_t)record->expert_count * 4u;
        ranges[range_count++] = (struct checked_range){"the widths", {record->widths_offset, table_bytes}, table_bytes, false};
    }
    if (!ranges_are_valid(what, ranges, range_count, arena_byte_count) || record->workspace_offset % 256u != 0 ||
        (mixed && record->widths_offset % LINEAR_OFFSET_ALIGNMENT_BYTES != 0)) {
        if (record->workspace_offset % 256u != 0) {
            REFUSE("%s: the workspace begins off a multiple of 256", what);
        }
        return STATUS_INVALID_ARGUMENT;
    }
    static const char *const names[EXL3_TC_LAUNCHES] = {"exl3_tc_operands", "exl3_tc_products", "exl3_tc_activate",
                                                        "exl3_tc_products", "exl3_tc_combine"};
    const uint32_t gate_up_strips = GATE_UP_STRIPS, down_strips = DOWN_STRIPS;
    if (I % (EXL3_TC_STRIP_OUTPUTS * gate_up_strips) != 0 || hidden % (EXL3_TC_STRIP_OUTPUTS * down_strips) != 0) {
        REFUSE("%s: sizes that are no whole number of the products' blocks (%u and %u outputs)", what,
               EXL3_TC_STRIP_OUTPUTS * gate_up_strips, EXL3_TC_STRIP_OUTPUTS * down_strips);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t grid_x[EXL3_TC_LAUNCHES] = {hidden / 128u, I / (EXL3_TC_STRIP_OUTPUTS * gate_up_strips), I / 128u,
                                               hidden / (EXL3_TC_STRIP_OUTPUTS * down_strips), hidden / 128u};
    const uint32_t grid_y[EXL3_TC_LAUNCHES] = {record->job_capacity, record->job_capacity, record->job_capacity,
                                               record->job_capacity, record->row_count};
    const uint32_t grid_z[EXL3_TC_LAUNCHES] = {2u, (GATE_UP_ITEMS + PRODUCT_WAVES - 1u) / PRODUCT_WAVES, 1u,
                                               (DOWN_ITEMS + PRODUCT_WAVES - 1u) / PRODUCT_WAVES, 1u};
    const uint32_t threads[EXL3_TC_LAUNCHES] = {WAVE_THREADS, PRODUCT_THREADS, WAVE_THREADS, PRODUCT_THREADS, WAVE_THREADS * ROUTER_MOST_PICKS};
    struct kernel_launch launches[EXL3_TC_LAUNCHES];
    for (uint32_t index = 0; index < EXL3_TC_LAUNCHES; index++) {
        uint32_t kernel = BACKEND_NO_KERNEL;
        const result_status prepared = backend->kernel_prepare(card, EXL3_TC_KERNEL_FILE, names[index], sizeof *record, &kernel);
        if (prepared != STATUS_OK) {
            return prepared;
        }
        if (kernel == BACKEND_NO_KERNEL) {
            return STATUS_UNSUPPORTED;
        }
        struct exl3_tc_record stamped = *record;
        stamped.pass = index == 3u ? 1u : 0u;
        launch_fill(&launches[index], kernel, grid_x[index], grid_y[index], grid_z[index], threads[index], 0, &stamped,
                    sizeof stamped);
    }
    memcpy(launches_out, launches, sizeof launches);
    return STATUS_OK;
}

result_status exl3_tc_prepare(const struct exl3_tc_record *record, uint64_t arena_byte_count,
                              const struct backend_operations *backend, struct device_card *card,
                              struct kernel_launch launches_out[EXL3_TC_LAUNCHES])
{
    return tc_prepare(record, arena_byte_count, backend, card, launches_out, false);
}

result_status exl3_tc_prepare_short(const struct exl3_tc_record *record, uint64_t arena_byte_count,
                                    const struct backend_operations *backend, struct device_card *card,
                                    struct kernel_launch launches_out[EXL3_TC_LAUNCHES])
{
    return tc_prepare(record, arena_byte_count, backend, card, launches_out, false);
}

result_status exl3_tc_prepare_paired(const struct exl3_tc_record *record, uint64_t arena_byte_count,
                                     const struct backend_operations *backend, struct device_card *card,
                                     struct kernel_launch launches_out[EXL3_TC_LAUNCHES])
{
    return tc_prepare(record, arena_byte_count, backend, card, launches_out, false);
}

/* The launches of exl3_tc_prepare for a workspace that is no range of the arena: every other range is checked against
 * the arena as there, the workspace's offset only for its alignment. For exl3_tc_run_static. */
result_status exl3_tc_prepare_detached(const struct exl3_tc_record *record, uint64_t arena_byte_count,
                                       const struct backend_operations *backend, struct device_card *card,
                                       struct kernel_launch launches_out[EXL3_TC_LAUNCHES])
{
    return tc_prepare(record, arena_byte_count, backend, card, launches_out, true);
}

/*
 * The prefill form (include/anemone/exl3_tc.h:40-59 of the reference): seven launches of one record.
 *
 *   launch      kernel              grid                                             block
 *   count       exl3_tcp_count      (ceil(rows / 384), 1, 1)                         512
 *   place       exl3_tcp_place      (ceil(rows / 384), 1, 1)                         512
 *   operands    exl3_tcp_operands   (hidden / 128, chunk capacity, 2)                64
 *   gate/up     exl3_tcp_gemm       (ceil(intermediate / 256), chunk capacity, 2)    256   pass EXL3_TCP_GATE_AND_UP
 *   activate    exl3_tcp_activate   (intermediate / 128, chunk capacity, 1)          64
 *   down        exl3_tcp_gemm       (ceil(hidden / 256), chunk capacity, 1)          256   pass EXL3_TCP_DOWN
 *   combine     exl3_tcp_combine    (hidden / 128, rows, 1)                          64
 * chunk capacity = pairs / EXL3_TCP_CHUNK_PAIRS + experts: an expert's pairs cut in chunks of EXL3_TCP_CHUNK_PAIRS (160), the
 * last ragged.
 */
static result_status tcp_prepare(const struct exl3_tcp_record *record, uint64_t arena_byte_count,
                                 const struct backend_operations *backend, struct device_card *card,
                                 struct kernel_launch launches_out[EXL3_TCP_MOST_LAUNCHES], uint32_t *launch_count_out)
{
    static const char what[] = "EXL3 prefill";
    if (record == NULL || backend == NULL || backend->kernel_prepare == NULL || card == NULL || launches_out == NULL ||
        launch_count_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t H = record->hidden, I = record->intermediate, P = record->pairs_per_row, E = record->expert_count;
    if (record->row_count == 0 || record->row_count > EXL3_TCP_MOST_ROWS || record->pass != 0 || record->reserved_zero != 0 ||
        P == 0 || P > ROUTER_MOST_PICKS || E == 0 || E > ROUTER_MOST_EXPERTS || !(record->activation_limit >= 0.0f) ||
        !isfinite(record->activation_limit)) {
        REFUSE("%s: 1 to %u rows of 1 to %u pairs, 1 to %u experts, pass 0, an activation limit of zero (none) or above", what,
               EXL3_TCP_MOST_ROWS, ROUTER_MOST_PICKS, ROUTER_MOST_EXPERTS);
        return STATUS_INVALID_ARGUMENT;
    }
    if (record->rotation != 0 || record->half_rows != 0 || record->part != 0 || record->cone_layer != 0 || record->two_blocks != 0) {
        REFUSE("%s: rotation, halves of rows, cone layers and the two-blocks forms are forms this library does not build", what);
        return STATUS_UNSUPPORTED;
    }
    if (H == 0 || I == 0 || I % EXL3_TRANSFORM != 0 || H % EXL3_TRANSFORM != 0 || I > 2u * H) {
        /* the activation writes the down operands [pairs][intermediate] over the gate and up operands [2][pairs][hidden] */
        REFUSE("%s: hidden %u and intermediate %u: multiples of 128, the intermediate size at most twice the hidden", what, H, I);
        return STATUS_UNSUPPORTED;
    }
    const bool mixed = record->widths_offset != 0;
    if (!mixed && (record->bits_x2 != 4u && record->bits_x2 != 5u && record->bits_x2 != 6u && record->bits_x2 != 8u)) {
        REFUSE("%s: bits_x2 %u: this build decodes 4, 5, 6 and 8", what, record->bits_x2);
        return exl3_width_name(record->bits_x2) == NULL && (record->bits_x2 == 0 || record->bits_x2 > 16u)
                   ? STATUS_INVALID_ARGUMENT
                   : STATUS_UNSUPPORTED;
    }
    const uint64_t rows = record->row_count, pairs = rows * P;
    const struct exl3_tcp_layout layout = exl3_tcp_layout_of(rows, P, E, H, I);
    if (layout.chunk_capacity > MOST_GRID_ROWS) {
        REFUSE("%s: %u chunks of pairs are more than a grid holds", what, layout.chunk_capacity);
        return STATUS_INVALID_ARGUMENT;
    }
    const struct checked_range ranges[] = {
        {"the picks", {record->picks_offset, pairs * sizeof(struct router_pick)}, pairs * sizeof(struct router_pick), false},
        {"the expert offsets", {record->expert_offsets_offset, (uint64_t)E * MODEL_EXPERT_MATRICES * 8u},
         (uint64_t)E * MODEL_EXPERT_MATRICES * 8u, false},
        {"the rows", {record->hidden_offset, rows * H * 2u}, rows * H * 2u, false},
        {"the workspace", {record->workspace_offset, layout.total}, layout.total, false},
        {"the output", {record->output_offset, rows * H * 4u}, rows * H * 4u, false},
        {"the widths", {record->widths_offset, (uint64_t)E * 4u}, (uint64_t)E * 4u, false}, /* where a table is named */
    };
    if (!ranges_are_valid(what, ranges, mixed ? 6u : 5u, arena_byte_count) || record->workspace_offset % 256u != 0 ||
        (mixed && record->widths_offset % LINEAR_OFFSET_ALIGNMENT_BYTES != 0)) {
        if (record->workspace_offset % 256u != 0) {
            REFUSE("%s: the workspace begins off a multiple of 256", what);
        }
        return STATUS_INVALID_ARGUMENT;
    }
    static const char *const names[EXL3_TCP_LAUNCHES] = {"exl3_tcp_count",    "exl3_tcp_place", "exl3_tcp_operands", "exl3_tcp_gemm",
                                                         "exl3_tcp_activate", "exl3_tcp_gemm",  "exl3_tcp_combine"};
    const uint32_t blocks = (uint32_t)((rows + ROUTER_SORT_ROWS - 1u) / ROUTER_SORT_ROWS), capacity = layout.chunk_capacity;
    /* an element-wise launch's wavefront takes four blocks of 128 channels */
    const uint32_t grid_x[EXL3_TCP_LAUNCHES] = {blocks, blocks, (H + 511u) / 512u, (I + EXL3_TCP_BLOCK_OUTPUTS - 1u) / EXL3_TCP_BLOCK_OUTPUTS,
                                                (I + 511u) / 512u, (H + EXL3_TCP_BLOCK_OUTPUTS - 1u) / EXL3_TCP_BLOCK_OUTPUTS, (H + 511u) / 512u};
    const uint32_t grid_y[EXL3_TCP_LAUNCHES] = {1u, 1u, capacity, capacity, capacity, capacity, record->row_count};
    const uint32_t grid_z[EXL3_TCP_LAUNCHES] = {1u, 1u, EXL3_TCP_COLUMN_PARTS, 2u, EXL3_TCP_COLUMN_PARTS, 1u, 1u};
    const uint32_t threads[EXL3_TCP_LAUNCHES] = {512u, 512u, WAVE_THREADS, PRODUCT_THREADS, WAVE_THREADS, PRODUCT_THREADS, WAVE_THREADS};
    struct kernel_launch launches[EXL3_TCP_LAUNCHES];
    for (uint32_t index = 0; index < EXL3_TCP_LAUNCHES; index++) {
        uint32_t kernel = BACKEND_NO_KERNEL;
        const result_status prepared = backend->kernel_prepare(card, EXL3_TCP_KERNEL_FILE, names[index], sizeof *record, &kernel);
        if (prepared != STATUS_OK) {
            return prepared;
        }
        if (kernel == BACKEND_NO_KERNEL) {
            return STATUS_UNSUPPORTED;
        }
        struct exl3_tcp_record stamped = *record;
        stamped.pass = index == EXL3_TCP_DOWN_LAUNCH ? EXL3_TCP_DOWN : EXL3_TCP_GATE_AND_UP;
        launch_fill(&launches[index], kernel, grid_x[index], grid_y[index], grid_z[index], threads[index], 0, &stamped, sizeof stamped);
    }
    memcpy(launches_out, launches, sizeof launches);
    *launch_count_out = EXL3_TCP_LAUNCHES;
    return STATUS_OK;
}

result_status exl3_tcp_prepare(const struct exl3_tcp_record *record, uint64_t arena_byte_count,
                               const struct backend_operations *backend, struct device_card *card,
                               struct kernel_launch launches_out[EXL3_TCP_MOST_LAUNCHES], uint32_t *launch_count_out)
{
    return tcp_prepare(record, arena_byte_count, backend, card, launches_out, launch_count_out);
}

/* the reference's _base and _hybrid forms pick between two GEMM forms of its 640-column geometry that give the same
 * bits; here there is one form */
result_status exl3_tcp_prepare_base(const struct exl3_tcp_record *record, uint64_t arena_byte_count,
                                    const struct backend_operations *backend, struct device_card *card,
                                    struct kernel_launch launches_out[EXL3_TCP_MOST_LAUNCHES], uint32_t *launch_count_out)
{
    return tcp_prepare(record, arena_byte_count, backend, card, launches_out, launch_count_out);
}

result_status exl3_tcp_prepare_hybrid(const struct exl3_tcp_record *record, uint64_t arena_byte_count,
                                      const struct backend_operations *backend, struct device_card *card,
                                      struct kernel_launch launches_out[EXL3_TCP_MOST_LAUNCHES], uint32_t *launch_count_out)
{
    return tcp_prepare(record, arena_byte_count, backend, card, launches_out, launch_count_out);
}
