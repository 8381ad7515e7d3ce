/*
 * router.c -- load-time preparation of the router's launches: the score projection, the select (at most eight
 * rows, whose job table the routed experts read) and the wide select. Entry points and refusal rules follow the
 * reference's source/router.c:41-385 and include/anemone/router.h; the expert count, picks a row, affinity and
 * route scale are members of the description instead of one model's constants, and an EXL3 layer may name a
 * per-matrix widths table.
 *
 *   launch        kernel                grid                        block
 *   projection    router_projection     (ceil(E / 8), ceil(rows / 4), 1)   128   eight experts and four rows a block
 *                 router_projection_tiles (E / 16, ceil(rows / 64), 1)     256   257 rows and more of a width in whole 128, E in whole 16:
 *                                                                                16 experts by 64 rows a block
 *   select        router_select_entry   (1, 1, 1)                   512   a wavefront a row
 *   wide select   router_wide_select    (ceil(rows / 8), 1, 1)      512   a wavefront a row
 *   wide count    router_wide_count     (ceil(rows / 384), 1, 1)    512   a thread an expert
 *   wide place    router_wide_place     (ceil(rows / 384), 1, 1)    512   a thread an expert; block 0 the runs and tiles
 *   wide jobs     router_wide_jobs      (1, 1, 1)                   512   a thread a job
 *   wide small    router_wide_small     (1, 1, 1)                   512   count, place and jobs of at most 384 rows
 */
#include <inttypes.h>
#include <string.h>

#include "prepare_common.h"

#define SELECT_THREADS (LINEAR_MAXIMUM_ROWS * 64u)
#define WIDE_SORT_THREADS 512u
#define PROJECTION_THREADS 128u
#define PROJECTION_OUTPUTS 8u /* experts a block */
#define PROJECTION_ROWS 4u    /* rows a block takes at once */
#define PROJECTION_BY_ROW_MOST_BLOCKS 1024u

result_status router_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                     struct router_kernels_record *kernels_out)
{
    static const struct {
        const char *function;
        uint32_t record_bytes;
        uint32_t required;
    } names[] = {
        {KERNEL_ROUTER_SELECT, sizeof(struct router_select_arguments), 1},
        {KERNEL_ROUTER_WIDE_SELECT, sizeof(struct router_wide_arguments), 0},
        {KERNEL_ROUTER_WIDE_COUNT, sizeof(struct router_wide_arguments), 0},
        {KERNEL_ROUTER_WIDE_PLACE, sizeof(struct router_wide_arguments), 0},
        {KERNEL_ROUTER_WIDE_JOBS, sizeof(struct router_wide_arguments), 0},
        {KERNEL_ROUTER_WIDE_SMALL, sizeof(struct router_wide_arguments), 0},
    };
    if (backend == NULL || backend->kernel_prepare == NULL || card == NULL || kernels_out == NULL) {
        REFUSE("the kernels of the router: a missing argument");
        return STATUS_INVALID_ARGUMENT;
    }
    uint32_t handles[8];
    for (uint32_t i = 0; i < 8u; i++) {
        handles[i] = BACKEND_NO_KERNEL;
    }
    for (uint32_t i = 0; i < sizeof names / sizeof names[0]; i++) {
        const result_status prepared =
            backend->kernel_prepare(card, KERNEL_FILE_ROUTER, names[i].function, names[i].record_bytes, &handles[i]);
        if (prepared != STATUS_OK && names[i].required) {
            REFUSE("the kernels of the router: %s is not prepared: %s", names[i].function, status_text(prepared));
            return prepared;
        }
        if (prepared != STATUS_OK) {
            handles[i] = BACKEND_NO_KERNEL; /* an entry this build does not hold yet: its prepare refuses */
        }
    }
    const result_status projected = backend->kernel_prepare(card, KERNEL_FILE_ROUTER, KERNEL_ROUTER_PROJECTION,
                                                            sizeof(struct router_projection_arguments), &handles[7]);
    if (projected != STATUS_OK) {
        return projected;
    }
    uint32_t tiles = BACKEND_NO_KERNEL;
    if (backend->kernel_prepare(card, KERNEL_FILE_ROUTER, KERNEL_ROUTER_PROJECTION_TILES, sizeof(struct router_projection_arguments),
                                &tiles) != STATUS_OK) {
        tiles = BACKEND_NO_KERNEL; /* every row count then takes router_projection */
    }
    memcpy(kernels_out, handles, sizeof handles);
    kernels_out->projection_tiles = tiles;
    return STATUS_OK;
}

/* bytes of the gate/up and of the down matrix of expert e, by the format and, for EXL3, by its widths */
static bool expert_bytes(enum weight_format_code format, const struct matrix_shape_record *gate_up,
                         const struct matrix_shape_record *down, const uint32_t *widths, uint32_t expert,
                         uint64_t bytes_out[MODEL_EXPERT_MATRICES])
{
    const struct weight_format_operations *operations = weight_format_operations_of(format);
    if (operations == NULL) {
        return false;
    }
    for (uint32_t matrix = 0; matrix < MODEL_EXPERT_MATRICES; matrix++) {
        struct matrix_shape_record shape = matrix == 2u ? *down : *gate_up;
        if (format == WEIGHT_FORMAT_EXL3) {
            /* the stored shape of an EXL3 matrix names outputs and inputs as the others do */
            if (widths != NULL) {
                shape.bits_per_weight = exl3_width_of(widths[expert], matrix);
            }
        }
        if (operations->stored_byte_count(&shape, &bytes_out[matrix]) != STATUS_OK) {
            return false;
        }
    }
    return true;
}

static bool table_is_valid(const char *what, enum weight_format_code format,
                           const struct matrix_shape_record *gate_up, const struct matrix_shape_record *down,
                           const uint64_t *offsets, const uint32_t *widths, uint32_t expert_count,
                           const struct linear_range *weights, uint64_t *least_gate_up_out, uint64_t *least_down_out)
{
    uint64_t least_gate_up = UINT64_MAX, least_down = UINT64_MAX;
    const uint64_t end = weights->byte_offset + weights->byte_count;
    for (uint32_t expert = 0; expert < expert_count; expert++) {
        uint64_t bytes[MODEL_EXPERT_MATRICES];
        if (!expert_bytes(format, gate_up, down, widths, expert, bytes)) {
            REFUSE("%s: expert %u has a matrix its format does not store in this shape", what, expert);
            return false;
        }
        for (uint32_t matrix = 0; matrix < MODEL_EXPERT_MATRICES; matrix++) {
            const uint64_t at = offsets[expert * MODEL_EXPERT_MATRICES + matrix];
            if (at % LINEAR_OFFSET_ALIGNMENT_BYTES != 0 || at < weights->byte_offset || at > end || bytes[matrix] > end - at) {
                REFUSE("%s: entry %u of the offsets table, byte %" PRIu64 ", is no multiple of %u whose matrix lies "
                       "wholly inside the experts' range", what, expert * MODEL_EXPERT_MATRICES + matrix, at,
                       LINEAR_OFFSET_ALIGNMENT_BYTES);
                return false;
            }
        }
        least_gate_up = bytes[0] < least_gate_up ? bytes[0] : least_gate_up;
        least_gate_up = bytes[1] < least_gate_up ? bytes[1] : least_gate_up;
        least_down = bytes[2] < least_down ? bytes[2] : least_down;
    }
    *least_gate_up_out = least_gate_up;
    *least_down_out = least_down;
    return true;
}

static bool shape_counts_are_valid(const char *what, uint32_t expert_count, uint32_t pick_count,
                                   uint32_t affinity_kind, enum linear_order_code order)
{
    if (expert_count == 0 || expert_count > ROUTER_MOST_EXPERTS || expert_count % 64u != 0 || pick_count == 0 ||
        pick_count > ROUTER_MOST_PICKS || pick_count > expert_count || affinity_kind > ROUTER_AFFINITY_SIGMOID ||
        (order != LINEAR_ORDER_FIXED && order != LINEAR_ORDER_REFERENCE) ||
        (order == LINEAR_ORDER_REFERENCE && pick_count != 6u)) {
        REFUSE("%s: %u experts of %u picks a row, affinity %u, order %u: experts a multiple of 64 up to %u, picks up to "
               "%u, the reference order for six picks alone", what, expert_count, pick_count, affinity_kind,
               (uint32_t)order, ROUTER_MOST_EXPERTS, ROUTER_MOST_PICKS);
        return false;
    }
    return true;
}

result_status router_select_prepare(const struct router_description *description, uint64_t arena_byte_count,
                                    const struct router_kernels_record *kernels, struct kernel_launch *launch_out)
{
    static const char what[] = "the router";
    if (description == NULL || kernels == NULL || launch_out == NULL || description->experts == NULL ||
        description->expert_offsets == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const struct linear_routed_experts_description *experts = description->experts;
    const uint32_t E = description->expert_count, P = description->pick_count;
    if (experts->reserved_zero != 0 || kernels->select == BACKEND_NO_KERNEL ||
        !shape_counts_are_valid(what, E, P, description->affinity_kind, description->order)) {
        if (experts->reserved_zero != 0 || kernels->select == BACKEND_NO_KERNEL) {
            REFUSE("%s: a reserved field that is not zero, or %s is not prepared", what, KERNEL_ROUTER_SELECT);
        }
        return STATUS_INVALID_ARGUMENT;
    }
    if (experts->row_count == 0 || experts->row_count > LINEAR_MAXIMUM_ROWS || experts->pairs_per_row != P ||
        experts->job_count != experts->row_count * P ||
        (experts->weight_format != WEIGHT_FORMAT_E2M1_SCALED && experts->weight_format != WEIGHT_FORMAT_E4M3_SCALED &&
         experts->weight_format != WEIGHT_FORMAT_EXL3 && experts->weight_format != WEIGHT_FORMAT_E4M3_BLOCK128 &&
         experts->weight_format != WEIGHT_FORMAT_E2M1_GFX950 && experts->weight_format != WEIGHT_FORMAT_E4M3_GFX950 &&
         experts->weight_format != WEIGHT_FORMAT_E4M3_BLOCK128_GFX950) ||
        !(description->route_scale > 0.0f)) {
        REFUSE("%s: the select writes 1 to %u rows of %u pairs, a job a pair, with a route scale above zero", what,
               LINEAR_MAXIMUM_ROWS, P);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t row_bytes = (uint64_t)E * 4u, rows_bytes = experts->row_count * row_bytes;
    const struct checked_range ranges[] = {
        {"the step block", description->step, sizeof(struct step_block), false},
        {"the router scores", description->scores, rows_bytes, false},
        {"the bias", description->bias, row_bytes, false},
        {"the expert offsets", description->offsets, (uint64_t)E * MODEL_EXPERT_MATRICES * 8u, false},
        {"the affinities", description->affinities, rows_bytes, false},
        {"the job table", experts->jobs, (uint64_t)experts->job_count * sizeof(struct expert_job_record), false},
        {"the experts' matrices", experts->expert_weights, 0, false},
        {"the rows' codes", experts->codes, 0, false},
        {"the rows' exponents", experts->exponents, 0, false},
        {"the rows' operands", experts->operands, 0, false},
        {"the hidden values", experts->hidden, 0, false},
        {"the hidden codes", experts->hidden_codes, 0, false},
        {"the hidden exponents", experts->hidden_exponents, 0, false},
        {"the hidden operands", experts->hidden_operands, 0, false},
        {"the pair outputs", experts->pair_output, 0, false},
        {"the row outputs", experts->row_output, 0, false},
    };
    uint64_t least_gate_up = 0, least_down = 0;
    if (!ranges_are_valid(what, ranges, sizeof ranges / sizeof ranges[0], arena_byte_count) ||
        !table_is_valid(what, experts->weight_format, &experts->gate_up_shape, &experts->down_shape,
                        description->expert_offsets, description->expert_widths, E, &experts->expert_weights,
                        &least_gate_up, &least_down)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t end = experts->expert_weights.byte_offset + experts->expert_weights.byte_count;
    const struct router_select_arguments record = {
        .step_offset = description->step.byte_offset,
        .scores_offset = description->scores.byte_offset,
        .bias_offset = description->bias.byte_offset,
        .expert_offsets_offset = description->offsets.byte_offset,
        .affinities_offset = description->affinities.byte_offset,
        .jobs_offset = experts->jobs.byte_offset,
        .weights_offset = experts->expert_weights.byte_offset,
        .gate_up_last_offset = end - least_gate_up,
        .down_last_offset = end - least_down,
        .row_count = experts->row_count,
        .reference_order = description->order == LINEAR_ORDER_REFERENCE ? 1u : 0u,
        .expert_count = E,
        .pick_count = P,
        .affinity_kind = description->affinity_kind,
        .route_scale = description->route_scale,
    };
    launch_fill(launch_out, kernels->select, 1, 1, 1, SELECT_THREADS, 0, &record, sizeof record);
    return STATUS_OK;
}

result_status router_projection_prepare(const struct router_projection_description *description,
                                        uint64_t arena_byte_count, const struct router_kernels_record *kernels,
                                        struct kernel_launch *launch_out)
{
    static const char what[] = "the router's projection";
    if (description == NULL || kernels == NULL || launch_out == NULL || kernels->projection == BACKEND_NO_KERNEL ||
        description->reserved_zero != 0 || description->row_count == 0 || description->row_count > 65535u ||
        description->hidden == 0 || description->hidden % 32u != 0 || description->expert_count == 0) {
        REFUSE("%s: a missing argument, an unprepared kernel or a count of zero", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const struct checked_range ranges[] = {
        {"the router's weights", description->weights, (uint64_t)description->expert_count * description->hidden * 2u, false},
        {"the rows", description->rows, (uint64_t)description->row_count * description->hidden * 2u, false},
        {"the scores", description->output, (uint64_t)description->row_count * description->expert_count * 4u, false},
    };
    if (!ranges_are_valid(what, ranges, 3, arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct router_projection_arguments record = {
        .weights_offset = description->weights.byte_offset,
        .rows_offset = description->rows.byte_offset,
        .output_offset = description->output.byte_offset,
        .row_count = description->row_count,
        .hidden = description->hidden,
        .expert_count = description->expert_count,
    };
    if (kernels->projection_tiles != BACKEND_NO_KERNEL && description->row_count >= PROJECTION_TILE_LEAST_ROWS &&
        description->expert_count % 16u == 0 &&
        description->hidden % PROJECTION_STAGE_INPUTS == 0) { /* many rows: the chains on the matrix unit, 16 experts by 64 rows a block */
        launch_fill(launch_out, kernels->projection_tiles, description->expert_count / 16u,
                    (description->row_count + PROJECTION_TILE_ROWS - 1u) / PROJECTION_TILE_ROWS, 1, PROJECTION_TILE_THREADS, 0, &record,
                    sizeof record);
        return STATUS_OK;
    }
    /* a thin step: a row a block (the kernel takes the rows its grid leaves it: four a block, or one) */
    const uint32_t expert_blocks = (description->expert_count + PROJECTION_OUTPUTS - 1u) / PROJECTION_OUTPUTS;
    const bool by_row = description->row_count <= LINEAR_MAXIMUM_ROWS && expert_blocks * description->row_count <= PROJECTION_BY_ROW_MOST_BLOCKS;
    launch_fill(launch_out, kernels->projection, expert_blocks,
                by_row ? description->row_count : (description->row_count + PROJECTION_ROWS - 1u) / PROJECTION_ROWS, 1, PROJECTION_THREADS, 0,
                &record, sizeof record);
    return STATUS_OK;
}

/* the wide select's launches: the four of any row count, or (small) the select and router_wide_small */
static result_status wide_launches(const struct router_wide_description *description, uint64_t arena_byte_count,
                                   const struct router_kernels_record *kernels, bool small, struct kernel_launch *launches_out)
{
    const char *what = small ? "the router's wide select in one block" : "the router's wide select";
    if (description == NULL || kernels == NULL || launches_out == NULL || description->expert_offsets == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t E = description->expert_count, P = description->pick_count, R = description->row_count;
    if (description->reserved_zero != 0 || kernels->wide_select == BACKEND_NO_KERNEL ||
        (small ? kernels->wide_small == BACKEND_NO_KERNEL
               : kernels->wide_count == BACKEND_NO_KERNEL || kernels->wide_place == BACKEND_NO_KERNEL || kernels->wide_jobs == BACKEND_NO_KERNEL)) {
        REFUSE("%s: a reserved field that is not zero, or a kernel of its launches is not prepared", what);
        return STATUS_INVALID_ARGUMENT;
    }
    if (small && description->row_count > ROUTER_SORT_ROWS) {
        REFUSE("%s: %u rows, at most %u", what, description->row_count, ROUTER_SORT_ROWS);
        return STATUS_INVALID_ARGUMENT;
    }
    if (!shape_counts_are_valid(what, E, P, description->affinity_kind, description->order)) {
        return STATUS_INVALID_ARGUMENT;
    }
    if (R == 0 || R > ROUTER_WIDE_MOST_ROWS || !(description->route_scale > 0.0f) ||
        (description->weight_format != WEIGHT_FORMAT_E2M1_SCALED && description->weight_format != WEIGHT_FORMAT_E4M3_SCALED &&
         description->weight_format != WEIGHT_FORMAT_EXL3 && description->weight_format != WEIGHT_FORMAT_E4M3_BLOCK128 &&
         description->weight_format != WEIGHT_FORMAT_E2M1_GFX950 && description->weight_format != WEIGHT_FORMAT_E4M3_GFX950 &&
         description->weight_format != WEIGHT_FORMAT_E4M3_BLOCK128_GFX950)) {
        REFUSE("%s: 1 to %u rows, a route scale above zero, experts of a format the path holds", what, ROUTER_WIDE_MOST_ROWS);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t row_bytes = (uint64_t)E * 4u, rows_bytes = R * row_bytes, pairs = (uint64_t)R * P;
    const uint64_t blocks = (R + ROUTER_SORT_ROWS - 1u) / ROUTER_SORT_ROWS;
    const struct checked_range ranges[] = {
        {"the step block", description->step, sizeof(struct step_block), false},
        {"the router scores", description->scores, rows_bytes, false},
        {"the bias", description->bias, row_bytes, false},
        {"the expert offsets", description->offsets, (uint64_t)E * MODEL_EXPERT_MATRICES * 8u, false},
        {"the experts' matrices", description->expert_weights, 0, false},
        {"the affinities", description->affinities, rows_bytes, false},
        {"the picks", description->picks, pairs * sizeof(struct router_pick), false},
        {"the counts", description->counts, blocks * row_bytes, false},
        {"the sorted pairs", description->pairs, pairs * sizeof(struct wide_pair), false},
        {"the runs", description->runs, (uint64_t)E * sizeof(struct wide_run), false},
        {"the tiles", description->tiles, (uint64_t)ROUTER_WIDE_TILES_OF(R, P, E) * sizeof(struct wide_expert_tile), false},
        {"the job table", description->jobs, (uint64_t)ROUTER_WIDE_JOBS_OF(R, P, E) * sizeof(struct expert_job_record), false},
    };
    uint64_t least_gate_up = 0, least_down = 0;
    if (!ranges_are_valid(what, ranges, sizeof ranges / sizeof ranges[0], arena_byte_count) ||
        !table_is_valid(what, description->weight_format, &description->gate_up_shape, &description->down_shape,
                        description->expert_offsets, description->expert_widths, E, &description->expert_weights,
                        &least_gate_up, &least_down)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t end = description->expert_weights.byte_offset + description->expert_weights.byte_count;
    const struct router_wide_arguments record = {
        .step_offset = description->step.byte_offset,
        .scores_offset = description->scores.byte_offset,
        .bias_offset = description->bias.byte_offset,
        .expert_offsets_offset = description->offsets.byte_offset,
        .affinities_offset = description->affinities.byte_offset,
        .picks_offset = description->picks.byte_offset,
        .counts_offset = description->counts.byte_offset,
        .pairs_offset = description->pairs.byte_offset,
        .runs_offset = description->runs.byte_offset,
        .tiles_offset = description->tiles.byte_offset,
        .jobs_offset = description->jobs.byte_offset,
        .weights_offset = description->expert_weights.byte_offset,
        .gate_up_last_offset = end - least_gate_up,
        .down_last_offset = end - least_down,
        .row_count = R,
        .reference_order = description->order == LINEAR_ORDER_REFERENCE ? 1u : 0u,
        .expert_count = E,
        .pick_count = P,
        .affinity_kind = description->affinity_kind,
        .route_scale = description->route_scale,
    };
    struct kernel_launch launches[ROUTER_WIDE_LAUNCH_COUNT];
    launch_fill(&launches[ROUTER_WIDE_SELECT_LAUNCH], kernels->wide_select, (R + LINEAR_MAXIMUM_ROWS - 1u) / LINEAR_MAXIMUM_ROWS, 1, 1,
                SELECT_THREADS, 0, &record, sizeof record);
    if (small) {
        launch_fill(&launches[1], kernels->wide_small, 1, 1, 1, WIDE_SORT_THREADS, 0, &record, sizeof record);
        memcpy(launches_out, launches, ROUTER_WIDE_SMALL_LAUNCH_COUNT * sizeof launches[0]);
        return STATUS_OK;
    }
    launch_fill(&launches[ROUTER_WIDE_COUNT_LAUNCH], kernels->wide_count, (uint32_t)blocks, 1, 1, WIDE_SORT_THREADS, 0, &record, sizeof record);
    launch_fill(&launches[ROUTER_WIDE_PLACE_LAUNCH], kernels->wide_place, (uint32_t)blocks, 1, 1, WIDE_SORT_THREADS, 0, &record, sizeof record);
    launch_fill(&launches[ROUTER_WIDE_JOBS_LAUNCH], kernels->wide_jobs, 1, 1, 1, WIDE_SORT_THREADS, 0, &record, sizeof record);
    memcpy(launches_out, launches, sizeof launches);
    return STATUS_OK;
}

result_status router_wide_prepare(const struct router_wide_description *description, uint64_t arena_byte_count,
                                  const struct router_kernels_record *kernels, struct kernel_launch *launches_out)
{
    return wide_launches(description, arena_byte_count, kernels, false, launches_out);
}

result_status router_wide_small_prepare(const struct router_wide_description *description, uint64_t arena_byte_count,
                                        const struct router_kernels_record *kernels, struct kernel_launch *launches_out)
{
    return wide_launches(description, arena_byte_count, kernels, true, launches_out);
}
