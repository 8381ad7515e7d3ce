/*
 * site.c -- load-time preparation of the launches a block's site front stands for: the dense product (a site's mix
 * project, the router's scores) and the site's mix finish and post. Entry points and refusal rules follow the
 * reference's source/dense_linear.c and source/hyper_connection.c (include/anemone/dense_linear.h:27-99,
 * include/anemone/hyper_connection.h:6-71).
 *
 *   launch        kernel                                grid                               block
 *   dense         dense_linear_<type>_<R>[_narrow]      (outputs / (4 or 1), 1 or rows, 1) 256
 *   dense, wide   dense_linear_<type>_8_wide            (outputs / 8, ceil(rows / 8), 1)   256
 *   mix finish    hyper_mix_finish                      (1, rows, 1)                       width / 8
 *   post          hyper_post_entry                      (width / 1024, rows, 1)            128
 */
#include <stdio.h>
#include <string.h>

#include "prepare_common.h"

#define SITE_DEFAULT_WIDTH 5120u
#define DENSE_BY_ROW_MOST_BLOCKS 4096u /* a block a row and an output while that leaves at most so many blocks */
#define SITE_MOST_WIDTH 8192u
#define SITE_WIDTH_STEP (HYPER_VALUES_PER_THREAD * HYPER_PIECE_THREADS)

static const char *const dense_type_names[DENSE_TYPE_COUNT] = {"bfloat16", "float32"};
static const uint32_t dense_row_forms[DENSE_ROW_INSTANCES] = {1u, 8u};

result_status dense_linear_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                           struct dense_linear_kernels *kernels_out)
{
    if (backend == NULL || backend->kernel_prepare == NULL || card == NULL || kernels_out == NULL) {
        REFUSE("the kernels of the dense products: a missing argument");
        return STATUS_INVALID_ARGUMENT;
    }
    struct dense_linear_kernels kernels;
    for (uint32_t instance = 0; instance < DENSE_INSTANCES; instance++) {
        const uint32_t form = instance / DENSE_FORM_INSTANCES, type = instance % DENSE_FORM_INSTANCES / DENSE_ROW_INSTANCES;
        char name[56];
        (void)snprintf(name, sizeof name, "%s%s_%u%s", KERNEL_DENSE_LINEAR_STEM, dense_type_names[type],
                       dense_row_forms[instance % DENSE_ROW_INSTANCES], form != 0u ? "_narrow" : "");
        const result_status status =
            backend->kernel_prepare(card, KERNEL_FILE_DENSE_LINEAR, name, sizeof(struct dense_linear_arguments), &kernels.products[instance]);
        if (status != STATUS_OK) {
            REFUSE("the kernels of the dense products: %s is not prepared: %s", name, status_text(status));
            return status;
        }
    }
    for (uint32_t type = 0; type < DENSE_TYPE_COUNT; type++) {
        char name[56];
        (void)snprintf(name, sizeof name, "%s%s_8_wide", KERNEL_DENSE_LINEAR_STEM, dense_type_names[type]);
        const result_status status =
            backend->kernel_prepare(card, KERNEL_FILE_DENSE_LINEAR, name, sizeof(struct dense_linear_arguments), &kernels.wide_products[type]);
        if (status != STATUS_OK) {
            REFUSE("the kernels of the dense products: %s is not prepared: %s", name, status_text(status));
            return status;
        }
    }
    *kernels_out = kernels;
    return STATUS_OK;
}

result_status dense_linear_prepare(const struct dense_linear_description *description, uint64_t arena_byte_count,
                                   const struct dense_linear_kernels *kernels, struct kernel_launch *launch_out)
{
    static const char what[] = "a dense product";
    if (description == NULL || kernels == NULL || launch_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    if (description->weight_type >= DENSE_TYPE_COUNT || description->output_type >= DENSE_TYPE_COUNT ||
        (description->flags & ~DENSE_FLAGS) != 0u || description->row_count == 0u || description->output_size == 0u ||
        description->output_size % DENSE_OUTPUTS_PER_BLOCK != 0u || description->input_size == 0u ||
        description->input_size % DENSE_CHUNK_INPUTS != 0u) {
        REFUSE("%s: types below %u, flags inside 0x%X, 1 row or more, outputs in whole %u and inputs in whole %u", what, DENSE_TYPE_COUNT,
               DENSE_FLAGS, DENSE_OUTPUTS_PER_BLOCK, DENSE_CHUNK_INPUTS);
        return STATUS_INVALID_ARGUMENT;
    }
    if (description->row_count > DENSE_MOST_ROWS * LINEAR_MAXIMUM_ROWS) {
        REFUSE("%s: at most %u rows", what, DENSE_MOST_ROWS * LINEAR_MAXIMUM_ROWS);
        return STATUS_INVALID_ARGUMENT;
    }
    if ((description->flags & (DENSE_STEP_ROWS | DENSE_CONE_ROWS)) != 0u || description->cone_layer != 0u || description->step.byte_count != 0u) {
        REFUSE("%s: the head's step rows and the cone's rows are not built", what);
        return STATUS_UNSUPPORTED;
    }
    const uint64_t weight_bytes = description->weight_type == DENSE_FLOAT32 ? 4u : 2u, output_bytes = description->output_type == DENSE_FLOAT32 ? 4u : 2u;
    const uint64_t matrix = product_or_most(product_or_most(description->output_size, description->input_size), weight_bytes);
    const struct checked_range ranges[] = {
        {"the weights", description->weights, matrix, true},
        {"the rows", description->rows, (uint64_t)description->row_count * description->input_size * 2u, false},
        {"the output", description->output, (uint64_t)description->row_count * description->output_size * output_bytes, false},
    };
    if (!ranges_are_valid(what, ranges, 3, arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct dense_linear_arguments record = {description->weights.byte_offset, description->rows.byte_offset, description->output.byte_offset, 0,
                                                  description->output_size, description->input_size, description->row_count,
                                                  description->output_type, description->flags, description->output_scale, description->epsilon, 0};
    const bool few_blocks = description->output_size / DENSE_OUTPUTS_PER_BLOCK < DENSE_NARROW_BELOW_BLOCKS &&
                            (uint64_t)description->output_size * description->row_count <=
                                (description->row_count > LINEAR_MAXIMUM_ROWS ? DENSE_BY_ROW_MOST_BLOCKS : DENSE_BY_ROW_MOST_BLOCKS / 4u);
    if (description->row_count > LINEAR_MAXIMUM_ROWS && !few_blocks) {
        /* a wide launch: groups of 8 rows on grid[1]; 8 outputs a block where they divide, else the 8-row instance's 4 */
        const bool eight = description->output_size % DENSE_WIDE_OUTPUTS == 0u;
        const uint32_t wide = eight ? kernels->wide_products[description->weight_type]
                                    : kernels->products[description->weight_type * DENSE_ROW_INSTANCES + 1u];
        if (wide == BACKEND_NO_KERNEL) {
            REFUSE("%s: its kernel is not prepared", what);
            return STATUS_INVALID_ARGUMENT;
        }
        launch_fill(launch_out, wide, description->output_size / (eight ? DENSE_WIDE_OUTPUTS : DENSE_OUTPUTS_PER_BLOCK),
                    (description->row_count + LINEAR_MAXIMUM_ROWS - 1u) / LINEAR_MAXIMUM_ROWS, 1, DENSE_THREADS_VALUE, 0, &record, sizeof record);
        return STATUS_OK;
    }
    /* fewer than DENSE_NARROW_BELOW_BLOCKS blocks of four outputs: a block owns one, the same operations for every output */
    const uint32_t form = description->output_size / DENSE_OUTPUTS_PER_BLOCK < DENSE_NARROW_BELOW_BLOCKS ? 1u : 0u;
    /* few outputs and several rows (a site's 24 mixes, up to some 170 rows): a block a row and an output, the one-row
     * instance on a grid of (outputs, rows), so that many units are at work; every output's operations are the same */
    const bool by_row = form != 0u && description->row_count > 1u && few_blocks;
    const uint32_t kernel = kernels->products[form * DENSE_FORM_INSTANCES + description->weight_type * DENSE_ROW_INSTANCES +
                                              (description->row_count > 1u && !by_row ? 1u : 0u)];
    if (kernel == BACKEND_NO_KERNEL) {
        REFUSE("%s: its kernel is not prepared", what);
        return STATUS_INVALID_ARGUMENT;
    }
    launch_fill(launch_out, kernel, description->output_size / (form != 0u ? 1u : DENSE_OUTPUTS_PER_BLOCK), by_row ? description->row_count : 1, 1,
                DENSE_THREADS_VALUE, 0, &record, sizeof record);
    return STATUS_OK;
}

result_status hyper_kernels_prepare(const struct backend_operations *backend, struct device_card *card, struct hyper_kernels_record *kernels_out)
{
    if (backend == NULL || backend->kernel_prepare == NULL || card == NULL || kernels_out == NULL) {
        REFUSE("the kernels of the hyper connection: a missing argument");
        return STATUS_INVALID_ARGUMENT;
    }
    struct hyper_kernels_record kernels;
    memset(&kernels, 0xFF, sizeof kernels); /* every handle BACKEND_NO_KERNEL */
    result_status status = backend->kernel_prepare(card, KERNEL_FILE_HYPER_CONNECTION, KERNEL_HYPER_MIX_FINISH,
                                                   sizeof(struct hyper_finish_arguments), &kernels.mix_finish);
    if (status == STATUS_OK) {
        status = backend->kernel_prepare(card, KERNEL_FILE_HYPER_CONNECTION, KERNEL_HYPER_POST, sizeof(struct hyper_post_arguments), &kernels.post);
    }
    if (status != STATUS_OK) {
        REFUSE("the kernels of the hyper connection: the mix finish or the post is not prepared: %s", status_text(status));
        return status;
    }
    *kernels_out = kernels;
    return STATUS_OK;
}

result_status hyper_site_prepare(const struct hyper_site_description *description, uint64_t arena_byte_count,
                                 const struct hyper_kernels_record *kernels, struct kernel_launch *launches_out)
{
    static const char what[] = "a site of the hyper connection";
    if (description == NULL || kernels == NULL || launches_out == NULL || kernels->mix_finish == BACKEND_NO_KERNEL ||
        kernels->post == BACKEND_NO_KERNEL) {
        REFUSE("%s: a missing argument or an unprepared kernel", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t width = description->reserved_zero != 0u ? description->reserved_zero : SITE_DEFAULT_WIDTH, rows = description->row_count;
    if (rows == 0u || rows > DENSE_MOST_ROWS || width % SITE_WIDTH_STEP != 0u || width > SITE_MOST_WIDTH) {
        REFUSE("%s: 1 to %u rows of a width in whole %u up to %u", what, DENSE_MOST_ROWS, SITE_WIDTH_STEP, SITE_MOST_WIDTH);
        return STATUS_INVALID_ARGUMENT;
    }
    const bool combined = description->routed_sums.byte_count != 0u;
    const uint64_t row_values = (uint64_t)rows * width;
    const struct checked_range ranges[] = {
        {"the streams", description->streams, row_values * MODEL_STREAMS * 2u, false},
        {"the carried pre", description->carried_pre, (uint64_t)rows * MODEL_STREAMS * 4u, false},
        {"the mixes", description->mixes, (uint64_t)rows * MODEL_MIXES * 4u, false},
        {"the scale", description->scale, HYPER_SCALES * 4u, true},
        {"the base", description->base, MODEL_MIXES * 4u, true},
        {"the norm's weight", description->norm_weight, (uint64_t)width * 2u, true},
        {"post", description->post, (uint64_t)rows * MODEL_STREAMS * 4u, false},
        {"comb", description->comb, (uint64_t)rows * MODEL_STREAMS * MODEL_STREAMS * 4u, false},
        {"the hidden rows", description->hidden, row_values * 2u, false},
        {"the sublayer's output", description->output, row_values * 2u, false},
        {"the routed sums", description->routed_sums, row_values * 4u, false},
    };
    if (!ranges_are_valid(what, ranges, combined ? 11u : 10u, arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct hyper_finish_arguments finish = {description->streams.byte_offset, description->carried_pre.byte_offset,
                                                  description->mixes.byte_offset, description->scale.byte_offset, description->base.byte_offset,
                                                  description->post.byte_offset, description->comb.byte_offset,
                                                  description->norm_weight.byte_offset, description->hidden.byte_offset};
    const struct hyper_post_arguments post = {description->streams.byte_offset, description->post.byte_offset, description->comb.byte_offset,
                                              description->output.byte_offset, combined ? description->routed_sums.byte_offset : 0,
                                              combined ? 1u : 0u, 0};
    launch_fill(&launches_out[HYPER_SITE_MIX_FINISH], kernels->mix_finish, 1, rows, 1, width / HYPER_VALUES_PER_THREAD, 0, &finish, sizeof finish);
    launch_fill(&launches_out[HYPER_SITE_POST], kernels->post, width / SITE_WIDTH_STEP, rows, 1, HYPER_PIECE_THREADS, 0, &post, sizeof post);
    return STATUS_OK;
}
