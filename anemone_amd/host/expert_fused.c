/*
 * expert_fused.c -- load-time preparation of the producer: gate with up and the quantization of the hidden vectors
 * in one launch. Entry points and refusal rules follow the reference's source/expert_fused.c:114-204 and
 * include/anemone/expert_fused.h:37-60; and of the FFN site's join and shared join (source/expert_fused.c:207-368,
 * include/anemone/expert_fused.h:63-101).
 *
 *   launch        kernel                          grid                                   block
 *   producer      expert_gate_up_quantize_<S>     (ceil(outputs / strip), jobs + 1, 1)   64 S
 *   join          expert_join                     (width / 1024, rows, 1)                128
 *   post          hyper_post_entry                (width / 1024, rows, 1)                128
 *   shared join   expert_shared_join_<S>          (ceil(width / 32), 1, 1)               64 S
 * strip = 64 outputs of E2M1 weights, 32 of E4M3; the last row of blocks takes the pairs that stand in no job.
 */
#include <stdio.h>
#include <string.h>

#include "prepare_common.h"

static const uint32_t slice_counts[LINEAR_SLICE_INSTANCES] = {1u, 2u, 4u, 8u, 16u};
#define BUILT_INSTANCES 4u

result_status expert_fused_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                           uint32_t arithmetic_class, struct expert_fused_kernels *kernels_out)
{
    if (backend == NULL || backend->kernel_prepare == NULL || card == NULL || kernels_out == NULL ||
        arithmetic_class != ARITHMETIC_CLASS_GFX950) {
        REFUSE("the kernels of the fused experts: a missing argument, or a class other than %u", ARITHMETIC_CLASS_GFX950);
        return STATUS_INVALID_ARGUMENT;
    }
    struct expert_fused_kernels kernels;
    memset(&kernels, 0xFF, sizeof kernels); /* every handle BACKEND_NO_KERNEL */
    for (uint32_t instance = 0; instance < BUILT_INSTANCES; instance++) {
        char name[56];
        (void)snprintf(name, sizeof name, "%s%u", KERNEL_EXPERT_GATE_UP_QUANTIZE_STEM, slice_counts[instance]);
        result_status status = backend->kernel_prepare(card, KERNEL_FILE_EXPERT_LINEAR, name, sizeof(struct expert_gate_up_quantize_arguments),
                                                       &kernels.gate_up_quantize[instance]);
        if (status == STATUS_OK) {
            (void)snprintf(name, sizeof name, "%se4m3_%u", KERNEL_EXPERT_GATE_UP_QUANTIZE_STEM, slice_counts[instance]);
            status = backend->kernel_prepare(card, KERNEL_FILE_EXPERT_LINEAR, name, sizeof(struct expert_gate_up_quantize_arguments),
                                             &kernels.gate_up_quantize_e4m3[instance]);
        }
        if (status == STATUS_OK) {
            (void)snprintf(name, sizeof name, "%s%u", KERNEL_EXPERT_SHARED_JOIN_STEM, slice_counts[instance]);
            status = backend->kernel_prepare(card, KERNEL_FILE_TRUNK_LINEAR, name, sizeof(struct expert_shared_join_arguments),
                                             &kernels.shared_join[instance]);
        }
        if (status != STATUS_OK) {
            REFUSE("the kernels of the fused experts: %s is not prepared: %s", name, status_text(status));
            return status;
        }
    }
    result_status status = backend->kernel_prepare(card, KERNEL_FILE_HYPER_CONNECTION, KERNEL_EXPERT_JOIN,
                                                   sizeof(struct expert_join_arguments), &kernels.join);
    if (status == STATUS_OK) {
        status = backend->kernel_prepare(card, KERNEL_FILE_HYPER_CONNECTION, KERNEL_HYPER_POST, sizeof(struct hyper_post_arguments),
                                         &kernels.post);
    }
    if (status != STATUS_OK) {
        REFUSE("the kernels of the fused experts: the join or the post is not prepared: %s", status_text(status));
        return status;
    }
    *kernels_out = kernels;
    return STATUS_OK;
}

static bool ranges_share_a_byte(struct linear_range a, struct linear_range b)
{
    return a.byte_count != 0 && b.byte_count != 0 && a.byte_offset < b.byte_offset + b.byte_count &&
           b.byte_offset < a.byte_offset + a.byte_count;
}

result_status expert_producer_prepare(const struct linear_routed_experts_description *description,
                                      struct linear_range arrivals, uint64_t arena_byte_count,
                                      const struct linear_kernels_record *linear_kernels,
                                      const struct expert_fused_kernels *kernels, struct kernel_launch *launch_out)
{
    static const char what[] = "the producer";
    if (description == NULL || linear_kernels == NULL || kernels == NULL || launch_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    /* what the routed experts' prepare refuses is refused here, behind its one error line; its launches are discarded */
    struct kernel_launch discarded[LINEAR_ROUTED_EXPERTS_LAUNCH_COUNT];
    const result_status checked = linear_routed_experts_prepare(description, arena_byte_count, linear_kernels, discarded);
    if (checked != STATUS_OK) {
        return checked;
    }
    const uint64_t pairs = (uint64_t)description->row_count * description->pairs_per_row;
    const uint32_t outputs = description->gate_up_shape.output_size;
    if (description->row_count > LINEAR_MAXIMUM_ROWS || pairs > EXPERT_PRODUCER_MOST_PAIRS || outputs % 32u != 0) {
        REFUSE("%s: at most %u rows and %u pairs, outputs a multiple of 32", what, LINEAR_MAXIMUM_ROWS, EXPERT_PRODUCER_MOST_PAIRS);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t arrival_bytes = (uint64_t)description->job_count * (outputs / 32u) * 4u;
    const struct linear_range *others[] = {&description->jobs, &description->expert_weights, &description->codes, &description->exponents,
                                           &description->operands, &description->hidden, &description->hidden_codes,
                                           &description->hidden_exponents, &description->hidden_operands, &description->pair_output,
                                           &description->row_output};
    bool shares = false;
    for (uint32_t i = 0; i < sizeof others / sizeof others[0]; i++) {
        shares = shares || ranges_share_a_byte(arrivals, *others[i]);
    }
    if (arrivals.byte_offset % LINEAR_OFFSET_ALIGNMENT_BYTES != 0 || arrivals.byte_count < arrival_bytes ||
        arrivals.byte_offset > arena_byte_count || arrivals.byte_count > arena_byte_count - arrivals.byte_offset || shares) {
        REFUSE("%s: the arrival counters: %llu bytes on a multiple of %u inside the arena, sharing no byte with another range", what,
               (unsigned long long)arrival_bytes, LINEAR_OFFSET_ALIGNMENT_BYTES);
        return STATUS_INVALID_ARGUMENT;
    }
    const bool bytes = description->weight_format == WEIGHT_FORMAT_E4M3_SCALED;
    uint32_t instance = 0;
    while (instance < BUILT_INSTANCES && slice_counts[instance] != description->gate_up_slice_count) {
        instance++;
    }
    const uint32_t kernel = instance == BUILT_INSTANCES ? BACKEND_NO_KERNEL
                            : bytes                     ? kernels->gate_up_quantize_e4m3[instance]
                                                        : kernels->gate_up_quantize[instance];
    if (kernel == BACKEND_NO_KERNEL) {
        REFUSE("%s: the kernel of %u slices is not prepared", what, description->gate_up_slice_count);
        return STATUS_INVALID_ARGUMENT;
    }
    const struct expert_gate_up_quantize_arguments record = {
        description->jobs.byte_offset, description->codes.byte_offset, description->exponents.byte_offset,
        description->operands.byte_offset, description->hidden.byte_offset, description->hidden_codes.byte_offset,
        description->hidden_exponents.byte_offset, description->hidden_operands.byte_offset, arrivals.byte_offset,
        outputs, description->gate_up_shape.input_size, (uint32_t)pairs, description->pairs_per_row, description->activation_limit, 0};
    const uint32_t strip = bytes ? 32u : 64u;
    launch_fill(launch_out, kernel, (outputs + strip - 1u) / strip, description->job_count + 1u, 1,
                64u * description->gate_up_slice_count, 0, &record, sizeof record);
    return STATUS_OK;
}

/* ---- the join and the shared join ---- */
#define JOIN_ROW_VALUES (HYPER_VALUES_PER_THREAD * HYPER_PIECE_THREADS) /* values of a row a block of a join takes */
#define JOIN_MOST_ROWS 65535u
#define JOIN_DEFAULT_WIDTH 5120u /* the reference's model */
enum { JOIN_RANGES = 6, DOWN_RANGES = 4 };

static uint32_t join_width_of(const struct expert_join_description *join)
{
    return join->width == 0 ? JOIN_DEFAULT_WIDTH : join->width;
}

static bool join_counts_are_valid(const char *what, const struct expert_join_description *join, uint32_t most_rows)
{
    const uint32_t width = join_width_of(join);
    if (join->row_count == 0 || join->row_count > most_rows || join->pairs_per_row == 0 || width % JOIN_ROW_VALUES != 0 ||
        (uint64_t)join->row_count * join->pairs_per_row > UINT32_MAX) {
        REFUSE("%s: %u rows, %u pairs a row, %u wide: it takes 1 to %u rows, a pair or more, a width that is a multiple of %u", what,
               join->row_count, join->pairs_per_row, width, most_rows, JOIN_ROW_VALUES);
        return false;
    }
    return true;
}

/* the ranges of a join, the row sums last: JOIN_RANGES of them, or one fewer where it writes no row sums */
static uint32_t join_ranges_of(const struct expert_join_description *join, struct checked_range *ranges_out)
{
    const uint64_t rows = join->row_count, width = join_width_of(join);
    const struct checked_range ranges[JOIN_RANGES] = {
        {"the pair outputs", join->pair_output, linear_values_byte_count(rows * join->pairs_per_row, width), false},
        {"the shared expert's output", join->shared_output, linear_values_byte_count(rows, width), false},
        {"the streams", join->streams, linear_values_byte_count(rows * MODEL_STREAMS, width), false},
        {"the post", join->post, rows * MODEL_STREAMS * 4u, false},
        {"the comb", join->comb, rows * MODEL_STREAMS * MODEL_STREAMS * 4u, false},
        {"the row sums", join->row_sums, linear_sums_byte_count(rows, width), false},
    };
    memcpy(ranges_out, ranges, sizeof ranges);
    return join->row_sums.byte_count != 0 ? JOIN_RANGES : JOIN_RANGES - 1u;
}

static uint64_t row_sums_offset_of(const struct expert_join_description *join)
{
    return join->row_sums.byte_count != 0 ? join->row_sums.byte_offset : EXPERT_JOIN_NO_ROW_SUMS;
}

result_status expert_join_prepare(const struct expert_join_description *description, uint64_t arena_byte_count,
                                  const struct expert_fused_kernels *kernels, struct kernel_launch *launch_out)
{
    static const char what[] = "the join of the FFN site";
    struct checked_range ranges[JOIN_RANGES];
    if (description == NULL || kernels == NULL || launch_out == NULL || kernels->join == BACKEND_NO_KERNEL) {
        REFUSE("%s: a missing argument or an unprepared kernel", what);
        return STATUS_INVALID_ARGUMENT;
    }
    if (!join_counts_are_valid(what, description, JOIN_MOST_ROWS) ||
        !ranges_are_valid(what, ranges, join_ranges_of(description, ranges), arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct expert_join_arguments record = {
        description->pair_output.byte_offset, description->shared_output.byte_offset, description->streams.byte_offset,
        description->post.byte_offset, description->comb.byte_offset, row_sums_offset_of(description), description->pairs_per_row, 0};
    launch_fill(launch_out, kernels->join, join_width_of(description) / JOIN_ROW_VALUES, description->row_count, 1,
                HYPER_PIECE_THREADS, 0, &record, sizeof record);
    return STATUS_OK;
}

result_status expert_post_prepare(const struct expert_join_description *join, uint64_t arena_byte_count, uint32_t kernel,
                                  struct kernel_launch *launch_out)
{
    static const char what[] = "the post of the FFN site";
    struct checked_range ranges[JOIN_RANGES];
    if (join == NULL || launch_out == NULL || kernel == BACKEND_NO_KERNEL) {
        REFUSE("%s: a missing argument or an unprepared kernel", what);
        return STATUS_INVALID_ARGUMENT;
    }
    if (join->row_sums.byte_count == 0) {
        REFUSE("%s: it reads the row sums: their range has no bytes", what);
        return STATUS_INVALID_ARGUMENT;
    }
    if (!join_counts_are_valid(what, join, JOIN_MOST_ROWS) || !ranges_are_valid(what, ranges, join_ranges_of(join, ranges), arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct hyper_post_arguments record = {join->streams.byte_offset, join->post.byte_offset, join->comb.byte_offset,
                                                join->shared_output.byte_offset, join->row_sums.byte_offset, 1u, 0};
    launch_fill(launch_out, kernel, join_width_of(join) / JOIN_ROW_VALUES, join->row_count, 1, HYPER_PIECE_THREADS, 0, &record, sizeof record);
    return STATUS_OK;
}

result_status expert_shared_join_prepare(const struct expert_shared_join_description *description, uint64_t arena_byte_count,
                                         const struct linear_kernels_record *linear_kernels, const struct expert_fused_kernels *kernels,
                                         struct kernel_launch *launch_out)
{
    static const char what[] = "the shared join of the FFN site";
    struct checked_range ranges[DOWN_RANGES + JOIN_RANGES];
    struct kernel_launch separate;
    if (description == NULL || linear_kernels == NULL || kernels == NULL || launch_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const struct expert_join_description *join = &description->join;
    /* what the down's own launch refuses is refused here, behind its one error line; the launch is discarded */
    struct linear_trunk_quantized_description down;
    memset(&down, 0, sizeof down);
    down.matrices[0] = description->down;
    down.codes = description->codes;
    down.exponents = description->exponents;
    down.operands = description->operands;
    down.outputs[0] = join->shared_output;
    down.matrix_count = 1;
    down.row_count = join->row_count;
    const result_status status = linear_trunk_quantized_prepare(&down, arena_byte_count, linear_kernels, &separate);
    if (status != STATUS_OK) {
        return status;
    }
    uint32_t instance = 0;
    while (instance < BUILT_INSTANCES && slice_counts[instance] != description->down.slice_count) {
        instance++;
    }
    if (!join_counts_are_valid(what, join, LINEAR_MAXIMUM_ROWS) || instance == BUILT_INSTANCES ||
        kernels->shared_join[instance] == BACKEND_NO_KERNEL) {
        REFUSE("%s: at most %u rows, and a prepared kernel of %u slices", what, LINEAR_MAXIMUM_ROWS, description->down.slice_count);
        return STATUS_INVALID_ARGUMENT;
    }
    const struct matrix_shape_record *shape = &description->down.shape;
    if (shape->output_size != join_width_of(join)) {
        REFUSE("%s: down has %u outputs: the streams are %u wide", what, shape->output_size, join_width_of(join));
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t rows = join->row_count;
    const struct checked_range down_ranges[DOWN_RANGES] = {
        {"down", description->down.stored, description->down.stored.byte_count, true},
        {"the hidden codes", description->codes, linear_codes_byte_count(rows, shape->input_size), false},
        {"the hidden exponents", description->exponents, linear_exponents_byte_count(rows, shape->input_size), false},
        {"the hidden operands", description->operands, 0, false},
    };
    memcpy(ranges, down_ranges, sizeof down_ranges);
    const uint32_t range_count = DOWN_RANGES + join_ranges_of(join, ranges + DOWN_RANGES);
    if (!ranges_are_valid(what, ranges, range_count, arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct expert_shared_join_arguments record = {
        description->down.stored.byte_offset, description->codes.byte_offset, description->exponents.byte_offset,
        description->operands.byte_offset, join->shared_output.byte_offset, join->pair_output.byte_offset, join->streams.byte_offset,
        join->post.byte_offset, join->comb.byte_offset, row_sums_offset_of(join), shape->input_size, join->row_count,
        join->pairs_per_row, join->width};
    launch_fill(launch_out, kernels->shared_join[instance], (shape->output_size + TRUNK_STRIP_OUTPUTS - 1u) / TRUNK_STRIP_OUTPUTS, 1, 1,
                64u * description->down.slice_count, 0, &record, sizeof record);
    return STATUS_OK;
}
