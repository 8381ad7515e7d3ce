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
    if (!bytes && description->weight_format != WEIGHT_FORMAT_E2M1_SCALED) {
        REFUSE("%s: experts of format %u: the producer is built for formats %u and %u (the others take the launches it stands for)", what,
               (uint32_t)description->weight_format, (uint32_t)WEIGHT_FORMAT_E2M1_SCALED, (uint32_t)WEIGHT_FORMAT_E4M3_SCALED);
        return STATUS_INVALID_ARGUMENT;
    }
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

/* ---- the join and the shared join ---------------------------------------------------------------------------------
 * Written from the contract of the reference's include/anemone/expert_fused.h:63-101: what a join reads (the routed
 * experts' pair outputs, the shared expert's rows, the four streams, the row's post and comb) and what it writes (the
 * streams in place and, where the caller gives them room, the routed row sums). */

/* what a join's description comes to once read: the counts every range's size is made of */
struct join_extent {
    uint64_t rows;
    uint64_t pairs;      /* rows times the picks of a row */
    uint32_t width;      /* of a stream's row; the description's 0 stands for the reference's model */
    uint32_t row_blocks; /* blocks that share a row: grid[0] */
    bool stores_sums;
};

static const uint32_t join_block_values = HYPER_VALUES_PER_THREAD * HYPER_PIECE_THREADS;

static bool join_extent_read(const char *who, const struct expert_join_description *join, uint32_t row_limit, struct join_extent *extent_out)
{
    struct join_extent extent;
    extent.width = join->width != 0 ? join->width : 5120u;
    extent.rows = join->row_count;
    extent.pairs = extent.rows * join->pairs_per_row;
    extent.row_blocks = extent.width / join_block_values;
    extent.stores_sums = join->row_sums.byte_count != 0;
    const bool counts_fit = extent.rows >= 1 && extent.rows <= row_limit && join->pairs_per_row >= 1 && extent.pairs <= UINT32_MAX;
    if (!counts_fit || extent.row_blocks * join_block_values != extent.width) {
        REFUSE("%s: the join is built for 1..%u rows of one pick or more and rows of whole %u values; asked: %u rows, %u picks, %u values",
               who, row_limit, join_block_values, join->row_count, join->pairs_per_row, extent.width);
        return false;
    }
    *extent_out = extent;
    return true;
}

/* the ranges of one description, gathered as its parts name them and checked together */
struct range_list {
    struct checked_range item[12];
    uint32_t used;
};

static void list_range(struct range_list *list, const char *name, struct linear_range range, uint64_t touched, bool exact)
{
    const struct checked_range entry = {name, range, touched, exact};
    list->item[list->used++] = entry;
}

static void list_join_ranges(struct range_list *list, const struct expert_join_description *join, const struct join_extent *extent)
{
    const uint64_t stream_rows = extent->rows * MODEL_STREAMS;
    list_range(list, "pair_output (bfloat16, a row a pair)", join->pair_output, linear_values_byte_count(extent->pairs, extent->width), false);
    list_range(list, "shared_output (bfloat16, a row a row)", join->shared_output, linear_values_byte_count(extent->rows, extent->width), false);
    list_range(list, "streams (bfloat16, four rows a row)", join->streams, linear_values_byte_count(stream_rows, extent->width), false);
    list_range(list, "post (float32, four a row)", join->post, stream_rows * sizeof(float), false);
    list_range(list, "comb (float32, four by four a row)", join->comb, stream_rows * MODEL_STREAMS * sizeof(float), false);
    if (extent->stores_sums) {
        list_range(list, "row_sums (float32, a row a row)", join->row_sums, linear_sums_byte_count(extent->rows, extent->width), false);
    }
}

static bool list_holds(const char *who, const struct range_list *list, uint64_t arena_byte_count)
{
    return ranges_are_valid(who, list->item, list->used, arena_byte_count);
}

result_status expert_join_prepare(const struct expert_join_description *description, uint64_t arena_byte_count,
                                  const struct expert_fused_kernels *kernels, struct kernel_launch *launch_out)
{
    static const char who[] = "expert_join_prepare";
    if (description == NULL || kernels == NULL || launch_out == NULL) {
        REFUSE("%s: description, kernels and launch are all needed", who);
        return STATUS_INVALID_ARGUMENT;
    }
    if (kernels->join == BACKEND_NO_KERNEL) {
        REFUSE("%s: expert_fused_kernels_prepare has not found the join's kernel", who);
        return STATUS_INVALID_ARGUMENT;
    }
    struct join_extent extent;
    struct range_list list = {.used = 0};
    if (!join_extent_read(who, description, 65535u, &extent)) {
        return STATUS_INVALID_ARGUMENT;
    }
    list_join_ranges(&list, description, &extent);
    if (!list_holds(who, &list, arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    struct expert_join_arguments record;
    memset(&record, 0, sizeof record);
    record.pair_output_offset = description->pair_output.byte_offset;
    record.shared_output_offset = description->shared_output.byte_offset;
    record.streams_offset = description->streams.byte_offset;
    record.post_offset = description->post.byte_offset;
    record.comb_offset = description->comb.byte_offset;
    record.row_sums_offset = extent.stores_sums ? description->row_sums.byte_offset : EXPERT_JOIN_NO_ROW_SUMS;
    record.pairs_per_row = description->pairs_per_row;
    launch_fill(launch_out, kernels->join, extent.row_blocks, description->row_count, 1, HYPER_PIECE_THREADS, 0, &record, sizeof record);
    return STATUS_OK;
}

result_status expert_post_prepare(const struct expert_join_description *join, uint64_t arena_byte_count, uint32_t kernel,
                                  struct kernel_launch *launch_out)
{
    static const char who[] = "expert_post_prepare";
    if (join == NULL || launch_out == NULL || kernel == BACKEND_NO_KERNEL) {
        REFUSE("%s: the description, the launch and a prepared kernel are needed", who);
        return STATUS_INVALID_ARGUMENT;
    }
    struct join_extent extent;
    struct range_list list = {.used = 0};
    if (!join_extent_read(who, join, 65535u, &extent)) {
        return STATUS_INVALID_ARGUMENT;
    }
    if (!extent.stores_sums) {
        REFUSE("%s: the post adds the stored row sums; this description stores none", who);
        return STATUS_INVALID_ARGUMENT;
    }
    list_join_ranges(&list, join, &extent);
    if (!list_holds(who, &list, arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct hyper_post_arguments record = {join->streams.byte_offset, join->post.byte_offset, join->comb.byte_offset,
                                                join->shared_output.byte_offset, join->row_sums.byte_offset, 1u, 0};
    launch_fill(launch_out, kernel, extent.row_blocks, join->row_count, 1, HYPER_PIECE_THREADS, 0, &record, sizeof record);
    return STATUS_OK;
}

/* the built instance of a slice count, or BUILT_INSTANCES */
static uint32_t instance_of_slices(uint32_t slice_count)
{
    for (uint32_t instance = 0; instance < BUILT_INSTANCES; instance++) {
        if (slice_counts[instance] == slice_count) {
            return instance;
        }
    }
    return BUILT_INSTANCES;
}

result_status expert_shared_join_prepare(const struct expert_shared_join_description *description, uint64_t arena_byte_count,
                                         const struct linear_kernels_record *linear_kernels, const struct expert_fused_kernels *kernels,
                                         struct kernel_launch *launch_out)
{
    static const char who[] = "expert_shared_join_prepare";
    if (description == NULL || linear_kernels == NULL || kernels == NULL || launch_out == NULL) {
        REFUSE("%s: description, both kernel records and the launch are needed", who);
        return STATUS_INVALID_ARGUMENT;
    }
    const struct expert_join_description *join = &description->join;
    /* The launch is the shared expert's down product with the join behind it. The product's own prepare function is asked
     * first, on a launch that is thrown away: what it refuses is refused here under its own line. */
    struct linear_trunk_quantized_description product;
    struct kernel_launch thrown_away;
    memset(&product, 0, sizeof product);
    product.matrix_count = 1;
    product.matrices[0] = description->down;
    product.outputs[0] = join->shared_output;
    product.codes = description->codes;
    product.exponents = description->exponents;
    product.operands = description->operands;
    product.row_count = join->row_count;
    const result_status product_status = linear_trunk_quantized_prepare(&product, arena_byte_count, linear_kernels, &thrown_away);
    if (product_status != STATUS_OK) {
        return product_status;
    }
    struct join_extent extent;
    const uint32_t instance = instance_of_slices(description->down.slice_count);
    if (!join_extent_read(who, join, LINEAR_MAXIMUM_ROWS, &extent)) {
        return STATUS_INVALID_ARGUMENT;
    }
    if (instance == BUILT_INSTANCES || kernels->shared_join[instance] == BACKEND_NO_KERNEL) {
        REFUSE("%s: no prepared kernel for a down product of %u slices", who, description->down.slice_count);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t inputs = description->down.shape.input_size, outputs = description->down.shape.output_size;
    if (outputs != extent.width) {
        REFUSE("%s: the down matrix writes rows of %u values into streams of %u", who, outputs, extent.width);
        return STATUS_INVALID_ARGUMENT;
    }
    struct range_list list = {.used = 0};
    list_range(&list, "down (the stored matrix)", description->down.stored, description->down.stored.byte_count, true);
    list_range(&list, "codes of the hidden rows", description->codes, linear_codes_byte_count(extent.rows, inputs), false);
    list_range(&list, "exponents of the hidden rows", description->exponents, linear_exponents_byte_count(extent.rows, inputs), false);
    list_range(&list, "operands of the hidden rows", description->operands, 0, false);
    list_join_ranges(&list, join, &extent);
    if (!list_holds(who, &list, arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct expert_shared_join_arguments record = {
        description->down.stored.byte_offset, description->codes.byte_offset, description->exponents.byte_offset,
        description->operands.byte_offset, join->shared_output.byte_offset, join->pair_output.byte_offset, join->streams.byte_offset,
        join->post.byte_offset, join->comb.byte_offset, extent.stores_sums ? join->row_sums.byte_offset : EXPERT_JOIN_NO_ROW_SUMS, inputs,
        join->row_count, join->pairs_per_row, join->width};
    const uint32_t strips = (outputs + TRUNK_STRIP_OUTPUTS - 1u) / TRUNK_STRIP_OUTPUTS;
    launch_fill(launch_out, kernels->shared_join[instance], strips, 1, 1, 64u * description->down.slice_count, 0, &record, sizeof record);
    return STATUS_OK;
}
