/*
 * linear.c -- load-time preparation of the FP4 routed experts and of the activation quantizer: the routed part of
 * the reference's source/linear.c (linear_kernels_prepare :292-311, linear_default_slice_count :567-593,
 * linear_quantize_prepare :1088-1120, linear_routed_experts_prepare :1263-1390, the byte counts :716-724).
 *
 *   launch      kernel                      grid                                  block        shared
 *   gate/up     expert_gate_up_<S>          (output_size / 16, jobs, 1)           128 S        static
 *   quantize    activation_quantize_entry   (ceil(width / 1024), pairs, 1)        256          0
 *   down        expert_down_<S>             (output_size / 16, jobs, 1)           64 S         static
 *   row sum     expert_row_sum_entry        (ceil(width / 2048), rows, 1)         256          0
 * A wavefront is 64 lanes, so a slice is a wavefront (gate with up: two); 16 slices would be a block of 2,048
 * threads, which the card does not run: the instances are 1, 2, 4 and 8.
 */
#include <inttypes.h>
#include <math.h>
#include <string.h>

#include "prepare_common.h"

#define ROW_SUM_BLOCK_OUTPUTS (EXPERT_ROW_SUM_CHANNELS * LINEAR_ELEMENT_THREADS) /* outputs a block of the row sum takes */
#define QUANTIZE_BLOCK_VALUES (4u * LINEAR_ELEMENT_THREADS) /* a thread of activation_quantize_entry takes four values */
#define LINEAR_STRIP_OUTPUTS 64u /* a block of the expert kernels: a strip of four tiles of 16 outputs */
static const uint32_t slice_counts[LINEAR_SLICE_INSTANCES] = {1u, 2u, 4u, 8u, 16u};
#define BUILT_INSTANCES 4u
#define MOST_ROWS 4096u /* rows of one call: a wide step's chunk */

uint64_t linear_values_byte_count(uint64_t vector_count, uint64_t width)
{
    return product_or_most(product_or_most(vector_count, width), 2u);
}
uint64_t linear_codes_byte_count(uint64_t vector_count, uint64_t width)
{
    return product_or_most(vector_count, width);
}
uint64_t linear_exponents_byte_count(uint64_t vector_count, uint64_t width)
{
    return product_or_most(vector_count, width / LINEAR_VALUES_PER_BLOCK);
}
uint64_t linear_sums_byte_count(uint64_t row_count, uint64_t width)
{
    return product_or_most(product_or_most(row_count, width), 4u);
}
uint64_t linear_jobs_byte_count(uint64_t job_count)
{
    return product_or_most(job_count, sizeof(struct expert_job_record));
}

result_status linear_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                     uint32_t arithmetic_class, struct linear_kernels_record *kernels_out)
{
    if (backend == NULL || backend->kernel_prepare == NULL || card == NULL || kernels_out == NULL ||
        arithmetic_class != ARITHMETIC_CLASS_GFX950) {
        REFUSE("the kernels of the linear: a missing argument, or a class other than %u", ARITHMETIC_CLASS_GFX950);
        return STATUS_INVALID_ARGUMENT;
    }
    struct linear_kernels_record kernels;
    memset(&kernels, 0xFF, sizeof kernels); /* every handle BACKEND_NO_KERNEL */
    result_status status = backend->kernel_prepare(card, KERNEL_FILE_ACTIVATION_QUANTIZE, KERNEL_ACTIVATION_QUANTIZE,
                                                   sizeof(struct activation_quantize_arguments), &kernels.activation_quantize);
    for (uint32_t instance = 0; status == STATUS_OK && instance < BUILT_INSTANCES; instance++) {
        char name[40];
        (void)snprintf(name, sizeof name, "%s%u", KERNEL_EXPERT_GATE_UP_STEM, slice_counts[instance]);
        status = backend->kernel_prepare(card, KERNEL_FILE_EXPERT_LINEAR, name, sizeof(struct expert_gate_up_arguments),
                                         &kernels.expert_gate_up[instance]);
        if (status == STATUS_OK) {
            (void)snprintf(name, sizeof name, "%s%u", KERNEL_EXPERT_DOWN_STEM, slice_counts[instance]);
            status = backend->kernel_prepare(card, KERNEL_FILE_EXPERT_LINEAR, name, sizeof(struct expert_down_arguments),
                                             &kernels.expert_down[instance]);
        }
    }
    for (uint32_t instance = 0; status == STATUS_OK && instance < BUILT_INSTANCES; instance++) {
        char name[48];
        (void)snprintf(name, sizeof name, "%se4m3_%u", KERNEL_EXPERT_GATE_UP_STEM, slice_counts[instance]);
        status = backend->kernel_prepare(card, KERNEL_FILE_EXPERT_LINEAR, name, sizeof(struct expert_gate_up_arguments),
                                         &kernels.expert_gate_up_e4m3[instance]);
        if (status == STATUS_OK) {
            (void)snprintf(name, sizeof name, "%se4m3_%u", KERNEL_EXPERT_DOWN_STEM, slice_counts[instance]);
            status = backend->kernel_prepare(card, KERNEL_FILE_EXPERT_LINEAR, name, sizeof(struct expert_down_arguments),
                                             &kernels.expert_down_e4m3[instance]);
        }
    }
    for (uint32_t instance = 0; status == STATUS_OK && instance < BUILT_INSTANCES; instance++) {
        char name[48];
        (void)snprintf(name, sizeof name, "%sb128_%u", KERNEL_EXPERT_GATE_UP_STEM, slice_counts[instance]);
        status = backend->kernel_prepare(card, KERNEL_FILE_EXPERT_LINEAR, name, sizeof(struct expert_gate_up_arguments),
                                         &kernels.expert_gate_up_b128[instance]);
        if (status == STATUS_OK) {
            (void)snprintf(name, sizeof name, "%sb128_%u", KERNEL_EXPERT_DOWN_STEM, slice_counts[instance]);
            status = backend->kernel_prepare(card, KERNEL_FILE_EXPERT_LINEAR, name, sizeof(struct expert_down_arguments),
                                             &kernels.expert_down_b128[instance]);
        }
    }
    for (uint32_t instance = 0; status == STATUS_OK && instance < BUILT_INSTANCES; instance++) {
        /* the same four families of the formats in gfx950's lane order */
        const struct {
            const char *stem, *infix;
            uint32_t record_bytes, *handle;
        } native[] = {
            {KERNEL_EXPERT_GATE_UP_STEM, "gfx950_", sizeof(struct expert_gate_up_arguments), &kernels.expert_gate_up_gfx950[instance]},
            {KERNEL_EXPERT_DOWN_STEM, "gfx950_", sizeof(struct expert_down_arguments), &kernels.expert_down_gfx950[instance]},
            {KERNEL_EXPERT_GATE_UP_STEM, "e4m3_gfx950_", sizeof(struct expert_gate_up_arguments), &kernels.expert_gate_up_e4m3_gfx950[instance]},
            {KERNEL_EXPERT_DOWN_STEM, "e4m3_gfx950_", sizeof(struct expert_down_arguments), &kernels.expert_down_e4m3_gfx950[instance]},
            {KERNEL_EXPERT_GATE_UP_STEM, "b128_gfx950_", sizeof(struct expert_gate_up_arguments), &kernels.expert_gate_up_b128_gfx950[instance]},
            {KERNEL_EXPERT_DOWN_STEM, "b128_gfx950_", sizeof(struct expert_down_arguments), &kernels.expert_down_b128_gfx950[instance]},
        };
        for (uint32_t k = 0; status == STATUS_OK && k < sizeof native / sizeof native[0]; k++) {
            char name[56];
            (void)snprintf(name, sizeof name, "%s%s%u", native[k].stem, native[k].infix, slice_counts[instance]);
            status = backend->kernel_prepare(card, KERNEL_FILE_EXPERT_LINEAR, name, native[k].record_bytes, native[k].handle);
        }
    }
    if (status == STATUS_OK) {
        status = backend->kernel_prepare(card, KERNEL_FILE_ACTIVATION_QUANTIZE, KERNEL_ACTIVATION_QUANTIZE_128,
                                         sizeof(struct activation_quantize_arguments), &kernels.activation_quantize_128);
    }
    if (status == STATUS_OK) {
        status = backend->kernel_prepare(card, KERNEL_FILE_EXPERT_LINEAR, KERNEL_EXPERT_ROW_SUM,
                                         sizeof(struct expert_row_sum_arguments), &kernels.expert_row_sum);
    }
    for (uint32_t instance = 0; status == STATUS_OK && instance < BUILT_INSTANCES; instance++) {
        char name[48];
        (void)snprintf(name, sizeof name, "%s%u", KERNEL_TRUNK_LINEAR_QUANTIZED_STEM, slice_counts[instance]);
        status = backend->kernel_prepare(card, KERNEL_FILE_TRUNK_LINEAR, name, sizeof(struct trunk_linear_quantized_arguments),
                                         &kernels.trunk_linear_quantized[instance]);
        if (status == STATUS_OK) {
            (void)snprintf(name, sizeof name, "%s%u", KERNEL_TRUNK_LINEAR_QUANTIZED_WIDE_STEM, slice_counts[instance]);
            status = backend->kernel_prepare(card, KERNEL_FILE_TRUNK_LINEAR, name, sizeof(struct trunk_linear_quantized_arguments),
                                             &kernels.trunk_linear_quantized_wide[instance]);
        }
    }
    if (status == STATUS_OK) {
        status = backend->kernel_prepare(card, KERNEL_FILE_TRUNK_LINEAR, KERNEL_TRUNK_LINEAR_QUANTIZED_INTERLEAVED,
                                         sizeof(struct trunk_linear_quantized_arguments), &kernels.trunk_linear_quantized_interleaved);
    }
    if (status == STATUS_OK) {
        status = backend->kernel_prepare(card, KERNEL_FILE_TRUNK_LINEAR, KERNEL_TRUNK_HIDDEN, sizeof(struct trunk_hidden_arguments),
                                         &kernels.trunk_hidden);
    }
    if (status != STATUS_OK) {
        REFUSE("the kernels of the linear: a kernel is not prepared: %s", status_text(status));
        return status;
    }
    *kernels_out = kernels;
    return STATUS_OK;
}

result_status linear_default_slice_count(enum linear_profile_code profile, enum linear_order_code order,
                                         enum linear_family_code family, const struct matrix_shape_record *shape,
                                         uint32_t arithmetic_class, uint32_t *slice_count_out)
{
    if (shape == NULL || slice_count_out == NULL || (profile != LINEAR_PROFILE_PRECISION && profile != LINEAR_PROFILE_SPEED) ||
        (order != LINEAR_ORDER_FIXED && order != LINEAR_ORDER_REFERENCE) || arithmetic_class != ARITHMETIC_CLASS_GFX950 ||
        (family != LINEAR_FAMILY_EXPERT_GATE_UP && family != LINEAR_FAMILY_EXPERT_DOWN) || shape->input_size == 0 ||
        shape->input_size % 128u != 0) {
        REFUSE("the default slice count: a profile, order, family, shape or class the table has no row for");
        return STATUS_INVALID_ARGUMENT;
    }
    uint32_t count = order == LINEAR_ORDER_REFERENCE ? 1u : family == LINEAR_FAMILY_EXPERT_GATE_UP ? 4u : 2u;
    while (count > shape->input_size / 128u) { /* at most one slice a K step of 128 inputs */
        count /= 2u;
    }
    *slice_count_out = count;
    return STATUS_OK;
}

result_status linear_quantize_prepare(const struct linear_quantize_description *description, uint64_t arena_byte_count,
                                      const struct linear_kernels_record *kernels, struct kernel_launch *launch_out)
{
    static const char what[] = "the activation quantizer";
    if (description == NULL || kernels == NULL || launch_out == NULL || kernels->activation_quantize == BACKEND_NO_KERNEL) {
        REFUSE("%s: a missing argument or an unprepared kernel", what);
        return STATUS_INVALID_ARGUMENT;
    }
    if (description->width == 0 || description->width % LINEAR_VALUES_PER_LOAD != 0 || description->row_count == 0 ||
        description->row_count > 65535u) {
        REFUSE("%s: a width that is 0 or no multiple of %u, or a row count of 0 or above 65535", what, LINEAR_VALUES_PER_LOAD);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t rows = description->row_count, width = description->width;
    const struct checked_range ranges[] = {
        {"the values", description->values, linear_values_byte_count(rows, width), false},
        {"the codes", description->codes, linear_codes_byte_count(rows, width), false},
        {"the exponents", description->exponents, linear_exponents_byte_count(rows, width), false},
        {"the operands", description->operands, linear_values_byte_count(rows, width), false},
    };
    if (!ranges_are_valid(what, ranges, 4, arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct activation_quantize_arguments record = {description->values.byte_offset, description->codes.byte_offset,
                                                         description->exponents.byte_offset,
                                                         description->operands.byte_offset, description->width, 0};
    launch_fill(launch_out, kernels->activation_quantize, (description->width + QUANTIZE_BLOCK_VALUES - 1u) / QUANTIZE_BLOCK_VALUES,
                description->row_count, 1, LINEAR_ELEMENT_THREADS, 0, &record, sizeof record);
    return STATUS_OK;
}

#define QUANTIZE_128_BLOCK_VALUES (4u * LINEAR_ELEMENT_THREADS) /* a thread of activation_quantize_128_entry takes four values */

result_status linear_quantize_128_prepare(const struct linear_quantize_description *description, uint64_t arena_byte_count,
                                          const struct linear_kernels_record *kernels, struct kernel_launch *launch_out)
{
    static const char what[] = "the activation quantizer of 128 values a scale";
    if (description == NULL || kernels == NULL || launch_out == NULL || kernels->activation_quantize_128 == BACKEND_NO_KERNEL) {
        REFUSE("%s: a missing argument or an unprepared kernel", what);
        return STATUS_INVALID_ARGUMENT;
    }
    if (description->width == 0 || description->width % 128u != 0 || description->row_count == 0 || description->row_count > 65535u) {
        REFUSE("%s: a width that is 0 or no multiple of 128, or a row count of 0 or above 65535", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t rows = description->row_count, width = description->width;
    const struct checked_range ranges[] = {
        {"the values", description->values, linear_values_byte_count(rows, width), false},
        {"the codes", description->codes, linear_codes_byte_count(rows, width), false},
        {"the scales", description->exponents, linear_exponents_byte_count(rows, width), false},
    };
    if (!ranges_are_valid(what, ranges, 3, arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct activation_quantize_arguments record = {description->values.byte_offset, description->codes.byte_offset,
                                                         description->exponents.byte_offset, description->operands.byte_offset,
                                                         description->width, 0};
    launch_fill(launch_out, kernels->activation_quantize_128, (description->width + QUANTIZE_128_BLOCK_VALUES - 1u) / QUANTIZE_128_BLOCK_VALUES,
                description->row_count, 1, LINEAR_ELEMENT_THREADS, 0, &record, sizeof record);
    return STATUS_OK;
}

static bool instance_of(uint32_t slice_count, uint32_t input_size, uint32_t *instance_out)
{
    for (uint32_t instance = 0; instance < BUILT_INSTANCES; instance++) {
        if (slice_counts[instance] == slice_count && slice_count <= input_size / 128u) {
            *instance_out = instance;
            return true;
        }
    }
    return false;
}

result_status linear_routed_experts_prepare(const struct linear_routed_experts_description *description,
                                            uint64_t arena_byte_count, const struct linear_kernels_record *kernels,
                                            struct kernel_launch *launches_out)
{
    static const char what[] = "the routed experts";
    if (description == NULL || kernels == NULL || launches_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const struct matrix_shape_record *gate_up = &description->gate_up_shape, *down = &description->down_shape;
    const struct weight_format_operations *format = weight_format_operations_of(description->weight_format);
    uint64_t gate_up_bytes = 0, down_bytes = 0;
    uint32_t gate_up_instance = 0, down_instance = 0;
    const bool block128 = description->weight_format == WEIGHT_FORMAT_E4M3_BLOCK128 || description->weight_format == WEIGHT_FORMAT_E4M3_BLOCK128_GFX950;
    const bool native = description->weight_format == WEIGHT_FORMAT_E2M1_GFX950 || description->weight_format == WEIGHT_FORMAT_E4M3_GFX950 ||
                        description->weight_format == WEIGHT_FORMAT_E4M3_BLOCK128_GFX950;
    const bool bytes = description->weight_format == WEIGHT_FORMAT_E4M3_SCALED || description->weight_format == WEIGHT_FORMAT_E4M3_GFX950 || block128;
    const bool nibbles = description->weight_format == WEIGHT_FORMAT_E2M1_SCALED || description->weight_format == WEIGHT_FORMAT_E2M1_GFX950;
    const uint32_t strip_outputs = bytes ? LINEAR_STRIP_OUTPUTS / 2u : LINEAR_STRIP_OUTPUTS;
    if (description->reserved_zero != 0 || (!nibbles && !bytes) || format == NULL ||
        format->stored_byte_count(gate_up, &gate_up_bytes) != STATUS_OK ||
        format->stored_byte_count(down, &down_bytes) != STATUS_OK || gate_up->input_size % 128u != 0 ||
        down->input_size % 128u != 0 || down->input_size != gate_up->output_size ||
        gate_up->output_size < strip_outputs || down->output_size < strip_outputs) {
        REFUSE("%s: matrices of format %u, %u or %u to %u in shapes it stores, inputs a multiple of 128, at least %u outputs, down "
               "reading what gate and up write", what, (uint32_t)WEIGHT_FORMAT_E2M1_SCALED, (uint32_t)WEIGHT_FORMAT_E4M3_SCALED,
               (uint32_t)WEIGHT_FORMAT_E4M3_BLOCK128, (uint32_t)WEIGHT_FORMAT_E4M3_BLOCK128_GFX950, strip_outputs);
        return STATUS_INVALID_ARGUMENT;
    }
    if (!instance_of(description->gate_up_slice_count, gate_up->input_size, &gate_up_instance) ||
        !instance_of(description->down_slice_count, down->input_size, &down_instance)) {
        REFUSE("%s: slice counts %u and %u: 1, 2, 4 or 8, at most one a 128 inputs", what,
               description->gate_up_slice_count, description->down_slice_count);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t *const gate_up_family = block128 && native ? kernels->expert_gate_up_b128_gfx950
                                           : block128        ? kernels->expert_gate_up_b128
                                           : native && bytes ? kernels->expert_gate_up_e4m3_gfx950
                                           : native          ? kernels->expert_gate_up_gfx950
                                           : bytes           ? kernels->expert_gate_up_e4m3
                                                             : kernels->expert_gate_up;
    const uint32_t *const down_family = block128 && native ? kernels->expert_down_b128_gfx950
                                        : block128        ? kernels->expert_down_b128
                                        : native && bytes ? kernels->expert_down_e4m3_gfx950
                                        : native          ? kernels->expert_down_gfx950
                                        : bytes           ? kernels->expert_down_e4m3
                                                          : kernels->expert_down;
    const uint32_t gate_up_kernel = gate_up_family[gate_up_instance], down_kernel = down_family[down_instance];
    const uint32_t quantize_kernel = block128 ? kernels->activation_quantize_128 : kernels->activation_quantize;
    const uint32_t quantize_block_values = block128 ? QUANTIZE_128_BLOCK_VALUES : QUANTIZE_BLOCK_VALUES;
    if (gate_up_kernel == BACKEND_NO_KERNEL || down_kernel == BACKEND_NO_KERNEL ||
        quantize_kernel == BACKEND_NO_KERNEL || kernels->expert_row_sum == BACKEND_NO_KERNEL) {
        REFUSE("%s: a kernel of the chain is not prepared", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t rows = description->row_count, pairs = rows * description->pairs_per_row;
    if (rows == 0 || rows > MOST_ROWS || description->pairs_per_row == 0 || pairs > UINT32_MAX || description->job_count == 0 ||
        description->job_count > 65535u || pairs > 65535u || !(description->activation_limit > 0.0f)) {
        REFUSE("%s: 1 to %u rows, pairs and jobs from 1 to 65535, an activation limit above zero", what, MOST_ROWS);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t H = gate_up->input_size, I = gate_up->output_size, O = down->output_size;
    const struct checked_range ranges[] = {
        {"the job table", description->jobs, linear_jobs_byte_count(description->job_count), false},
        {"the experts' matrices", description->expert_weights, gate_up_bytes > down_bytes ? gate_up_bytes : down_bytes, false},
        {"the rows' codes", description->codes, linear_codes_byte_count(rows, H), false},
        {"the rows' exponents", description->exponents, linear_exponents_byte_count(rows, H), false},
        {"the rows' operands", description->operands, 0, false},
        {"the hidden values", description->hidden, linear_values_byte_count(pairs, I), false},
        {"the hidden codes", description->hidden_codes, linear_codes_byte_count(pairs, I), false},
        {"the hidden exponents", description->hidden_exponents, linear_exponents_byte_count(pairs, I), false},
        {"the hidden operands", description->hidden_operands, linear_values_byte_count(pairs, I), false},
        {"the pair outputs", description->pair_output, linear_values_byte_count(pairs, O), false},
        {"the row outputs", description->row_output, linear_sums_byte_count(rows, O), false},
    };
    if (!ranges_are_valid(what, ranges, sizeof ranges / sizeof ranges[0], arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct expert_gate_up_arguments gate_up_record = {
        description->jobs.byte_offset, description->codes.byte_offset, description->exponents.byte_offset,
        description->operands.byte_offset, description->hidden.byte_offset, gate_up->output_size, gate_up->input_size,
        (uint32_t)pairs, description->pairs_per_row, description->activation_limit, 0};
    const struct activation_quantize_arguments quantize_record = {
        description->hidden.byte_offset, description->hidden_codes.byte_offset, description->hidden_exponents.byte_offset,
        description->hidden_operands.byte_offset, gate_up->output_size, 0};
    const struct expert_down_arguments down_record = {
        description->jobs.byte_offset, description->hidden_codes.byte_offset, description->hidden_exponents.byte_offset,
        description->hidden_operands.byte_offset, description->pair_output.byte_offset, down->output_size, down->input_size,
        (uint32_t)pairs, 0};
    const struct expert_row_sum_arguments row_sum_record = {description->pair_output.byte_offset,
                                                            description->row_output.byte_offset, down->output_size,
                                                            description->pairs_per_row};
    struct kernel_launch launches[LINEAR_ROUTED_EXPERTS_LAUNCH_COUNT];
    launch_fill(&launches[LINEAR_ROUTED_EXPERTS_GATE_UP], gate_up_kernel,
                (gate_up->output_size + strip_outputs - 1u) / strip_outputs,
                description->job_count, 1, 64u * description->gate_up_slice_count, 0, &gate_up_record, sizeof gate_up_record);
    launch_fill(&launches[LINEAR_ROUTED_EXPERTS_QUANTIZE], quantize_kernel,
                (gate_up->output_size + quantize_block_values - 1u) / quantize_block_values, (uint32_t)pairs, 1,
                LINEAR_ELEMENT_THREADS, 0, &quantize_record, sizeof quantize_record);
    launch_fill(&launches[LINEAR_ROUTED_EXPERTS_DOWN], down_kernel,
                (down->output_size + strip_outputs - 1u) / strip_outputs, description->job_count, 1, 64u * description->down_slice_count, 0, &down_record, sizeof down_record);
    launch_fill(&launches[LINEAR_ROUTED_EXPERTS_ROW_SUM], kernels->expert_row_sum,
                (down->output_size + ROW_SUM_BLOCK_OUTPUTS - 1u) / ROW_SUM_BLOCK_OUTPUTS, (uint32_t)rows, 1,
                LINEAR_ELEMENT_THREADS, 0, &row_sum_record, sizeof row_sum_record);
    memcpy(launches_out, launches, sizeof launches);
    return STATUS_OK;
}

/*
 * The shared expert: trunk products of quantized rows by E4M3_SCALED matrices (the reference's source/linear.c:
 * linear_trunk_quantized_prepare, linear_shared_expert_prepare :1392-1506).
 *
 *   rows      kernel                                  grid                                             block   LDS
 *   1..8      trunk_linear_quantized_<S>              (strips of both matrices, 1, 1)                  64 S    static
 *   9..       trunk_linear_quantized_wide_<S>         (strips x n, 1, 1), n = groups of 8 rows or 1    64 S    static
 *   9..       trunk_linear_quantized_interleaved_1    (blocks of both matrices, ceil(rows / 64), 1)    256     TRUNK_INTERLEAVED_WINDOW_BYTES
 *   hidden    trunk_hidden_entry                      (ceil(width / 2048), rows, 1)                    256     0
 * strip = TRUNK_STRIP_OUTPUTS outputs of one matrix, block = TRUNK_INTERLEAVED_BLOCK_OUTPUTS.
 */
static bool trunk_matrix_is_valid(const char *what, const struct linear_matrix *matrix, uint64_t *bytes_out, uint32_t *instance_out)
{
    const struct weight_format_operations *format = weight_format_operations_of(matrix->weight_format);
    if (matrix->weight_format != WEIGHT_FORMAT_E4M3_SCALED || format == NULL || matrix->reserved_zero != 0 ||
        format->stored_byte_count(&matrix->shape, bytes_out) != STATUS_OK || matrix->shape.input_size % 128u != 0 ||
        matrix->shape.output_size < TRUNK_STRIP_OUTPUTS || matrix->shape.output_size % 16u != 0) {
        REFUSE("%s: a matrix of format %u in a shape it stores, inputs a multiple of 128, outputs a multiple of 16 and at least %u",
               what, (uint32_t)WEIGHT_FORMAT_E4M3_SCALED, TRUNK_STRIP_OUTPUTS);
        return false;
    }
    if (!instance_of(matrix->slice_count, matrix->shape.input_size, instance_out)) {
        REFUSE("%s: a slice count of %u: 1, 2, 4 or 8, at most one a 128 inputs", what, matrix->slice_count);
        return false;
    }
    if ((uint32_t)matrix->wide_form >= (uint32_t)LINEAR_WIDE_FORM_COUNT) {
        REFUSE("%s: a wide form of %u", what, (uint32_t)matrix->wide_form);
        return false;
    }
    return true;
}

/* the launch of a trunk product whose description is checked: thin up to LINEAR_MAXIMUM_ROWS rows, else the
 * first matrix's wide form; false where that form's kernel is not prepared or takes no such matrix */
static bool trunk_launch_fill(const char *what, struct kernel_launch *launch, const struct linear_kernels_record *kernels,
                              uint32_t instance, const struct linear_matrix *matrices, uint32_t matrix_count,
                              const struct linear_range *codes, const struct linear_range *exponents,
                              const struct linear_range *operands, const struct linear_range *outputs, uint32_t row_count)
{
    struct trunk_linear_quantized_arguments record;
    memset(&record, 0, sizeof record);
    uint32_t strips = 0, blocks = 0;
    for (uint32_t m = 0; m < matrix_count; m++) {
        record.weights_offset[m] = matrices[m].stored.byte_offset;
        record.output_offset[m] = outputs[m].byte_offset;
        record.output_size[m] = matrices[m].shape.output_size;
        strips += (matrices[m].shape.output_size + TRUNK_STRIP_OUTPUTS - 1u) / TRUNK_STRIP_OUTPUTS;
        blocks += (matrices[m].shape.output_size + TRUNK_INTERLEAVED_BLOCK_OUTPUTS - 1u) / TRUNK_INTERLEAVED_BLOCK_OUTPUTS;
    }
    record.codes_offset = codes->byte_offset;
    record.exponents_offset = exponents->byte_offset;
    record.operands_offset = operands->byte_offset;
    record.input_size = matrices[0].shape.input_size;
    record.row_count = row_count;
    const uint32_t threads = 64u * matrices[0].slice_count;
    const enum linear_wide_form form = matrices[0].wide_form;
    uint32_t kernel;
    if (row_count <= LINEAR_MAXIMUM_ROWS) {
        kernel = kernels->trunk_linear_quantized[instance];
        launch_fill(launch, kernel, strips, 1, 1, threads, 0, &record, sizeof record);
    } else if (form == LINEAR_WIDE_GROUP_BLOCKS || form == LINEAR_WIDE_TILE_BLOCKS) {
        const uint32_t groups = (row_count + LINEAR_MAXIMUM_ROWS - 1u) / LINEAR_MAXIMUM_ROWS;
        kernel = kernels->trunk_linear_quantized_wide[instance];
        launch_fill(launch, kernel, strips * (form == LINEAR_WIDE_GROUP_BLOCKS ? groups : 1u), 1, 1, threads, 0, &record, sizeof record);
    } else {
        if (matrices[0].slice_count != 1u) {
            REFUSE("%s: the interleaved form takes a matrix of one slice, not %u", what, matrices[0].slice_count);
            return false;
        }
        kernel = kernels->trunk_linear_quantized_interleaved;
        launch_fill(launch, kernel, blocks, (row_count + TRUNK_INTERLEAVED_ROWS - 1u) / TRUNK_INTERLEAVED_ROWS, 1, WIDE_BLOCK_THREADS,
                    TRUNK_INTERLEAVED_WINDOW_BYTES, &record, sizeof record);
    }
    if (kernel == BACKEND_NO_KERNEL) {
        REFUSE("%s: the kernel of its rows and form is not prepared", what);
        return false;
    }
    return true;
}

result_status linear_trunk_quantized_prepare(const struct linear_trunk_quantized_description *description, uint64_t arena_byte_count,
                                             const struct linear_kernels_record *kernels, struct kernel_launch *launch_out)
{
    static const char what[] = "a trunk product of quantized rows";
    if (description == NULL || kernels == NULL || launch_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    if (description->matrix_count == 0 || description->matrix_count > LINEAR_MERGED_MATRICES || description->row_count == 0 ||
        description->row_count > LINEAR_TRUNK_MOST_ROWS) {
        REFUSE("%s: one or two matrices, 1 to %u rows", what, LINEAR_TRUNK_MOST_ROWS);
        return STATUS_INVALID_ARGUMENT;
    }
    uint64_t bytes[LINEAR_MERGED_MATRICES] = {0, 0};
    uint32_t instance = 0;
    const struct linear_matrix *first = &description->matrices[0];
    for (uint32_t m = 0; m < description->matrix_count; m++) {
        const struct linear_matrix *matrix = &description->matrices[m];
        if (!trunk_matrix_is_valid(what, matrix, &bytes[m], &instance)) {
            return STATUS_INVALID_ARGUMENT;
        }
        if (matrix->shape.input_size != first->shape.input_size || matrix->slice_count != first->slice_count ||
            matrix->wide_form != first->wide_form) {
            REFUSE("%s: two matrices of one launch are of one input size, slice count and wide form", what);
            return STATUS_INVALID_ARGUMENT;
        }
    }
    const uint64_t rows = description->row_count, inputs = first->shape.input_size;
    struct checked_range ranges[3 + 2 * LINEAR_MERGED_MATRICES] = {
        {"the rows' codes", description->codes, linear_codes_byte_count(rows, inputs), false},
        {"the rows' exponents", description->exponents, linear_exponents_byte_count(rows, inputs), false},
        {"the rows' operands", description->operands, 0, false},
    };
    uint32_t count = 3;
    for (uint32_t m = 0; m < description->matrix_count; m++) {
        ranges[count++] = (struct checked_range){"a matrix", description->matrices[m].stored, bytes[m], true};
        ranges[count++] = (struct checked_range){"an output", description->outputs[m],
                                                 linear_values_byte_count(rows, description->matrices[m].shape.output_size), false};
    }
    if (!ranges_are_valid(what, ranges, count, arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    struct kernel_launch launch;
    if (!trunk_launch_fill(what, &launch, kernels, instance, description->matrices, description->matrix_count, &description->codes,
                           &description->exponents, &description->operands, description->outputs, description->row_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    *launch_out = launch;
    return STATUS_OK;
}

result_status linear_shared_expert_prepare(const struct linear_shared_expert_description *description, uint64_t arena_byte_count,
                                           const struct linear_kernels_record *kernels, struct kernel_launch *launches_out)
{
    static const char what[] = "the shared expert";
    if (description == NULL || kernels == NULL || launches_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const struct linear_matrix gate_up[LINEAR_MERGED_MATRICES] = {description->gate, description->up};
    const struct linear_range gate_up_outputs[LINEAR_MERGED_MATRICES] = {description->gate_output, description->up_output};
    const struct matrix_shape_record *gate = &description->gate.shape, *up = &description->up.shape, *down = &description->down.shape;
    uint64_t gate_bytes = 0, up_bytes = 0, down_bytes = 0;
    uint32_t gate_up_instance = 0, up_instance = 0, down_instance = 0;
    if (!trunk_matrix_is_valid(what, &description->gate, &gate_bytes, &gate_up_instance) ||
        !trunk_matrix_is_valid(what, &description->up, &up_bytes, &up_instance) ||
        !trunk_matrix_is_valid(what, &description->down, &down_bytes, &down_instance)) {
        return STATUS_INVALID_ARGUMENT;
    }
    if (up->output_size != gate->output_size || up->input_size != gate->input_size || up_instance != gate_up_instance ||
        description->up.wide_form != description->gate.wide_form || down->input_size != gate->output_size) {
        REFUSE("%s: up is of gate's shape, slice count and wide form; down reads what they write", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t rows = description->row_count;
    if (rows == 0 || rows > LINEAR_TRUNK_MOST_ROWS || !(description->activation_limit > 0.0f)) {
        REFUSE("%s: 1 to %u rows, an activation limit above zero", what, LINEAR_TRUNK_MOST_ROWS);
        return STATUS_INVALID_ARGUMENT;
    }
    if (kernels->trunk_hidden == BACKEND_NO_KERNEL || kernels->activation_quantize == BACKEND_NO_KERNEL) {
        REFUSE("%s: a kernel of the chain is not prepared", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t H = gate->input_size, I = gate->output_size, hidden_bytes = linear_values_byte_count(rows, I);
    const struct checked_range ranges[] = {
        {"gate", description->gate.stored, gate_bytes, true},
        {"up", description->up.stored, up_bytes, true},
        {"down", description->down.stored, down_bytes, true},
        {"the rows' codes", description->codes, linear_codes_byte_count(rows, H), false},
        {"the rows' exponents", description->exponents, linear_exponents_byte_count(rows, H), false},
        {"the rows' operands", description->operands, 0, false},
        {"the output of gate", description->gate_output, hidden_bytes, false},
        {"the output of up", description->up_output, hidden_bytes, false},
        {"the hidden values", description->hidden, hidden_bytes, false},
        {"the hidden codes", description->hidden_codes, linear_codes_byte_count(rows, I), false},
        {"the hidden exponents", description->hidden_exponents, linear_exponents_byte_count(rows, I), false},
        {"the hidden operands", description->hidden_operands, hidden_bytes, false},
        {"the output", description->output, linear_values_byte_count(rows, down->output_size), false},
    };
    if (!ranges_are_valid(what, ranges, sizeof ranges / sizeof ranges[0], arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    struct kernel_launch launches[LINEAR_SHARED_EXPERT_LAUNCH_COUNT];
    if (!trunk_launch_fill(what, &launches[LINEAR_SHARED_EXPERT_GATE_UP], kernels, gate_up_instance, gate_up, LINEAR_MERGED_MATRICES,
                           &description->codes, &description->exponents, &description->operands, gate_up_outputs, description->row_count) ||
        !trunk_launch_fill(what, &launches[LINEAR_SHARED_EXPERT_DOWN], kernels, down_instance, &description->down, 1,
                           &description->hidden_codes, &description->hidden_exponents, &description->hidden_operands,
                           &description->output, description->row_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct trunk_hidden_arguments hidden_record = {description->gate_output.byte_offset, description->up_output.byte_offset,
                                                         description->hidden.byte_offset, gate->output_size, description->activation_limit};
    const struct activation_quantize_arguments quantize_record = {
        description->hidden.byte_offset, description->hidden_codes.byte_offset, description->hidden_exponents.byte_offset,
        description->hidden_operands.byte_offset, gate->output_size, 0};
    launch_fill(&launches[LINEAR_SHARED_EXPERT_HIDDEN], kernels->trunk_hidden,
                (gate->output_size + ROW_SUM_BLOCK_OUTPUTS - 1u) / ROW_SUM_BLOCK_OUTPUTS, description->row_count, 1,
                LINEAR_ELEMENT_THREADS, 0, &hidden_record, sizeof hidden_record);
    launch_fill(&launches[LINEAR_SHARED_EXPERT_QUANTIZE], kernels->activation_quantize,
                (gate->output_size + QUANTIZE_BLOCK_VALUES - 1u) / QUANTIZE_BLOCK_VALUES, description->row_count, 1,
                LINEAR_ELEMENT_THREADS, 0, &quantize_record, sizeof quantize_record);
    memcpy(launches_out, launches, sizeof launches);
    return STATUS_OK;
}

/*
 * The wide form: a grouped GEMM over the tiles of a wide select.
 *
 *   launch      kernel                       grid                                       block   dynamic LDS
 *   gate/up     wide_expert_gate_up_1        (ceil(I / 128), tile_count, 1)             256     WIDE_GATE_UP_WINDOW_BYTES
 *   down        wide_expert_down_1           (ceil(H / (4 strips)), tile_count, 1)      256     WIDE_DOWN_WINDOW_BYTES
 *   row sum     expert_row_sum_entry         (ceil(H / 2048), rows, 1)                  256
 * strip = 64 outputs of E2M1 weights, 32 of E4M3.
 */
#define WIDE_MOST_ROWS 16384u

result_status linear_wide_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                          uint32_t arithmetic_class, struct linear_wide_kernels_record *kernels_out)
{
    if (backend == NULL || backend->kernel_prepare == NULL || card == NULL || kernels_out == NULL ||
        arithmetic_class != ARITHMETIC_CLASS_GFX950) {
        REFUSE("the kernels of the wide linear: a missing argument, or a class other than %u", ARITHMETIC_CLASS_GFX950);
        return STATUS_INVALID_ARGUMENT;
    }
    static const struct {
        const char *name;
        uint32_t record_bytes;
    } wanted[6] = {{KERNEL_WIDE_EXPERT_GATE_UP_STEM "1", sizeof(struct wide_expert_gate_up_arguments)},
                   {KERNEL_WIDE_EXPERT_DOWN_STEM "1", sizeof(struct wide_expert_down_arguments)},
                   {KERNEL_WIDE_EXPERT_GATE_UP_STEM "e4m3_1", sizeof(struct wide_expert_gate_up_arguments)},
                   {KERNEL_WIDE_EXPERT_DOWN_STEM "e4m3_1", sizeof(struct wide_expert_down_arguments)},
                   {KERNEL_WIDE_EXPERT_GATE_UP_STEM "b128_1", sizeof(struct wide_expert_gate_up_arguments)},
                   {KERNEL_WIDE_EXPERT_DOWN_STEM "b128_1", sizeof(struct wide_expert_down_arguments)}};
    uint32_t handles[6];
    _Static_assert(sizeof(struct linear_wide_kernels_record) == sizeof handles, "a handle a member, in the members' order");
    for (uint32_t i = 0; i < 6u; i++) {
        const result_status status = backend->kernel_prepare(card, KERNEL_FILE_WIDE_LINEAR, wanted[i].name, wanted[i].record_bytes, &handles[i]);
        if (status != STATUS_OK) {
            REFUSE("the kernels of the wide linear: %s is not prepared: %s", wanted[i].name, status_text(status));
            return status;
        }
    }
    memcpy(kernels_out, handles, sizeof handles);
    return STATUS_OK;
}

/* block128: the launches of WEIGHT_FORMAT_E4M3_BLOCK128 experts (four: the hidden vectors' quantizer is a launch of its
 * own between the products); else those of the reference's formats (three) */
static result_status wide_experts_prepare(const struct linear_wide_experts_description *description, uint64_t arena_byte_count,
                                          const struct linear_kernels_record *linear_kernels,
                                          const struct linear_wide_kernels_record *kernels, const struct linear_native_kernels_record *native_kernels,
                                          bool block128, struct kernel_launch *launches_out)
{
    const bool native = native_kernels != NULL; /* experts in gfx950's lane order: the same launches by the native kernels */
    const char *what = native ? "the wide routed experts in gfx950's lane order" : block128 ? "the wide routed experts of float32 block scales" : "the wide routed experts";
    if (description == NULL || linear_kernels == NULL || (kernels == NULL && !native) || launches_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const struct linear_routed_experts_description *experts = &description->experts;
    const struct matrix_shape_record *gate_up = &experts->gate_up_shape, *down = &experts->down_shape;
    const struct weight_format_operations *format = weight_format_operations_of(experts->weight_format);
    if (block128 != (experts->weight_format == (native ? WEIGHT_FORMAT_E4M3_BLOCK128_GFX950 : WEIGHT_FORMAT_E4M3_BLOCK128))) {
        REFUSE("%s: a weight format of %u", what, (uint32_t)experts->weight_format);
        return STATUS_INVALID_ARGUMENT;
    }
    const enum weight_format_code nibbles_format = native ? WEIGHT_FORMAT_E2M1_GFX950 : WEIGHT_FORMAT_E2M1_SCALED;
    const enum weight_format_code bytes_format = native ? WEIGHT_FORMAT_E4M3_GFX950 : WEIGHT_FORMAT_E4M3_SCALED;
    const bool bytes = experts->weight_format == bytes_format || block128;
    const uint32_t strip_outputs = bytes ? LINEAR_STRIP_OUTPUTS / 2u : LINEAR_STRIP_OUTPUTS;
    uint64_t gate_up_bytes = 0, down_bytes = 0;
    if (description->reserved_zero != 0 || experts->reserved_zero != 0 || (experts->weight_format != nibbles_format && !bytes) ||
        format == NULL || format->stored_byte_count(gate_up, &gate_up_bytes) != STATUS_OK ||
        format->stored_byte_count(down, &down_bytes) != STATUS_OK || gate_up->input_size % 128u != 0 || down->input_size % 128u != 0 ||
        down->input_size != gate_up->output_size || gate_up->output_size < strip_outputs || down->output_size < strip_outputs ||
        gate_up->output_size % 32u != 0) {
        REFUSE("%s: matrices of format %u or %u in shapes it stores, inputs a multiple of 128, gate/up outputs of 32, at least %u outputs, "
               "down reading what gate and up write", what, (uint32_t)nibbles_format, (uint32_t)bytes_format, strip_outputs);
        return STATUS_INVALID_ARGUMENT;
    }
    if (experts->gate_up_slice_count != 1u || experts->down_slice_count != 1u) {
        REFUSE("%s: slice counts %u and %u: the wide products are built for one slice", what, experts->gate_up_slice_count,
               experts->down_slice_count);
        return STATUS_INVALID_ARGUMENT;
    }
    uint32_t gate_up_kernel, down_kernel, gate_up_window, down_window;
    if (native) {
        gate_up_kernel = block128 ? native_kernels->native_expert_gate_up_b128
                         : bytes  ? native_kernels->native_expert_gate_up_e4m3
                                  : native_kernels->native_expert_gate_up;
        down_kernel = block128 ? native_kernels->native_expert_down_b128 : bytes ? native_kernels->native_expert_down_e4m3 : native_kernels->native_expert_down;
        gate_up_window = down_window = bytes ? NATIVE_WINDOW_BYTES(NATIVE_E4M3_COLUMN_BLOCKS, NATIVE_E4M3_STAGES)
                                             : NATIVE_WINDOW_BYTES(NATIVE_E2M1_COLUMN_BLOCKS, NATIVE_E2M1_STAGES);
    } else {
        gate_up_kernel = block128 ? kernels->wide_expert_gate_up_b128 : bytes ? kernels->wide_expert_gate_up_e4m3 : kernels->wide_expert_gate_up;
        down_kernel = block128 ? kernels->wide_expert_down_b128 : bytes ? kernels->wide_expert_down_e4m3 : kernels->wide_expert_down;
        gate_up_window = bytes ? WIDE_GATE_UP_E4M3_WINDOW_BYTES : WIDE_GATE_UP_WINDOW_BYTES;
        down_window = bytes ? WIDE_DOWN_E4M3_WINDOW_BYTES : WIDE_DOWN_WINDOW_BYTES;
    }
    if (gate_up_kernel == BACKEND_NO_KERNEL || down_kernel == BACKEND_NO_KERNEL || linear_kernels->expert_row_sum == BACKEND_NO_KERNEL ||
        (block128 && linear_kernels->activation_quantize_128 == BACKEND_NO_KERNEL)) {
        REFUSE("%s: a kernel of the chain is not prepared", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t rows = experts->row_count, pairs = rows * experts->pairs_per_row;
    if (rows == 0 || rows > WIDE_MOST_ROWS || experts->pairs_per_row == 0 || pairs > UINT32_MAX || description->tile_count == 0 ||
        description->tile_count > 65535u || !(experts->activation_limit > 0.0f)) {
        REFUSE("%s: 1 to %u rows, 1 to 65535 tiles, an activation limit above zero", what, WIDE_MOST_ROWS);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t H = gate_up->input_size, I = gate_up->output_size, O = down->output_size;
    const struct checked_range ranges[] = {
        {"the tiles", description->tiles, (uint64_t)description->tile_count * sizeof(struct wide_expert_tile), false},
        {"the sorted pairs", description->pairs, pairs * sizeof(struct wide_pair), false},
        {"the experts' matrices", experts->expert_weights, gate_up_bytes > down_bytes ? gate_up_bytes : down_bytes, false},
        {"the rows' codes", experts->codes, linear_codes_byte_count(rows, H), false},
        {"the rows' exponents", experts->exponents, linear_exponents_byte_count(rows, H), false},
        {"the rows' operands", experts->operands, 0, false},
        {"the hidden codes", experts->hidden_codes, linear_codes_byte_count(pairs, I), false},
        {"the hidden exponents", experts->hidden_exponents, linear_exponents_byte_count(pairs, I), false},
        {"the hidden operands", experts->hidden_operands, linear_values_byte_count(pairs, I), false},
        {"the pair outputs", experts->pair_output, linear_values_byte_count(pairs, O), false},
        {"the row outputs", experts->row_output, linear_sums_byte_count(rows, O), false},
    };
    if (!ranges_are_valid(what, ranges, sizeof ranges / sizeof ranges[0], arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct wide_expert_gate_up_arguments gate_up_record = {
        description->tiles.byte_offset, description->pairs.byte_offset, experts->codes.byte_offset, experts->exponents.byte_offset,
        experts->operands.byte_offset, experts->hidden_codes.byte_offset, experts->hidden_exponents.byte_offset,
        experts->hidden_operands.byte_offset, gate_up->output_size, gate_up->input_size, description->tile_count,
        experts->pairs_per_row, experts->activation_limit, (uint32_t)pairs};
    const struct wide_expert_down_arguments down_record = {
        description->tiles.byte_offset, description->pairs.byte_offset, experts->hidden_codes.byte_offset,
        experts->hidden_exponents.byte_offset, experts->hidden_operands.byte_offset, experts->pair_output.byte_offset,
        down->output_size, down->input_size, description->tile_count, (uint32_t)pairs};
    const struct expert_row_sum_arguments row_sum_record = {experts->pair_output.byte_offset, experts->row_output.byte_offset,
                                                            down->output_size, experts->pairs_per_row};
    const uint32_t block_outputs = 4u * strip_outputs;
    const uint32_t gate_up_outputs = bytes ? WIDE_GATE_UP_E4M3_BLOCK_OUTPUTS : WIDE_GATE_UP_BLOCK_OUTPUTS;
    struct kernel_launch launches[LINEAR_WIDE_EXPERTS_BLOCK128_LAUNCH_COUNT];
    uint32_t at = 0;
    launch_fill(&launches[at++], gate_up_kernel,
                (gate_up->output_size + gate_up_outputs - 1u) / gate_up_outputs, description->tile_count, 1,
                WIDE_BLOCK_THREADS, gate_up_window, &gate_up_record, sizeof gate_up_record);
    if (block128) { /* the hidden values, which the gate/up launch left where the operands go, to their codes and scales */
        const struct activation_quantize_arguments quantize_record = {
            experts->hidden_operands.byte_offset, experts->hidden_codes.byte_offset, experts->hidden_exponents.byte_offset,
            experts->hidden_operands.byte_offset, gate_up->output_size, 0};
        launch_fill(&launches[at++], linear_kernels->activation_quantize_128,
                    (gate_up->output_size + QUANTIZE_128_BLOCK_VALUES - 1u) / QUANTIZE_128_BLOCK_VALUES, (uint32_t)pairs, 1,
                    LINEAR_ELEMENT_THREADS, 0, &quantize_record, sizeof quantize_record);
    }
    launch_fill(&launches[at++], down_kernel, (down->output_size + block_outputs - 1u) / block_outputs,
                description->tile_count, 1, WIDE_BLOCK_THREADS, down_window, &down_record, sizeof down_record);
    launch_fill(&launches[at++], linear_kernels->expert_row_sum,
                (down->output_size + ROW_SUM_BLOCK_OUTPUTS - 1u) / ROW_SUM_BLOCK_OUTPUTS, (uint32_t)rows, 1, LINEAR_ELEMENT_THREADS, 0,
                &row_sum_record, sizeof row_sum_record);
    memcpy(launches_out, launches, at * sizeof launches[0]);
    return STATUS_OK;
}

result_status linear_wide_experts_prepare(const struct linear_wide_experts_description *description, uint64_t arena_byte_count,
                                          const struct linear_kernels_record *linear_kernels,
                                          const struct linear_wide_kernels_record *kernels, struct kernel_launch *launches_out)
{
    return wide_experts_prepare(description, arena_byte_count, linear_kernels, kernels, NULL, false, launches_out);
}

result_status linear_wide_experts_block128_prepare(const struct linear_wide_experts_description *description, uint64_t arena_byte_count,
                                                   const struct linear_kernels_record *linear_kernels,
                                                   const struct linear_wide_kernels_record *kernels, struct kernel_launch *launches_out)
{
    return wide_experts_prepare(description, arena_byte_count, linear_kernels, kernels, NULL, true, launches_out);
}

/* ---- the same launches for experts stored in gfx950's lane order ---- */

result_status linear_native_kernels_prepare(const struct backend_operations *backend, struct device_card *card, uint32_t arithmetic_class,
                                            struct linear_native_kernels_record *kernels_out)
{
    if (backend == NULL || backend->kernel_prepare == NULL || card == NULL || kernels_out == NULL || arithmetic_class != ARITHMETIC_CLASS_GFX950) {
        REFUSE("linear_native_kernels_prepare: a backend, a card of class %u and a record to fill are needed", ARITHMETIC_CLASS_GFX950);
        return STATUS_INVALID_ARGUMENT;
    }
    static const struct {
        const char *name;
        uint32_t record_bytes;
    } wanted[6] = {{KERNEL_NATIVE_EXPERT_GATE_UP_STEM "1", sizeof(struct wide_expert_gate_up_arguments)},
                   {KERNEL_NATIVE_EXPERT_DOWN_STEM "1", sizeof(struct wide_expert_down_arguments)},
                   {KERNEL_NATIVE_EXPERT_GATE_UP_STEM "e4m3_1", sizeof(struct wide_expert_gate_up_arguments)},
                   {KERNEL_NATIVE_EXPERT_DOWN_STEM "e4m3_1", sizeof(struct wide_expert_down_arguments)},
                   {KERNEL_NATIVE_EXPERT_GATE_UP_STEM "b128_1", sizeof(struct wide_expert_gate_up_arguments)},
                   {KERNEL_NATIVE_EXPERT_DOWN_STEM "b128_1", sizeof(struct wide_expert_down_arguments)}};
    uint32_t handles[6];
    _Static_assert(sizeof(struct linear_native_kernels_record) == sizeof handles, "a handle a member, in the members' order");
    for (uint32_t i = 0; i < 6u; i++) {
        const result_status status = backend->kernel_prepare(card, KERNEL_FILE_NATIVE_LINEAR, wanted[i].name, wanted[i].record_bytes, &handles[i]);
        if (status != STATUS_OK) {
            REFUSE("linear_native_kernels_prepare: %s: %s", wanted[i].name, status_text(status));
            return status;
        }
    }
    memcpy(kernels_out, handles, sizeof handles);
    return STATUS_OK;
}

result_status linear_native_experts_prepare(const struct linear_wide_experts_description *description, uint64_t arena_byte_count,
                                            const struct linear_kernels_record *linear_kernels,
                                            const struct linear_native_kernels_record *kernels, struct kernel_launch *launches_out)
{
    if (kernels == NULL) {
        REFUSE("linear_native_experts_prepare: the native kernels' record is needed");
        return STATUS_INVALID_ARGUMENT;
    }
    const bool block128 = description != NULL && description->experts.weight_format == WEIGHT_FORMAT_E4M3_BLOCK128_GFX950;
    return wide_experts_prepare(description, arena_byte_count, linear_kernels, NULL, kernels, block128, launches_out);
}
