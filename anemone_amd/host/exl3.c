/*
 * exl3.c -- load-time preparation of the EXL3 kernels: reconstruction, the five launches of the routed experts'
 * chain, and the row sum. Entry points and refusal rules follow the reference's source/exl3.c:58-323 and
 * source/exl3_tp.c:250-290; the launch geometry is gfx950's:
 *
 *   launch          kernel                      grid                                  block
 *   input           exl3_input                  (input_size / 128, jobs, 2)           64   one wavefront a transform
 *   gate/up         exl3_gate_up_<k>|_mixed     (inner_size / 128, jobs, 2)           256  4 K slices x 8 output tiles
 *   activate        exl3_activate               (inner_size / 128, jobs, 1)           64
 *   down            exl3_down_<k>|_mixed        (input_size / 128, jobs, 1)           256
 *   (a product launch of fewer than EXL3_THIN_BELOW_BLOCKS such blocks: the _thin instance, x = size / 16)
 *   finish          exl3_finish                 (input_size / 128, jobs, 1)           64
 *   row sum         exl3_row_sum                (ceil(width / 256), rows, 1)          256
 *
 * <k> is the record's one width; "_mixed" is taken when the record names a per-matrix widths table.
 */
#include <math.h>
#include <string.h>

#include "prepare_common.h"

#define WAVE_THREADS 64u
#define PRODUCT_THREADS 256u
#define STRIP_OUTPUTS 128u /* eight output tiles a block */
#define MOST_GRID_ROWS 65535u

const char *exl3_width_name(uint32_t bits_x2)
{
    switch (bits_x2) {
    case 4u: return "k2";
    case 5u: return "k2_5";
    case 6u: return "k3";
    case 8u: return "k4";
    default: return NULL;
    }
}

uint64_t exl3_scratch_byte_count(uint32_t pair_count, uint32_t input_size)
{
    /* fp16 operands [2][pairs][input] = 4 bytes an input, float32 products [2][pairs][inner <= input] = 8 */
    return product_or_most((uint64_t)pair_count * input_size, 12u);
}

result_status exl3_reconstruct_prepare(const struct exl3_reconstruct_record *record, uint64_t arena_byte_count,
                                       uint32_t kernel, struct kernel_launch *launch_out)
{
    if (record == NULL || launch_out == NULL || kernel == BACKEND_NO_KERNEL || record->reserved_zero != 0) {
        REFUSE("EXL3 reconstruction: a missing argument, an unprepared kernel or a reserved field that is not zero");
        return STATUS_INVALID_ARGUMENT;
    }
    const struct matrix_shape_record shape = {record->output_size, record->input_size, record->bits_per_weight, 0};
    uint64_t stored = 0;
    const result_status counted = exl3_weight_operations.stored_byte_count(&shape, &stored);
    if (counted != STATUS_OK) {
        REFUSE("EXL3 reconstruction: %u x %u at stored width %u is no matrix this build decodes", record->input_size,
               record->output_size, record->bits_per_weight);
        return counted;
    }
    const uint64_t elements = (uint64_t)record->input_size * record->output_size;
    const struct checked_range ranges[] = {
        {"the matrix", {record->matrix_offset, stored}, stored, true},
        {"the reconstructed weights", {record->output_offset, elements * 2u}, elements * 2u, false},
    };
    const uint64_t blocks = (elements + LINEAR_ELEMENT_THREADS - 1u) / LINEAR_ELEMENT_THREADS;
    if (!ranges_are_valid("EXL3 reconstruction", ranges, 2, arena_byte_count) || blocks > 0x7FFFFFFFu) {
        return STATUS_INVALID_ARGUMENT;
    }
    launch_fill(launch_out, kernel, (uint32_t)blocks, 1, 1, LINEAR_ELEMENT_THREADS, 0, record, sizeof *record);
    return STATUS_OK;
}

static result_status chain_prepare(const struct exl3_expert_record *record, uint64_t arena_byte_count,
                                   const struct backend_operations *backend, struct device_card *card,
                                   uint32_t arithmetic_class, struct kernel_launch *launches_out)
{
    static const char what[] = "EXL3 experts";
    if (record == NULL || backend == NULL || backend->kernel_prepare == NULL || card == NULL || launches_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    if (arithmetic_class != ARITHMETIC_CLASS_GFX950) {
        REFUSE("%s: arithmetic class %u: this library holds kernels of class %u alone", what, arithmetic_class,
               ARITHMETIC_CLASS_GFX950);
        return STATUS_INVALID_ARGUMENT;
    }
    const bool whole_rows = record->pairs_per_row >= 1u && record->pair_count >= 1u && record->pair_count % record->pairs_per_row == 0u;
    const bool jobs_fit_a_grid = record->job_count >= 1u && record->job_count <= MOST_GRID_ROWS;
    const bool sums_in_place = record->products_offset == record->output_offset; /* the finish launch overwrites the products it reads */
    const bool limit_holds = isfinite(record->activation_limit) && record->activation_limit > 0.0f;
    if (!whole_rows || !jobs_fit_a_grid || !sums_in_place || !limit_holds || record->input_size < record->inner_size ||
        record->reserved_zero != 0) {
        REFUSE("%s: counts, the in-place output rule or the activation limit", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const bool mixed = record->widths_offset != 0;
    /* shapes: with per-matrix widths the widest supported one stands for the byte bound */
    const struct matrix_shape_record shape = {record->inner_size, record->input_size,
                                              mixed ? EXL3_K4 : record->bits_per_weight, 0};
    uint64_t stored = 0;
    const result_status counted = exl3_weight_operations.stored_byte_count(&shape, &stored);
    if (counted != STATUS_OK) {
        REFUSE("%s: %u x %u at stored width %u is no matrix this build decodes", what, record->input_size,
               record->inner_size, shape.bits_per_weight);
        return counted == STATUS_UNSUPPORTED ? STATUS_UNSUPPORTED : STATUS_INVALID_ARGUMENT;
    }
    const uint64_t inputs = (uint64_t)record->pair_count * record->input_size;
    if (exl3_scratch_byte_count(record->pair_count, record->input_size) == UINT64_MAX) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct checked_range ranges[] = {
        {"the jobs", {record->jobs_offset, (uint64_t)record->job_count * sizeof(struct expert_job_record)},
         (uint64_t)record->job_count * sizeof(struct expert_job_record), false},
        {"the input rows", {record->input_offset, inputs / record->pairs_per_row * 2u}, inputs / record->pairs_per_row * 2u, false},
        {"the operands", {record->operands_offset, inputs * 4u}, inputs * 4u, false},
        {"the products", {record->products_offset, inputs * 8u}, inputs * 8u, false},
        {"the hidden values", {record->hidden_offset, (uint64_t)record->pair_count * record->inner_size * 2u},
         (uint64_t)record->pair_count * record->inner_size * 2u, false},
    };
    if (!ranges_are_valid(what, ranges, 5, arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    if (mixed && record->widths_offset % LINEAR_OFFSET_ALIGNMENT_BYTES != 0) {
        REFUSE("%s: the widths table begins off a multiple of %u", what, LINEAR_OFFSET_ALIGNMENT_BYTES);
        return STATUS_INVALID_ARGUMENT;
    }
    char gate_up_name[40], down_name[40];
    const char *width = mixed ? "mixed" : exl3_width_name(exl3_bits_x2(record->bits_per_weight));
    /* a product launch of few blocks (a job or two) takes the instances of one output tile a block: eight times the
     * blocks, the same sums */
    const bool thin_gate_up = (uint64_t)record->inner_size / STRIP_OUTPUTS * record->job_count * 2u < EXL3_THIN_BELOW_BLOCKS;
    const bool thin_down = (uint64_t)record->input_size / STRIP_OUTPUTS * record->job_count < EXL3_THIN_BELOW_BLOCKS;
    (void)snprintf(gate_up_name, sizeof gate_up_name, "exl3_gate_up_%s%s", width, thin_gate_up ? "_thin" : "");
    (void)snprintf(down_name, sizeof down_name, "exl3_down_%s%s", width, thin_down ? "_thin" : "");
    const struct {
        const char *name;
        uint32_t width, threads, projections, block_outputs;
    } stages[EXL3_EXPERT_LAUNCHES] = {
        {"exl3_input", record->input_size, WAVE_THREADS, 2u, EXL3_TRANSFORM},
        {gate_up_name, record->inner_size, PRODUCT_THREADS, 2u, (thin_gate_up ? EXL3_THIN_STRIP_TILES : EXL3_STRIP_TILES) * EXL3_TILE},
        {"exl3_activate", record->inner_size, WAVE_THREADS, 1u, EXL3_TRANSFORM},
        {down_name, record->input_size, PRODUCT_THREADS, 1u, (thin_down ? EXL3_THIN_STRIP_TILES : EXL3_STRIP_TILES) * EXL3_TILE},
        {"exl3_finish", record->input_size, WAVE_THREADS, 1u, EXL3_TRANSFORM},
    };
    struct kernel_launch launches[EXL3_EXPERT_LAUNCHES];
    for (uint32_t stage = 0; stage < EXL3_EXPERT_LAUNCHES; stage++) {
        uint32_t kernel = BACKEND_NO_KERNEL;
        const result_status prepared =
            backend->kernel_prepare(card, EXL3_KERNEL_FILE, stages[stage].name, sizeof *record, &kernel);
        if (prepared != STATUS_OK) {
            return prepared;
        }
        if (kernel == BACKEND_NO_KERNEL) {
            return STATUS_UNSUPPORTED;
        }
        _Static_assert(STRIP_OUTPUTS == EXL3_STRIP_TILES * EXL3_TILE && STRIP_OUTPUTS == EXL3_TRANSFORM,
                       "a strip of outputs and a transform block are both 128 wide");
        launch_fill(&launches[stage], kernel, stages[stage].width / stages[stage].block_outputs, record->job_count,
                    stages[stage].projections, stages[stage].threads, 0, record, sizeof *record);
    }
    memcpy(launches_out, launches, sizeof launches);
    return STATUS_OK;
}

result_status exl3_experts_prepare(const struct exl3_expert_record *record, uint64_t arena_byte_count,
                                   const struct backend_operations *backend, struct device_card *card,
                                   uint32_t arithmetic_class, struct kernel_launch *launches_out)
{
    return chain_prepare(record, arena_byte_count, backend, card, arithmetic_class, launches_out);
}

result_status exl3_experts_fast_prepare(const struct exl3_expert_record *record, uint64_t arena_byte_count,
                                        const struct backend_operations *backend, struct device_card *card,
                                        uint32_t arithmetic_class, struct kernel_launch *launches_out)
{
    return chain_prepare(record, arena_byte_count, backend, card, arithmetic_class, launches_out);
}

result_status exl3_experts_relaxed_prepare(const struct exl3_expert_record *record, uint64_t arena_byte_count,
                                           const struct backend_operations *backend, struct device_card *card,
                                           uint32_t arithmetic_class, struct kernel_launch *launches_out)
{
    struct kernel_launch unused[EXL3_EXPERT_LAUNCHES];
    const result_status checked = chain_prepare(record, arena_byte_count, backend, card, arithmetic_class, unused);
    (void)launches_out;
    return checked != STATUS_OK ? checked : STATUS_UNSUPPORTED; /* the relaxed order belongs to one other class */
}

result_status exl3_row_sum_prepare(const struct expert_row_sum_arguments *record, uint32_t rows,
                                   uint64_t arena_bytes, const struct backend_operations *backend,
                                   struct device_card *card, struct kernel_launch *launch_out)
{
    if (record == NULL || backend == NULL || backend->kernel_prepare == NULL || card == NULL || launch_out == NULL ||
        rows == 0 || rows > MOST_GRID_ROWS || record->width == 0 || record->pairs_per_row == 0) {
        REFUSE("EXL3 row sum: a missing argument or a count of zero");
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t row_bytes = (uint64_t)rows * record->width * 4u;
    const struct checked_range ranges[] = {
        {"the pair outputs", {record->pair_output_offset, product_or_most(row_bytes, record->pairs_per_row)},
         product_or_most(row_bytes, record->pairs_per_row), false},
        {"the row outputs", {record->row_output_offset, row_bytes}, row_bytes, false},
    };
    if (!ranges_are_valid("EXL3 row sum", ranges, 2, arena_bytes)) {
        return STATUS_INVALID_ARGUMENT;
    }
    uint32_t kernel = BACKEND_NO_KERNEL;
    const result_status prepared = backend->kernel_prepare(card, EXL3_KERNEL_FILE, EXL3_ROW_SUM, sizeof *record, &kernel);
    if (prepared != STATUS_OK) {
        return prepared;
    }
    launch_fill(launch_out, kernel, (record->width + LINEAR_ELEMENT_THREADS - 1u) / LINEAR_ELEMENT_THREADS, rows, 1,
                LINEAR_ELEMENT_THREADS, 0, record, sizeof *record);
    return STATUS_OK;
}
