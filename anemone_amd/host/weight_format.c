/*
 * weight_format.c -- how many bytes a matrix of a shape occupies, per format, exactly as the kernels read it.
 * Byte counts follow include/anemone/weight_format_seam.h:22-46 (E2M1_SCALED, E4M3_SCALED) and
 * include/anemone/exl3_records.h:2-9 with source/exl3.c:10-37 (EXL3) of the reference; E4M3_BLOCK128 is this build's own.
 */
#include "anemone_ops.h"

#include <stddef.h>

static result_status e2m1_bytes(const struct matrix_shape_record *shape, uint64_t *out)
{
    if (shape == NULL || out == NULL || shape->reserved_must_be_zero != 0 || shape->bits_per_weight != 4 ||
        shape->output_size == 0 || shape->input_size == 0 || shape->output_size % 16u != 0 ||
        shape->input_size % 64u != 0) {
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t weights = (uint64_t)shape->output_size * shape->input_size;
    *out = weights / 2u + weights / 32u;
    return STATUS_OK;
}

static result_status e4m3_bytes(const struct matrix_shape_record *shape, uint64_t *out)
{
    if (shape == NULL || out == NULL || shape->reserved_must_be_zero != 0 || shape->bits_per_weight != 8 ||
        shape->output_size == 0 || shape->input_size == 0 || shape->output_size % 16u != 0 ||
        shape->input_size % 32u != 0) {
        return STATUS_INVALID_ARGUMENT;
    }
    *out = (uint64_t)shape->output_size * shape->input_size +
           (uint64_t)((shape->output_size + 31u) / 32u) * (shape->input_size / 32u);
    return STATUS_OK;
}

static result_status e4m3_block128_bytes(const struct matrix_shape_record *shape, uint64_t *out)
{
    if (shape == NULL || out == NULL || shape->reserved_must_be_zero != 0 || shape->bits_per_weight != 8 ||
        shape->output_size == 0 || shape->input_size == 0 || shape->output_size % 128u != 0 || shape->input_size % 128u != 0) {
        return STATUS_INVALID_ARGUMENT;
    }
    *out = (uint64_t)shape->output_size * shape->input_size + (uint64_t)(shape->output_size / 128u) * (shape->input_size / 128u) * 4u;
    return STATUS_OK;
}

static result_status exl3_bytes(const struct matrix_shape_record *shape, uint64_t *out)
{
    /* whole 128-wide transforms on both sides; a width the format defines but this build has no kernels for is
     * UNSUPPORTED, a value that is no width INVALID */
    if (shape == NULL || out == NULL || shape->reserved_must_be_zero != 0 || shape->output_size == 0 ||
        shape->input_size == 0 || shape->output_size % EXL3_TRANSFORM != 0 || shape->input_size % EXL3_TRANSFORM != 0 ||
        exl3_bits_x2(shape->bits_per_weight) == 0) {
        return STATUS_INVALID_ARGUMENT;
    }
    if (!exl3_width_supported(shape->bits_per_weight)) {
        return STATUS_UNSUPPORTED;
    }
    *out = exl3_code_bytes(shape->input_size, shape->output_size, exl3_bits_x2(shape->bits_per_weight)) +
           2ull * ((uint64_t)shape->input_size + shape->output_size);
    return STATUS_OK;
}

static const struct weight_format_operations e2m1_operations = {"e2m1_scaled", e2m1_bytes};
static const struct weight_format_operations e4m3_operations = {"e4m3_scaled", e4m3_bytes};
static const struct weight_format_operations e4m3_block128_operations = {"e4m3_block128", e4m3_block128_bytes};
const struct weight_format_operations exl3_weight_operations = {"exl3", exl3_bytes};

const struct weight_format_operations *weight_format_operations_of(enum weight_format_code format)
{
    switch (format) {
    case WEIGHT_FORMAT_E2M1_SCALED: return &e2m1_operations;
    case WEIGHT_FORMAT_E4M3_SCALED: return &e4m3_operations;
    case WEIGHT_FORMAT_EXL3: return &exl3_weight_operations;
    case WEIGHT_FORMAT_E4M3_BLOCK128: return &e4m3_block128_operations;
    default: return NULL;
    }
}
