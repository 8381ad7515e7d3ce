/*
 * exl3_layout.c -- load-time slices of stored EXL3 matrices: what a card that takes a share of a layer's columns copies
 * out of the whole matrices, byte for byte. Entry points and refusal rules follow the reference's source/exl3_layout.c
 * (include/anemone/exl3_layout.h:15-103). Host-only: no decode, no floating arithmetic, no allocation.
 *
 * A stored matrix: code rows (one a tile row of 16 inputs, outputs / 16 tiles of 32 K bytes each), then suh[inputs],
 * svh[outputs] as fp16. A slice of whole transforms of 128 channels is again such a matrix.
 */
#include <string.h>

#include "prepare_common.h"

#define HALF_BYTES 2u
#define RELAXED_SLICES 8u /* the eight-part order's K slices (EXL3_RELAXED_SLICES of the reference) */

struct stored_matrix {
    uint64_t row_bytes;  /* of one tile row of codes */
    uint64_t code_bytes; /* of all of them */
    uint64_t bytes;      /* with suh and svh */
};

static struct stored_matrix stored_matrix_of(uint32_t inputs, uint32_t outputs, uint32_t bits_x2)
{
    struct stored_matrix matrix;
    matrix.row_bytes = exl3_code_bytes(EXL3_TILE, outputs, bits_x2);
    matrix.code_bytes = exl3_code_bytes(inputs, outputs, bits_x2);
    matrix.bytes = matrix.code_bytes + ((uint64_t)inputs + outputs) * HALF_BYTES;
    return matrix;
}

/* a range of whole transforms inside a dimension of whole transforms, not empty */
static bool range_is_valid(uint32_t size, uint32_t begin, uint32_t count)
{
    return size % EXL3_TRANSFORM == 0 && begin % EXL3_TRANSFORM == 0 && count % EXL3_TRANSFORM == 0 && count != 0 && begin <= size &&
           count <= size - begin;
}

result_status bb_exl3_matrix_slice_prepare(const struct bb_exl3_matrix_slice *slice, struct bb_exl3_slice_sizes *sizes_out)
{
    if (slice == NULL || sizes_out == NULL || slice->reserved_zero != 0 || !exl3_width_supported(slice->bits_per_weight) ||
        !range_is_valid(slice->input_size, slice->input_begin, slice->input_count) ||
        !range_is_valid(slice->output_size, slice->output_begin, slice->output_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t bits_x2 = exl3_bits_x2(slice->bits_per_weight);
    sizes_out->source_bytes = stored_matrix_of(slice->input_size, slice->output_size, bits_x2).bytes;
    sizes_out->packed_bytes = stored_matrix_of(slice->input_count, slice->output_count, bits_x2).bytes;
    return STATUS_OK;
}

result_status bb_exl3_matrix_slice_copy(const struct bb_exl3_matrix_slice *slice, const void *source, size_t source_bytes, void *destination,
                                        size_t destination_bytes)
{
    struct bb_exl3_slice_sizes sizes;
    if (slice == NULL || source == NULL || destination == NULL) {
        return STATUS_INVALID_ARGUMENT;
    }
    const struct bb_exl3_matrix_slice taken = *slice; /* the destination may hold the description */
    if (bb_exl3_matrix_slice_prepare(&taken, &sizes) != STATUS_OK || sizes.source_bytes > source_bytes || sizes.packed_bytes > destination_bytes) {
        return STATUS_INVALID_ARGUMENT;
    }
    const uintptr_t from = (uintptr_t)source, to = (uintptr_t)destination;
    if (source_bytes > UINTPTR_MAX - from || destination_bytes > UINTPTR_MAX - to || (from < to + destination_bytes && to < from + source_bytes)) {
        return STATUS_INVALID_ARGUMENT; /* an extent that wraps, or the two share a byte */
    }
    const uint32_t bits_x2 = exl3_bits_x2(taken.bits_per_weight);
    const struct stored_matrix whole = stored_matrix_of(taken.input_size, taken.output_size, bits_x2);
    const struct stored_matrix part = stored_matrix_of(taken.input_count, taken.output_count, bits_x2);
    const unsigned char *in = source;
    unsigned char *out = destination;
    /* the code rows of the input range, each cut to the output range's tiles */
    const unsigned char *row = in + (uint64_t)(taken.input_begin / EXL3_TILE) * whole.row_bytes + exl3_code_bytes(EXL3_TILE, taken.output_begin, bits_x2);
    for (uint32_t tile_row = 0; tile_row < taken.input_count / EXL3_TILE; tile_row++) {
        memcpy(out, row, (size_t)part.row_bytes);
        out += part.row_bytes;
        row += whole.row_bytes;
    }
    /* suh of the input range, svh of the output range */
    const unsigned char *scales = in + whole.code_bytes;
    memcpy(out, scales + (uint64_t)taken.input_begin * HALF_BYTES, (size_t)taken.input_count * HALF_BYTES);
    out += (size_t)taken.input_count * HALF_BYTES;
    memcpy(out, scales + ((uint64_t)taken.input_size + taken.output_begin) * HALF_BYTES, (size_t)taken.output_count * HALF_BYTES);
    return STATUS_OK;
}

result_status bb_exl3_output_shard_prepare(uint32_t outer_size, uint32_t inner_size, uint32_t bits_per_weight, uint32_t rank_count, uint32_t rank,
                                           enum bb_exl3_product_order order, struct bb_exl3_output_shard_plan *plan_out)
{
    if (plan_out == NULL || (rank_count != 1u && rank_count != BB_EXL3_TP_RANKS) || rank >= rank_count ||
        (order != BB_EXL3_REFERENCE_ORDER && order != BB_EXL3_EIGHT_PART_ORDER) || outer_size % EXL3_TRANSFORM != 0 ||
        inner_size % EXL3_TRANSFORM != 0 || outer_size / EXL3_TRANSFORM < rank_count || inner_size / EXL3_TRANSFORM < rank_count) {
        return STATUS_INVALID_ARGUMENT;
    }
    /* a rank's share of a dimension's transforms: from blocks rank / ranks to blocks (rank + 1) / ranks */
    const uint32_t outer_blocks = outer_size / EXL3_TRANSFORM, inner_blocks = inner_size / EXL3_TRANSFORM;
    const uint32_t outer_begin = outer_blocks * rank / rank_count * EXL3_TRANSFORM, outer_end = outer_blocks * (rank + 1u) / rank_count * EXL3_TRANSFORM;
    const uint32_t inner_begin = inner_blocks * rank / rank_count * EXL3_TRANSFORM, inner_end = inner_blocks * (rank + 1u) / rank_count * EXL3_TRANSFORM;
    struct bb_exl3_output_shard_plan plan;
    memset(&plan, 0, sizeof plan);
    plan.gate_up = (struct bb_exl3_matrix_slice){outer_size, inner_size, 0, outer_size, inner_begin, inner_end - inner_begin, bits_per_weight, 0};
    plan.down = (struct bb_exl3_matrix_slice){inner_size, outer_size, 0, inner_size, outer_begin, outer_end - outer_begin, bits_per_weight, 0};
    plan.rank_count = rank_count;
    plan.rank = rank;
    plan.product_slices = order == BB_EXL3_REFERENCE_ORDER ? EXL3_PRODUCT_SLICES : RELAXED_SLICES;
    plan.order = order;
    struct bb_exl3_slice_sizes sizes;
    result_status status = bb_exl3_matrix_slice_prepare(&plan.gate_up, &sizes);
    if (status == STATUS_OK) {
        status = bb_exl3_matrix_slice_prepare(&plan.down, &sizes);
    }
    if (status != STATUS_OK) {
        return status;
    }
    *plan_out = plan;
    return STATUS_OK;
}
