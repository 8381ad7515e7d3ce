/*
 * exl3_layout.c -- cutting stored EXL3 matrices at load time. Written from the contract of the reference's
 * include/anemone/exl3_layout.h:15-103: a cut that keeps whole 128-channel transforms on both axes is again a stored
 * matrix, and a card of a group of four takes such cuts of an expert's three matrices. Host-only: bytes move, nothing is
 * decoded, nothing is allocated.
 *
 * Stored matrix (include/anemone/exl3_records.h:2-9 of the reference): inputs/16 bands of codes, a band holding outputs/16
 * tiles of 32*K bytes side by side; behind the bands fp16 suh[inputs], then fp16 svh[outputs].
 */
#include <string.h>

#include "prepare_common.h"

enum { FP16_BYTES = 2, EIGHT_PART_SLICES = 8 };

/* ---- one axis of a cut ------------------------------------------------------------------------------------------ */

struct stretch {
    uint32_t of;  /* the axis' channels */
    uint32_t at;  /* first channel taken */
    uint32_t len; /* channels taken */
};

static bool whole_transforms(uint32_t channels)
{
    return channels % EXL3_TRANSFORM == 0;
}

static bool stretch_holds(struct stretch axis)
{
    if (axis.len == 0 || !whole_transforms(axis.of) || !whole_transforms(axis.at) || !whole_transforms(axis.len)) {
        return false;
    }
    return axis.at < axis.of && axis.len <= axis.of - axis.at;
}

/* ---- byte geometry of a stored matrix ------------------------------------------------------------------------------- */

struct footprint {
    uint64_t band;  /* one band of codes: 16 inputs by every output */
    uint64_t codes; /* every band */
    uint64_t suh;   /* where suh begins; svh follows it */
    uint64_t end;   /* the matrix' bytes */
};

static struct footprint footprint_of(uint32_t inputs, uint32_t outputs, uint32_t bits_x2)
{
    struct footprint f;
    f.band = exl3_code_bytes(EXL3_TILE, outputs, bits_x2);
    f.codes = f.band * (inputs / EXL3_TILE);
    f.suh = f.codes;
    f.end = f.codes + (uint64_t)FP16_BYTES * inputs + (uint64_t)FP16_BYTES * outputs;
    return f;
}

static bool cut_is_sound(const struct bb_exl3_matrix_slice *cut)
{
    const struct stretch over_inputs = {cut->input_size, cut->input_begin, cut->input_count};
    const struct stretch over_outputs = {cut->output_size, cut->output_begin, cut->output_count};
    return cut->reserved_zero == 0 && exl3_width_supported(cut->bits_per_weight) && stretch_holds(over_inputs) && stretch_holds(over_outputs);
}

result_status bb_exl3_matrix_slice_prepare(const struct bb_exl3_matrix_slice *slice, struct bb_exl3_slice_sizes *sizes_out)
{
    if (slice == NULL || sizes_out == NULL || !cut_is_sound(slice)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t bits_x2 = exl3_bits_x2(slice->bits_per_weight);
    const struct bb_exl3_slice_sizes sizes = {footprint_of(slice->input_size, slice->output_size, bits_x2).end,
                                              footprint_of(slice->input_count, slice->output_count, bits_x2).end};
    *sizes_out = sizes;
    return STATUS_OK;
}

/* ---- the copy: three gathers of equal runs at a fixed pitch ------------------------------------------------------ */

struct gather {
    uint64_t first; /* source offset of the first run */
    uint64_t pitch; /* from one run's start to the next */
    uint64_t run;   /* bytes of a run */
    uint64_t runs;
};

static unsigned char *gather_into(unsigned char *to, const unsigned char *source, struct gather g)
{
    const unsigned char *from = source + g.first;
    for (uint64_t k = 0; k < g.runs; k++, from += g.pitch, to += g.run) {
        memcpy(to, from, (size_t)g.run);
    }
    return to;
}

/* false where an extent runs past the end of the address space or the two extents have a byte in common */
static bool apart(const void *a, size_t a_bytes, const void *b, size_t b_bytes)
{
    const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
    if (a_bytes > UINTPTR_MAX - a0 || b_bytes > UINTPTR_MAX - b0) {
        return false;
    }
    return a0 + a_bytes <= b0 || b0 + b_bytes <= a0;
}

result_status bb_exl3_matrix_slice_copy(const struct bb_exl3_matrix_slice *slice, const void *source, size_t source_bytes, void *destination,
                                        size_t destination_bytes)
{
    if (slice == NULL || source == NULL || destination == NULL) {
        return STATUS_INVALID_ARGUMENT;
    }
    struct bb_exl3_matrix_slice cut;
    memcpy(&cut, slice, sizeof cut); /* read once: the description is not promised to lie outside the destination */
    if (!cut_is_sound(&cut)) {
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t bits_x2 = exl3_bits_x2(cut.bits_per_weight);
    const struct footprint whole = footprint_of(cut.input_size, cut.output_size, bits_x2);
    const struct footprint part = footprint_of(cut.input_count, cut.output_count, bits_x2);
    if (whole.end > source_bytes || part.end > destination_bytes || !apart(source, source_bytes, destination, destination_bytes)) {
        return STATUS_INVALID_ARGUMENT;
    }
    /* a tile's codes lie in its band at tile * 32K bytes, so the taken outputs of a band are one run */
    const uint64_t into_band = exl3_code_bytes(EXL3_TILE, cut.output_begin, bits_x2);
    const struct gather pieces[3] = {
        {(uint64_t)(cut.input_begin / EXL3_TILE) * whole.band + into_band, whole.band, part.band, cut.input_count / EXL3_TILE},
        {whole.suh + (uint64_t)FP16_BYTES * cut.input_begin, 0, (uint64_t)FP16_BYTES * cut.input_count, 1},
        {whole.suh + (uint64_t)FP16_BYTES * cut.input_size + (uint64_t)FP16_BYTES * cut.output_begin, 0, (uint64_t)FP16_BYTES * cut.output_count, 1},
    };
    unsigned char *to = destination;
    for (unsigned p = 0; p < 3; p++) {
        to = gather_into(to, source, pieces[p]);
    }
    return STATUS_OK;
}

/* ---- what a card of a group takes ------------------------------------------------------------------------------- */

/* the member's share of an axis, in whole transforms: transforms [n*member/members, n*(member+1)/members) */
static struct stretch share_of(uint32_t channels, uint32_t member, uint32_t members)
{
    const uint32_t transforms = channels / EXL3_TRANSFORM;
    const uint32_t first = transforms * member / members, behind = transforms * (member + 1u) / members;
    const struct stretch share = {channels, first * EXL3_TRANSFORM, (behind - first) * EXL3_TRANSFORM};
    return share;
}

/* the cut of a matrix [inputs][outputs] that keeps every input and the given stretch of outputs */
static struct bb_exl3_matrix_slice columns_of(uint32_t inputs, struct stretch outputs, uint32_t stored_width)
{
    struct bb_exl3_matrix_slice cut;
    memset(&cut, 0, sizeof cut);
    cut.input_size = cut.input_count = inputs;
    cut.output_size = outputs.of;
    cut.output_begin = outputs.at;
    cut.output_count = outputs.len;
    cut.bits_per_weight = stored_width;
    return cut;
}

result_status bb_exl3_output_shard_prepare(uint32_t outer_size, uint32_t inner_size, uint32_t bits_per_weight, uint32_t rank_count, uint32_t rank,
                                           enum bb_exl3_product_order order, struct bb_exl3_output_shard_plan *plan_out)
{
    uint32_t slices;
    switch (order) {
    case BB_EXL3_REFERENCE_ORDER: slices = EXL3_PRODUCT_SLICES; break;
    case BB_EXL3_EIGHT_PART_ORDER: slices = EIGHT_PART_SLICES; break;
    default: return STATUS_INVALID_ARGUMENT;
    }
    const bool group_known = rank_count == 1u || rank_count == BB_EXL3_TP_RANKS;
    if (plan_out == NULL || !group_known || rank >= rank_count || !whole_transforms(outer_size) || !whole_transforms(inner_size)) {
        return STATUS_INVALID_ARGUMENT;
    }
    /* gate and up give the member a stretch of the inner channels, down a stretch of the outer ones; none may be empty */
    const struct stretch inner = share_of(inner_size, rank, rank_count), outer = share_of(outer_size, rank, rank_count);
    if (outer_size / EXL3_TRANSFORM < rank_count || inner_size / EXL3_TRANSFORM < rank_count) {
        return STATUS_INVALID_ARGUMENT;
    }
    struct bb_exl3_output_shard_plan plan;
    memset(&plan, 0, sizeof plan);
    plan.gate_up = columns_of(outer_size, inner, bits_per_weight);
    plan.down = columns_of(inner_size, outer, bits_per_weight);
    plan.rank_count = rank_count;
    plan.rank = rank;
    plan.product_slices = slices;
    plan.order = order;
    if (!cut_is_sound(&plan.gate_up) || !cut_is_sound(&plan.down)) {
        return STATUS_INVALID_ARGUMENT;
    }
    *plan_out = plan;
    return STATUS_OK;
}
