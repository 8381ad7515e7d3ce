/*
 * weight_format.c -- how many bytes a matrix of a shape occupies, per format, exactly as the kernels read it.
 * Byte counts follow include/anemone/weight_format_seam.h:22-46 (E2M1_SCALED, E4M3_SCALED) and
 * include/anemone/exl3_records.h:2-9 with source/exl3.c:10-37 (EXL3) of the reference; E4M3_BLOCK128 is this build's own.
 */
#include "anemone_ops.h"

#include <stddef.h>
#include <string.h>

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

/* the GFX950 formats hold what their _SCALED counterparts hold, in whole K steps of 128 inputs */
static result_status e2m1_gfx950_bytes(const struct matrix_shape_record *shape, uint64_t *out)
{
    if (shape == NULL || shape->input_size % 128u != 0 || shape->output_size % 64u != 0) {
        return STATUS_INVALID_ARGUMENT;
    }
    return e2m1_bytes(shape, out);
}

static result_status e4m3_gfx950_bytes(const struct matrix_shape_record *shape, uint64_t *out)
{
    if (shape == NULL || shape->input_size % 128u != 0 || shape->output_size % 32u != 0) {
        return STATUS_INVALID_ARGUMENT;
    }
    return e4m3_bytes(shape, out);
}

static const struct weight_format_operations e2m1_operations = {"e2m1_scaled", e2m1_bytes};
static const struct weight_format_operations e4m3_operations = {"e4m3_scaled", e4m3_bytes};
static const struct weight_format_operations e4m3_block128_operations = {"e4m3_block128", e4m3_block128_bytes};
const struct weight_format_operations exl3_weight_operations = {"exl3", exl3_bytes};
static const struct weight_format_operations e2m1_gfx950_operations = {"e2m1_gfx950", e2m1_gfx950_bytes};
static const struct weight_format_operations e4m3_gfx950_operations = {"e4m3_gfx950", e4m3_gfx950_bytes};
static const struct weight_format_operations e4m3_block128_gfx950_operations = {"e4m3_block128_gfx950", e4m3_block128_bytes}; /* whole blocks of 128 x 128 either way */

const struct weight_format_operations *weight_format_operations_of(enum weight_format_code format)
{
    switch (format) {
    case WEIGHT_FORMAT_E2M1_SCALED: return &e2m1_operations;
    case WEIGHT_FORMAT_E4M3_SCALED: return &e4m3_operations;
    case WEIGHT_FORMAT_EXL3: return &exl3_weight_operations;
    case WEIGHT_FORMAT_E4M3_BLOCK128: return &e4m3_block128_operations;
    case WEIGHT_FORMAT_E2M1_GFX950: return &e2m1_gfx950_operations;
    case WEIGHT_FORMAT_E4M3_GFX950: return &e4m3_gfx950_operations;
    case WEIGHT_FORMAT_E4M3_BLOCK128_GFX950: return &e4m3_block128_gfx950_operations;
    default: return NULL;
    }
}

/* ---- between the reference's lane order and gfx950's ------------------------------------------------------------------
 * The reference's E2M1_SCALED (include/anemone/weight_format_seam.h:26-34 there): a tile of 16 outputs by a load of 64
 * inputs is 32 lanes x 4 words; lane 4 G + t, word `step`: nibble 4 r + 16 h is output G + 8 (r % 2), input
 * 16 step + 2 t + 8 (r / 2) + h; behind all words, a tile's load's 8 x 4 scale bytes: byte 4 G + 2 q + r is output
 * G + 8 r, inputs 32 q .. + 31 of the load. E4M3_SCALED (:35-42): a tile by a group of 32 inputs is 32 lanes x 16 bytes;
 * lane 4 G + t, byte b: output G + 8 (b % 2), input 8 (b / 4) + 2 t + (b / 2) % 2. */

static bool apart(const void *a, uint64_t a_bytes, const void *b, uint64_t b_bytes)
{
    const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
    return a_bytes <= UINTPTR_MAX - a0 && b_bytes <= UINTPTR_MAX - b0 && (a0 + a_bytes <= b0 || b0 + b_bytes <= a0);
}

static uint32_t word_at(const unsigned char *bytes, uint64_t word)
{
    uint32_t value;
    memcpy(&value, bytes + word * 4u, sizeof value);
    return value;
}

/* where E2M1_GFX950 holds the scale code of a lane of a tile's K step: the tiles in groups of four (64 outputs), a group's
 * K step 64 lanes x 4 bytes, byte tile % 4 */
static uint64_t e2m1_gfx950_scale_at(uint32_t tile, uint32_t step, uint32_t steps, uint32_t lane)
{
    return (((uint64_t)(tile / 4u) * steps + step) * 64u + lane) * 4u + tile % 4u;
}

/* E2M1: a K step's lane 16 g + o takes, for each of its four words T, the words `2 (g % 2)` and `2 (g % 2) + 1` of the
 * reference's lane 4 (o % 8) + T of load 2 step + g / 2: its output's nibbles of the first below those of the second */
static void e2m1_to_gfx950(uint32_t outputs, uint32_t inputs, const unsigned char *from, unsigned char *to)
{
    const uint32_t tiles = outputs / 16u, steps = inputs / 128u, loads = inputs / 64u;
    const unsigned char *from_scales = from + (uint64_t)outputs * inputs / 2u;
    unsigned char *to_scales = to + (uint64_t)outputs * inputs / 2u;
    for (uint32_t tile = 0; tile < tiles; tile++) {
        for (uint32_t step = 0; step < steps; step++) {
            for (uint32_t lane = 0; lane < 64u; lane++) {
                const uint32_t g = lane / 16u, o = lane % 16u, nibble_shift = 4u * (o / 8u);
                const uint64_t load = (uint64_t)tile * loads + 2u * step + g / 2u;
                for (uint32_t T = 0; T < 4u; T++) {
                    const uint64_t first = (load * 32u + 4u * (o % 8u) + T) * 4u + 2u * (g % 2u);
                    const uint32_t low = (word_at(from, first) >> nibble_shift) & 0x0F0F0F0Fu;
                    const uint32_t high = (word_at(from, first + 1u) >> nibble_shift) & 0x0F0F0F0Fu;
                    const uint32_t word = low | (high << 4);
                    memcpy(to + ((((uint64_t)tile * steps + step) * 64u + lane) * 4u + T) * 4u, &word, sizeof word);
                }
                to_scales[e2m1_gfx950_scale_at(tile, step, steps, lane)] = from_scales[(load * 8u + o % 8u) * 4u + 2u * (g % 2u) + o / 8u];
            }
        }
    }
}

static void e2m1_from_gfx950(uint32_t outputs, uint32_t inputs, const unsigned char *from, unsigned char *to)
{
    const uint32_t tiles = outputs / 16u, steps = inputs / 128u, loads = inputs / 64u;
    const unsigned char *from_scales = from + (uint64_t)outputs * inputs / 2u;
    unsigned char *to_scales = to + (uint64_t)outputs * inputs / 2u;
    static const uint32_t input_of_byte[4] = {0, 8, 1, 9};
    memset(to, 0, (size_t)((uint64_t)outputs * inputs / 2u));
    for (uint32_t tile = 0; tile < tiles; tile++) {
        for (uint32_t step = 0; step < steps; step++) {
            for (uint32_t lane = 0; lane < 64u; lane++) {
                const uint32_t g = lane / 16u, o = lane % 16u;
                const unsigned char *mine = from + (((uint64_t)tile * steps + step) * 64u + lane) * 16u;
                for (uint32_t e = 0; e < 32u; e++) { /* nibble n of byte b of word T */
                    const uint32_t T = e / 8u, b = (e % 8u) / 2u, n = e % 2u;
                    const uint32_t code = (mine[4u * T + b] >> (4u * n)) & 15u;
                    const uint32_t input = 128u * step + 32u * g + 16u * n + 2u * T + input_of_byte[b];
                    /* where the reference holds (16 tile + o, input) */
                    const uint32_t within = input % 64u, j = within % 16u, r = o / 8u + 2u * (j / 8u), h = j % 2u;
                    const uint64_t word = ((((uint64_t)tile * loads + input / 64u) * 32u + 4u * (o % 8u) + (j % 8u) / 2u) * 4u + within / 16u);
                    const uint32_t bit = 4u * r + 16u * h;
                    to[word * 4u + bit / 8u] |= (unsigned char)(code << (bit % 8u));
                }
                const uint64_t load = (uint64_t)tile * loads + 2u * step + g / 2u;
                to_scales[(load * 8u + o % 8u) * 4u + 2u * (g % 2u) + o / 8u] = from_scales[e2m1_gfx950_scale_at(tile, step, steps, lane)];
            }
        }
    }
}

/* E4M3: byte c of word v of lane 16 g + o is byte 8 (g % 2) + 4 (c % 2) + 2 (c / 2) + o / 8 of the reference's lane
 * 4 (o % 8) + v % 4 of the group 4 step + 2 (v / 4) + g / 2; the scale codes stay where they are */
static void e4m3_between(uint32_t outputs, uint32_t inputs, const unsigned char *from, unsigned char *to, bool to_gfx950, uint64_t scale_bytes)
{
    const uint32_t tiles = outputs / 16u, steps = inputs / 128u, groups = inputs / 32u;
    for (uint32_t tile = 0; tile < tiles; tile++) {
        for (uint32_t step = 0; step < steps; step++) {
            for (uint32_t lane = 0; lane < 64u; lane++) {
                const uint32_t g = lane / 16u, o = lane % 16u;
                for (uint32_t v = 0; v < 8u; v++) {
                    const uint64_t group = (uint64_t)tile * groups + 4u * step + 2u * (v / 4u) + g / 2u;
                    for (uint32_t c = 0; c < 4u; c++) {
                        const uint64_t reference = (group * 32u + 4u * (o % 8u) + v % 4u) * 16u + 8u * (g % 2u) + 4u * (c % 2u) + 2u * (c / 2u) + o / 8u;
                        const uint64_t native = ((uint64_t)tile * steps + step) * 2048u + (v / 4u) * 1024u + lane * 16u + (v % 4u) * 4u + c;
                        if (to_gfx950) {
                            to[native] = from[reference];
                        } else {
                            to[reference] = from[native];
                        }
                    }
                }
            }
        }
    }
    const uint64_t codes = (uint64_t)outputs * inputs;
    memcpy(to + codes, from + codes, (size_t)scale_bytes); /* E8M0 rows or float32 blocks: where they are */
}

static result_status gfx950_move(enum weight_format_code format, const struct matrix_shape_record *shape, const void *from, uint64_t from_bytes,
                                 void *to, uint64_t to_bytes, bool to_gfx950)
{
    const struct weight_format_operations *operations =
        format == WEIGHT_FORMAT_E2M1_GFX950 || format == WEIGHT_FORMAT_E4M3_GFX950 || format == WEIGHT_FORMAT_E4M3_BLOCK128_GFX950
            ? weight_format_operations_of(format)
            : NULL;
    uint64_t bytes = 0;
    if (operations == NULL || from == NULL || to == NULL || operations->stored_byte_count(shape, &bytes) != STATUS_OK || from_bytes != bytes ||
        to_bytes != bytes || !apart(from, from_bytes, to, to_bytes)) {
        return STATUS_INVALID_ARGUMENT; /* the _SCALED counterpart's byte count is the same for every shape both store */
    }
    if (format == WEIGHT_FORMAT_E4M3_GFX950 || format == WEIGHT_FORMAT_E4M3_BLOCK128_GFX950) {
        e4m3_between(shape->output_size, shape->input_size, from, to, to_gfx950, bytes - (uint64_t)shape->output_size * shape->input_size);
    } else if (to_gfx950) {
        e2m1_to_gfx950(shape->output_size, shape->input_size, from, to);
    } else {
        e2m1_from_gfx950(shape->output_size, shape->input_size, from, to);
    }
    return STATUS_OK;
}

result_status weight_format_gfx950_pack(enum weight_format_code format, const struct matrix_shape_record *shape, const void *reference_bytes,
                                        uint64_t reference_byte_count, void *packed_out, uint64_t packed_byte_count)
{
    return gfx950_move(format, shape, reference_bytes, reference_byte_count, packed_out, packed_byte_count, true);
}

result_status weight_format_gfx950_unpack(enum weight_format_code format, const struct matrix_shape_record *shape, const void *packed_bytes,
                                          uint64_t packed_byte_count, void *reference_out, uint64_t reference_byte_count)
{
    return gfx950_move(format, shape, packed_bytes, packed_byte_count, reference_out, reference_byte_count, false);
}
