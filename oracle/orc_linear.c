/*
 * orc_linear.c -- CPU oracle of the FP4 / FP8 expert linears. Contract and citations: orc_linear.h.
 * TEST INFRASTRUCTURE, never the product path. Build with -ffp-contract=off.
 */
#include "orc_linear.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#include "orc_common.h"
#include "orc_exl3.h" /* orc_expf */

#define BLOCK 32u

static int holds_nibbles(int format)
{
    return format == ORC_FORMAT_E2M1_SCALED || format == ORC_FORMAT_E2M1_GFX950;
}

static int holds_float_scales(int format)
{
    return format == ORC_FORMAT_E4M3_BLOCK128 || format == ORC_FORMAT_E4M3_BLOCK128_GFX950;
}

static int bytes_in_lane_order(int format)
{
    return format == ORC_FORMAT_E4M3_GFX950 || format == ORC_FORMAT_E4M3_BLOCK128_GFX950;
}

static int shape_is_stored(int format, uint32_t outputs, uint32_t inputs)
{
    if (outputs == 0u || inputs == 0u || outputs % 16u != 0u) {
        return 0;
    }
    if (format == ORC_FORMAT_E2M1_GFX950) {
        return inputs % 128u == 0u && outputs % 64u == 0u;
    }
    if (format == ORC_FORMAT_E4M3_GFX950) {
        return inputs % 128u == 0u && outputs % 32u == 0u;
    }
    if (format == ORC_FORMAT_E2M1_SCALED) {
        return inputs % 64u == 0u;
    }
    if (format == ORC_FORMAT_E4M3_SCALED) {
        return inputs % 32u == 0u;
    }
    if (holds_float_scales(format)) {
        return inputs % 128u == 0u && outputs % 128u == 0u;
    }
    return 0;
}

uint64_t orc_linear_scale_count(int format, uint32_t outputs, uint32_t inputs)
{
    if (holds_nibbles(format)) {
        return (uint64_t)outputs * (inputs / BLOCK);
    }
    if (holds_float_scales(format)) {
        return (uint64_t)(outputs / 128u) * (inputs / 128u) * 4u; /* float32 scales, counted in bytes */
    }
    return (uint64_t)((outputs + 31u) / 32u) * (inputs / BLOCK);
}

uint64_t orc_linear_stored_bytes(int format, uint32_t outputs, uint32_t inputs)
{
    const uint64_t weights = (uint64_t)outputs * inputs;
    return (holds_nibbles(format) ? weights / 2u : weights) + orc_linear_scale_count(format, outputs, inputs);
}

/* ---- lay-out: walk the stored words and ask which weight lies in each ---- */

int orc_linear_lay_out(int format, uint32_t outputs, uint32_t inputs, const uint8_t *codes,
                       const uint8_t *scale_codes, uint8_t *stored)
{
    if (!shape_is_stored(format, outputs, inputs)) {
        return -1;
    }
    const uint32_t tiles = outputs / 16u;
    if (format == ORC_FORMAT_E2M1_GFX950 || bytes_in_lane_order(format)) {
        /* walk the stored bytes of the definition and ask which weight lies in each */
        static const uint32_t input_of_byte[4] = {0, 8, 1, 9};
        const uint32_t steps = inputs / 128u;
        uint64_t at = 0;
        for (uint32_t tile = 0; tile < tiles; tile++) {
            for (uint32_t step = 0; step < steps; step++) {
                if (format == ORC_FORMAT_E2M1_GFX950) {
                    for (uint32_t lane = 0; lane < 64u; lane++) {
                        for (uint32_t T = 0; T < 4u; T++) {
                            for (uint32_t b = 0; b < 4u; b++, at++) {
                                uint32_t byte = 0;
                                for (uint32_t n = 0; n < 2u; n++) {
                                    const uint32_t input = 128u * step + 32u * (lane / 16u) + 16u * n + 2u * T + input_of_byte[b];
                                    const uint32_t code = codes[(uint64_t)(16u * tile + lane % 16u) * inputs + input];
                                    if (code > 15u) {
                                        return -1;
                                    }
                                    byte |= code << (4u * n);
                                }
                                stored[at] = (uint8_t)byte;
                            }
                        }
                    }
                } else {
                    for (uint32_t half = 0; half < 2u; half++) {
                        for (uint32_t lane = 0; lane < 64u; lane++) {
                            for (uint32_t k = 0; k < 16u; k++, at++) {
                                const uint32_t v = 4u * half + k / 4u, c = k % 4u;
                                const uint32_t input = 128u * step + 64u * (v / 4u) + 16u * (lane / 16u) + 8u * (c % 2u) + 2u * (v % 4u) + c / 2u;
                                stored[at] = codes[(uint64_t)(16u * tile + lane % 16u) * inputs + input];
                            }
                        }
                    }
                }
            }
        }
        if (bytes_in_lane_order(format)) { /* the scale codes, or the float32 scales, as they come */
            memcpy(stored + at, scale_codes, orc_linear_scale_count(format, outputs, inputs));
            return 0;
        }
        for (uint32_t group = 0; group < tiles / 4u; group++) { /* a word a lane a K step of a group of four tiles */
            for (uint32_t step = 0; step < steps; step++) {
                for (uint32_t lane = 0; lane < 64u; lane++) {
                    for (uint32_t n = 0; n < 4u; n++, at++) {
                        stored[at] = scale_codes[(uint64_t)(16u * (4u * group + n) + lane % 16u) * (inputs / BLOCK) + 4u * step + lane / 16u];
                    }
                }
            }
        }
        return 0;
    }
    if (format == ORC_FORMAT_E2M1_SCALED) {
        const uint32_t loads = inputs / 64u;
        uint64_t at = 0;
        for (uint32_t tile = 0; tile < tiles; tile++) {
            for (uint32_t load = 0; load < loads; load++) {
                for (uint32_t lane = 0; lane < 32u; lane++) {
                    const uint32_t g = lane / 4u, t = lane % 4u;
                    for (uint32_t step = 0; step < 4u; step++, at += 4u) {
                        uint32_t word = 0;
                        for (uint32_t r = 0; r < 4u; r++) {
                            for (uint32_t h = 0; h < 2u; h++) {
                                const uint32_t output = 16u * tile + g + 8u * (r % 2u);
                                const uint32_t input = 64u * load + 16u * step + 2u * t + 8u * (r / 2u) + h;
                                const uint32_t code = codes[(uint64_t)output * inputs + input];
                                if (code > 15u) {
                                    return -1;
                                }
                                word |= code << (4u * r + 16u * h);
                            }
                        }
                        memcpy(stored + at, &word, 4u);
                    }
                }
            }
        }
        for (uint32_t tile = 0; tile < tiles; tile++) {
            for (uint32_t load = 0; load < loads; load++) {
                for (uint32_t g = 0; g < 8u; g++, at += 4u) {
                    for (uint32_t q = 0; q < 2u; q++) {
                        for (uint32_t r = 0; r < 2u; r++) {
                            const uint32_t output = 16u * tile + g + 8u * r;
                            stored[at + 2u * q + r] = scale_codes[(uint64_t)output * (inputs / BLOCK) + 2u * load + q];
                        }
                    }
                }
            }
        }
        return 0;
    }
    const uint32_t groups = inputs / 32u;
    uint64_t at = 0;
    for (uint32_t tile = 0; tile < tiles; tile++) {
        for (uint32_t group = 0; group < groups; group++) {
            for (uint32_t lane = 0; lane < 32u; lane++) {
                const uint32_t g = lane / 4u, t = lane % 4u;
                for (uint32_t b = 0; b < 16u; b++, at++) {
                    const uint32_t output = 16u * tile + g + 8u * (b % 2u);
                    const uint32_t input = 32u * group + 8u * (b / 4u) + 2u * t + (b / 2u) % 2u;
                    stored[at] = codes[(uint64_t)output * inputs + input];
                }
            }
        }
    }
    memcpy(stored + at, scale_codes, orc_linear_scale_count(format, outputs, inputs));
    return 0;
}

/* ---- read: from a weight to its byte ---- */

int orc_linear_read(int format, uint32_t outputs, uint32_t inputs, const uint8_t *stored, uint32_t output,
                    uint32_t input, uint32_t *code_out, uint32_t *scale_out)
{
    if (!shape_is_stored(format, outputs, inputs) || output >= outputs || input >= inputs) {
        return -1;
    }
    const uint32_t tile = output / 16u, in_tile = output % 16u, g = in_tile % 8u, far_output = in_tile / 8u;
    if (format == ORC_FORMAT_E2M1_GFX950) {
        /* input = 128 step + 32 G + 16 n + r with r = 2 T + {0, 8, 1, 9}[b]: r below 8 is 2 T + (0 or 1), else 2 T + (8 or 9) */
        const uint32_t steps = inputs / 128u, step = input / 128u, G = (input % 128u) / 32u, n = (input % 32u) / 16u, r = input % 16u;
        const uint32_t T = (r % 8u) / 2u, b = 2u * (r % 2u) + r / 8u, lane = 16u * G + in_tile;
        *code_out = (stored[(((uint64_t)tile * steps + step) * 64u + lane) * 16u + 4u * T + b] >> (4u * n)) & 15u;
        *scale_out = stored[(uint64_t)outputs * inputs / 2u + ((((uint64_t)(tile / 4u) * steps + step) * 64u + lane) * 4u + tile % 4u)];
        return 0;
    }
    if (bytes_in_lane_order(format)) {
        /* input = 128 step + 64 half + 16 G + r with r = 8 (c % 2) + 2 (v % 4) + c / 2 */
        const uint32_t steps = inputs / 128u, step = input / 128u, half = (input % 128u) / 64u, G = (input % 64u) / 16u, r = input % 16u;
        const uint32_t word = (r % 8u) / 2u, c = 2u * (r % 2u) + r / 8u, lane = 16u * G + in_tile;
        *code_out = stored[((uint64_t)tile * steps + step) * 2048u + half * 1024u + lane * 16u + word * 4u + c];
        if (holds_float_scales(format)) {
            memcpy(scale_out, stored + (uint64_t)outputs * inputs + ((uint64_t)(output / 128u) * steps + step) * 4u, 4u);
            return 0;
        }
        *scale_out = stored[(uint64_t)outputs * inputs + (uint64_t)(output / 32u) * (inputs / BLOCK) + input / BLOCK];
        return 0;
    }
    if (format == ORC_FORMAT_E2M1_SCALED) {
        const uint32_t loads = inputs / 64u, load = input / 64u, within = input % 64u;
        const uint32_t step = within / 16u, j = within % 16u;
        const uint32_t t = (j % 8u) / 2u, h = j % 2u, r = far_output + 2u * (j / 8u);
        const uint64_t word_index = (((uint64_t)tile * loads + load) * 32u + 4u * g + t) * 4u + step;
        uint32_t word;
        memcpy(&word, stored + word_index * 4u, 4u);
        *code_out = (word >> (4u * r + 16u * h)) & 15u;
        const uint64_t scales = (uint64_t)outputs * inputs / 2u;
        *scale_out = stored[scales + (((uint64_t)tile * loads + load) * 8u + g) * 4u + 2u * (within / 32u) + far_output];
        return 0;
    }
    const uint32_t groups = inputs / 32u, group = input / 32u, within = input % 32u;
    const uint32_t t = (within % 8u) / 2u;
    const uint32_t b = 4u * (within / 8u) + 2u * (within % 2u) + far_output;
    *code_out = stored[(((uint64_t)tile * groups + group) * 32u + 4u * g + t) * 16u + b];
    if (format == ORC_FORMAT_E4M3_BLOCK128) { /* the float32 scale of the weight's 128 x 128 block, as its bits */
        memcpy(scale_out, stored + (uint64_t)outputs * inputs + ((uint64_t)(output / 128u) * (inputs / 128u) + input / 128u) * 4u, 4u);
        return 0;
    }
    *scale_out = stored[(uint64_t)outputs * inputs + (uint64_t)(output / 32u) * groups + group];
    return 0;
}

/* ---- activation quantizer ---- */

static uint32_t nearest_e4m3_magnitude(double magnitude)
{
    /* exhaustive over the 127 magnitudes 0x00..0x7E; of two equally near, the even code */
    uint32_t nearest = 0;
    double least = magnitude;
    for (uint32_t code = 1; code < 127u; code++) {
        const double distance = fabs(orc_e4m3_value(code) - magnitude);
        if (distance < least || (distance == least && (code & 1u) == 0u)) {
            nearest = code;
            least = distance;
        }
    }
    return nearest;
}

int orc_act_quantize(const uint16_t *values_bf16, uint32_t width, uint8_t *codes_out, uint8_t *exponents_out)
{
    if (width == 0u || width % BLOCK != 0u) {
        return -1;
    }
    for (uint32_t block = 0; block < width / BLOCK; block++) {
        const uint16_t *values = values_bf16 + block * BLOCK;
        float largest = 1e-4f;
        for (uint32_t i = 0; i < BLOCK; i++) {
            const float magnitude = orc_bf16_to_float(values[i] & 0x7FFFu);
            if (!(magnitude <= 3.4e38f)) {
                return -1; /* an infinity or a not-a-number */
            }
            largest = magnitude > largest ? magnitude : largest;
        }
        const float m = largest * (1.0f / 448.0f);
        /* the smallest power of two that is not below m */
        int exponent;
        const double fraction = frexp((double)m, &exponent); /* m = fraction 2^exponent, fraction in [1/2, 1) */
        const int power = fraction == 0.5 ? exponent - 1 : exponent;
        const uint32_t scale_code = (uint32_t)(power + 127);
        exponents_out[block] = (uint8_t)scale_code;
        for (uint32_t i = 0; i < BLOCK; i++) {
            double scaled = ldexp((double)orc_bf16_to_float(values[i] & 0x7FFFu), -power);
            if (scaled > 448.0) {
                scaled = 448.0;
            }
            codes_out[block * BLOCK + i] = (uint8_t)(nearest_e4m3_magnitude(scaled) | ((values[i] & 0x8000u) ? 0x80u : 0u));
        }
    }
    return 0;
}

void orc_codes_lane_order(const uint8_t *codes, uint32_t width, uint8_t *stored_out)
{
    /* byte ((4 l + t) 4 + s) 4 + j holds the code of value 64 l + 16 s + 2 t + j / 2 + 8 (j % 2) */
    for (uint32_t at = 0; at < width; at++) {
        const uint32_t j = at % 4u, s = (at / 4u) % 4u, t = (at / 16u) % 4u, l = at / 64u;
        stored_out[at] = codes[64u * l + 16u * s + 2u * t + j / 2u + 8u * (j % 2u)];
    }
}

void orc_operands_lay_out(const uint8_t *codes, const uint8_t *exponents, uint32_t width, uint16_t *operands_out)
{
    /* half ((4 l + t) 4 + s) 4 + 2 r + h holds the operand of value 64 l + 16 s + 2 t + h + 8 r: the bf16 of
     * value(code) 2^(c - 127) 2^100, the sign kept; an infinity of the sign where c is above 146 */
    for (uint32_t at = 0; at < width; at++) {
        const uint32_t h = at % 2u, r = (at / 2u) % 2u, s = (at / 4u) % 4u, t = (at / 16u) % 4u, l = at / 64u;
        const uint32_t value = 64u * l + 16u * s + 2u * t + h + 8u * r;
        const uint32_t code = codes[value], exponent = exponents[value / BLOCK];
        const uint16_t sign = (code & 0x80u) ? 0x8000u : 0u;
        if (exponent > 146u) {
            operands_out[at] = (uint16_t)(sign | 0x7F80u);
        } else {
            const double magnitude = ldexp(orc_e4m3_value(code & 0x7Fu), (int)exponent - 127 + 100);
            operands_out[at] = (uint16_t)(sign | (orc_bf16_from_float((float)magnitude) & 0x7FFFu));
        }
    }
}

/* ---- products ---- */

/* one tile of 16 outputs, every input: values_out [16][inputs] doubles of the codes, scales_out [16][inputs/32] */
static void tile_values(int format, uint32_t outputs, uint32_t inputs, const uint8_t *stored, uint32_t tile,
                        float *values_out, int *scale_exponents_out)
{
    for (uint32_t o = 0; o < 16u; o++) {
        for (uint32_t input = 0; input < inputs; input++) {
            uint32_t code, scale;
            (void)orc_linear_read(format, outputs, inputs, stored, 16u * tile + o, input, &code, &scale);
            values_out[(uint64_t)o * inputs + input] =
                (float)(holds_nibbles(format) ? orc_e2m1_value(code) : orc_e4m3_value(code));
            if (input % BLOCK == 0u) {
                scale_exponents_out[o * (inputs / BLOCK) + input / BLOCK] = (int)scale - 127;
            }
        }
    }
}

int orc_linear_products(int format, uint32_t outputs, uint32_t inputs, const uint8_t *stored, uint32_t first,
                        uint32_t count, const uint8_t *fed_codes, const uint8_t *fed_exponents, uint32_t vectors,
                        double *sums_out, double *magnitude_out)
{
    if (!shape_is_stored(format, outputs, inputs) || first % 16u != 0u || count % 16u != 0u ||
        first + count > outputs) {
        return -1;
    }
    const uint32_t blocks = inputs / BLOCK;
    float *values = malloc((size_t)16u * inputs * sizeof *values);
    int *scales = malloc((size_t)16u * blocks * sizeof *scales);
    float *fed = malloc((size_t)vectors * inputs * sizeof *fed);
    for (uint64_t i = 0; i < (uint64_t)vectors * inputs; i++) {
        fed[i] = (float)orc_e4m3_value(fed_codes[i]);
    }
    for (uint32_t tile = first / 16u; tile < (first + count) / 16u; tile++) {
        tile_values(format, outputs, inputs, stored, tile, values, scales);
        for (uint32_t v = 0; v < vectors; v++) {
            for (uint32_t o = 0; o < 16u; o++) {
                double sum = 0.0, magnitude = 0.0;
                for (uint32_t block = 0; block < blocks; block++) {
                    double block_sum = 0.0, block_magnitude = 0.0; /* exact: 41 bits hold it */
                    for (uint32_t i = 0; i < BLOCK; i++) {
                        const double product = (double)values[(uint64_t)o * inputs + block * BLOCK + i] *
                                               (double)fed[(uint64_t)v * inputs + block * BLOCK + i];
                        block_sum += product;
                        block_magnitude += fabs(product);
                    }
                    const int power = scales[o * blocks + block] + (int)fed_exponents[(uint64_t)v * blocks + block] - 127;
                    sum += ldexp(block_sum, power);
                    magnitude += ldexp(block_magnitude, power);
                }
                const uint64_t at = (uint64_t)v * count + (16u * tile - first) + o;
                sums_out[at] = sum;
                if (magnitude_out != NULL) {
                    magnitude_out[at] = magnitude;
                }
            }
        }
    }
    free(values);
    free(scales);
    free(fed);
    return 0;
}

int orc_linear_products_128_of(int format, uint32_t outputs, uint32_t inputs, const uint8_t *stored, uint32_t first,
                               uint32_t count, const uint8_t *fed_codes, const float *fed_scales, uint32_t vectors,
                               double *sums_out, double *magnitude_out)
{
    if (!holds_float_scales(format) || !shape_is_stored(format, outputs, inputs) || first + count > outputs) {
        return -1;
    }
    const uint32_t blocks = inputs / 128u;
    float *values = malloc((size_t)inputs * sizeof *values), *scales = malloc((size_t)blocks * sizeof *scales);
    for (uint32_t o = first; o < first + count; o++) {
        for (uint32_t input = 0; input < inputs; input++) {
            uint32_t code, scale;
            (void)orc_linear_read(format, outputs, inputs, stored, o, input, &code, &scale);
            values[input] = (float)orc_e4m3_value(code);
            if (input % 128u == 0u) {
                scales[input / 128u] = orc_f32_from_bits(scale);
            }
        }
        for (uint32_t v = 0; v < vectors; v++) {
            double sum = 0.0, magnitude = 0.0;
            for (uint32_t block = 0; block < blocks; block++) {
                double block_sum = 0.0, block_magnitude = 0.0; /* exact */
                for (uint32_t i = 0; i < 128u; i++) {
                    const double product = (double)values[block * 128u + i] * orc_e4m3_value(fed_codes[(uint64_t)v * inputs + block * 128u + i]);
                    block_sum += product;
                    block_magnitude += fabs(product);
                }
                const double w_scale = (double)scales[block], a_scale = (double)fed_scales[(uint64_t)v * blocks + block];
                sum += block_sum * w_scale * a_scale;
                magnitude += block_magnitude * fabs(w_scale) * fabs(a_scale);
            }
            sums_out[(uint64_t)v * count + (o - first)] = sum;
            if (magnitude_out != NULL) {
                magnitude_out[(uint64_t)v * count + (o - first)] = magnitude;
            }
        }
    }
    free(values);
    free(scales);
    return 0;
}

int orc_linear_products_128(uint32_t outputs, uint32_t inputs, const uint8_t *stored, uint32_t first, uint32_t count,
                            const uint8_t *fed_codes, const float *fed_scales, uint32_t vectors, double *sums_out,
                            double *magnitude_out)
{
    return orc_linear_products_128_of(ORC_FORMAT_E4M3_BLOCK128, outputs, inputs, stored, first, count, fed_codes, fed_scales,
                                      vectors, sums_out, magnitude_out);
}

static double bf16_last_place(uint16_t bits)
{
    const int exponent = (int)((bits >> 7) & 255u);
    return ldexp(1.0, (exponent == 0 ? 1 : exponent) - 127 - 7);
}

int orc_linear_within_tolerance(uint16_t output_bf16, double sum, double magnitude, uint32_t inputs, uint32_t slices)
{
    return orc_linear_within_allowance(output_bf16, sum, magnitude, inputs, slices, 64.0);
}

int orc_linear_within_allowance(uint16_t output_bf16, double sum, double magnitude, uint32_t inputs, uint32_t slices,
                                double allowance)
{
    /* bound = (T + B + S) 2^-24 m + B 2^-149; |c - y| <= last_place(c) / 2 + bound */
    const double blocks = inputs / BLOCK;
    const double bound = (allowance + blocks + slices) * ldexp(1.0, -24) * magnitude + blocks * ldexp(1.0, -149);
    const double c = (double)orc_bf16_to_float(output_bf16);
    if (c != c || sum != sum) {
        return c != c && sum != sum;
    }
    return fabs(c - sum) <= bf16_last_place(output_bf16) / 2.0 + bound;
}

/* ---- hidden step, row sum ---- */

double orc_hidden_value(double gate, double up, double limit, double route_weight)
{
    const double g = gate > limit ? limit : gate;
    const double u = up > limit ? limit : (up < -limit ? -limit : up);
    if (g != g) {
        return g;
    }
    double gated;
    if (-g > 128.0 * 0.6931471805599453) {
        gated = -0.0; /* a float32 exponential is infinite there */
    } else {
        gated = g / (1.0 + exp(-g));
    }
    return gated * u * route_weight;
}

uint16_t orc_hidden_bits(float gate, float up, float limit, float route_weight)
{
    const float g = orc_bf16_to_float(orc_bf16_from_float(gate)), u = orc_bf16_to_float(orc_bf16_from_float(up));
    const float bounded_gate = fminf(g, limit);
    const float bounded_up = fminf(fmaxf(u, -limit), limit);
    const float hidden = ((bounded_gate / (1.0f + orc_expf(-bounded_gate))) * bounded_up) * route_weight;
    return orc_bf16_from_float(hidden);
}

float orc_row_sum_bf16(const uint16_t *pair_outputs, uint32_t pairs, uint32_t width, uint32_t column)
{
    float sum = 0.0f;
    for (uint32_t slot = 0; slot < pairs; slot++) {
        sum = sum + orc_bf16_to_float(pair_outputs[(uint64_t)slot * width + column]);
    }
    return sum;
}

/* ---- 128-block fp32-scale FP8 mode ---- */

static uint8_t e4m3_nearest_code(double value)
{
    double magnitude = fabs(value);
    if (magnitude > 448.0) {
        magnitude = 448.0;
    }
    return (uint8_t)(nearest_e4m3_magnitude(magnitude) | (signbit(value) ? 0x80u : 0u));
}

void orc_act_quantize_128(const uint16_t *values_bf16, uint32_t width, uint8_t *codes_out, float *scales_out)
{
    for (uint32_t block = 0; block < width / 128u; block++) {
        float largest = 1e-4f;
        for (uint32_t i = 0; i < 128u; i++) {
            const float magnitude = orc_bf16_to_float(values_bf16[block * 128u + i] & 0x7FFFu);
            largest = magnitude > largest ? magnitude : largest;
        }
        const float scale = largest / 448.0f;
        scales_out[block] = scale;
        for (uint32_t i = 0; i < 128u; i++) {
            const float scaled = orc_bf16_to_float(values_bf16[block * 128u + i]) / scale; /* one float32 rounding */
            codes_out[block * 128u + i] = e4m3_nearest_code((double)scaled);
        }
    }
}

void orc_fp8_block128_products(uint32_t outputs, uint32_t inputs, const uint8_t *w_codes, const float *w_scales,
                               const uint8_t *a_codes, const float *a_scales, uint32_t vectors, double *sums_out)
{
    const uint32_t blocks = inputs / 128u;
    for (uint32_t v = 0; v < vectors; v++) {
        for (uint32_t o = 0; o < outputs; o++) {
            double sum = 0.0;
            for (uint32_t block = 0; block < blocks; block++) {
                double block_sum = 0.0;
                for (uint32_t i = 0; i < 128u; i++) {
                    block_sum += orc_e4m3_value(w_codes[(uint64_t)o * inputs + block * 128u + i]) *
                                 orc_e4m3_value(a_codes[(uint64_t)v * inputs + block * 128u + i]);
                }
                sum += block_sum * (double)w_scales[(uint64_t)(o / 128u) * blocks + block] *
                       (double)a_scales[(uint64_t)v * blocks + block];
            }
            sums_out[(uint64_t)v * outputs + o] = sum;
        }
    }
}

/* ---- the layer ---- */

struct linear_layer {
    int format;
    const uint16_t *x_bf16;
    uint32_t rows, hidden, inner, picks, expert_count;
    const uint32_t *experts;
    const float *weights;
    const uint8_t *const *matrices;
    float limit;
    uint16_t *hidden_out, *pair_out;
    uint8_t *x_codes, *x_exponents; /* [rows][hidden], [rows][hidden/32] */
    uint32_t next_expert;
    pthread_mutex_t lock;
};

/* the quantizer and the product of the layer's format: E8M0 scale codes a 32 values, or float32 scales a 128 (the
 * scale arrays have the same bytes either way: width / 32 a vector) */
static void layer_quantize(int format, const uint16_t *values, uint32_t width, uint8_t *codes, uint8_t *scales)
{
    if (holds_float_scales(format)) {
        orc_act_quantize_128(values, width, codes, (float *)(void *)scales);
    } else {
        (void)orc_act_quantize(values, width, codes, scales);
    }
}

static void layer_products(int format, uint32_t outputs, uint32_t inputs, const uint8_t *stored, const uint8_t *codes,
                           const uint8_t *scales, uint32_t vectors, double *sums)
{
    if (holds_float_scales(format)) {
        (void)orc_linear_products_128_of(format, outputs, inputs, stored, 0, outputs, codes, (const float *)(const void *)scales, vectors, sums, NULL);
    } else {
        (void)orc_linear_products(format, outputs, inputs, stored, 0, outputs, codes, scales, vectors, sums, NULL);
    }
}

static void linear_expert(struct linear_layer *layer, uint32_t expert)
{
    const uint32_t H = layer->hidden, I = layer->inner, total = layer->rows * layer->picks;
    uint32_t *pairs = malloc(total * sizeof *pairs), count = 0;
    for (uint32_t pair = 0; pair < total; pair++) {
        if (layer->experts[pair] == expert) {
            pairs[count++] = pair;
        }
    }
    if (count == 0u) {
        free(pairs);
        return;
    }
    uint8_t *codes = malloc((size_t)count * (H > I ? H : I)), *exponents = malloc((size_t)count * (H > I ? H : I) / BLOCK);
    double *gate = malloc((size_t)count * I * sizeof(double)), *up = malloc((size_t)count * I * sizeof(double));
    double *down = malloc((size_t)count * H * sizeof(double));
    uint16_t *hidden = malloc((size_t)count * I * sizeof(uint16_t));
    for (uint32_t c = 0; c < count; c++) {
        const uint32_t row = pairs[c] / layer->picks;
        memcpy(codes + (uint64_t)c * H, layer->x_codes + (uint64_t)row * H, H);
        memcpy(exponents + (uint64_t)c * (H / BLOCK), layer->x_exponents + (uint64_t)row * (H / BLOCK), H / BLOCK);
    }
    layer_products(layer->format, I, H, layer->matrices[expert * 3u + 0u], codes, exponents, count, gate);
    layer_products(layer->format, I, H, layer->matrices[expert * 3u + 1u], codes, exponents, count, up);
    for (uint32_t c = 0; c < count; c++) {
        for (uint32_t i = 0; i < I; i++) {
            /* the products are rounded once to bfloat16, then the hidden step in float32 */
            const float g = orc_bf16_to_float(orc_bf16_from_float((float)gate[(uint64_t)c * I + i]));
            const float u = orc_bf16_to_float(orc_bf16_from_float((float)up[(uint64_t)c * I + i]));
            hidden[(uint64_t)c * I + i] = orc_hidden_bits(g, u, layer->limit, layer->weights[pairs[c]]);
        }
        if (layer->hidden_out != NULL) {
            memcpy(layer->hidden_out + (uint64_t)pairs[c] * I, hidden + (uint64_t)c * I, I * sizeof(uint16_t));
        }
        layer_quantize(layer->format, hidden + (uint64_t)c * I, I, codes + (uint64_t)c * I, exponents + (uint64_t)c * (I / BLOCK));
    }
    layer_products(layer->format, H, I, layer->matrices[expert * 3u + 2u], codes, exponents, count, down);
    for (uint32_t c = 0; c < count; c++) {
        for (uint32_t i = 0; i < H; i++) {
            layer->pair_out[(uint64_t)pairs[c] * H + i] = orc_bf16_from_float((float)down[(uint64_t)c * H + i]);
        }
    }
    free(pairs);
    free(codes);
    free(exponents);
    free(gate);
    free(up);
    free(down);
    free(hidden);
}

static void *linear_worker(void *argument)
{
    struct linear_layer *layer = argument;
    for (;;) {
        pthread_mutex_lock(&layer->lock);
        const uint32_t expert = layer->next_expert++;
        pthread_mutex_unlock(&layer->lock);
        if (expert >= layer->expert_count) {
            return NULL;
        }
        linear_expert(layer, expert);
    }
}

void orc_linear_moe_layer(int format, const uint16_t *x_bf16, uint32_t rows, uint32_t hidden, uint32_t inner,
                          uint32_t picks, const uint32_t *experts, const float *weights, uint32_t expert_count,
                          const uint8_t *const *matrices, float limit, float *out_rows, uint16_t *hidden_out,
                          uint16_t *pair_out, uint32_t threads)
{
    struct linear_layer layer = {.format = format, .x_bf16 = x_bf16, .rows = rows, .hidden = hidden, .inner = inner,
                                 .picks = picks, .expert_count = expert_count, .experts = experts,
                                 .weights = weights, .matrices = matrices, .limit = limit,
                                 .hidden_out = hidden_out, .next_expert = 0};
    uint16_t *own_pairs = NULL;
    pthread_t workers[64];
    if (pair_out == NULL) {
        own_pairs = calloc((size_t)rows * picks * hidden, sizeof(uint16_t));
        pair_out = own_pairs;
    }
    layer.pair_out = pair_out;
    layer.x_codes = malloc((size_t)rows * hidden);
    layer.x_exponents = malloc((size_t)rows * hidden / BLOCK);
    for (uint32_t row = 0; row < rows; row++) {
        layer_quantize(format, x_bf16 + (uint64_t)row * hidden, hidden, layer.x_codes + (uint64_t)row * hidden,
                       layer.x_exponents + (uint64_t)row * (hidden / BLOCK));
    }
    pthread_mutex_init(&layer.lock, NULL);
    threads = threads < 1u ? 1u : (threads > 64u ? 64u : threads);
    for (uint32_t t = 1; t < threads; t++) {
        pthread_create(&workers[t], NULL, linear_worker, &layer);
    }
    (void)linear_worker(&layer);
    for (uint32_t t = 1; t < threads; t++) {
        pthread_join(workers[t], NULL);
    }
    pthread_mutex_destroy(&layer.lock);
    for (uint32_t row = 0; row < rows; row++) {
        for (uint32_t column = 0; column < hidden; column++) {
            out_rows[(uint64_t)row * hidden + column] =
                orc_row_sum_bf16(pair_out + (uint64_t)row * picks * hidden, picks, hidden, column);
        }
    }
    free(layer.x_codes);
    free(layer.x_exponents);
    free(own_pairs);
}
