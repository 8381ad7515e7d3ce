/*
 * orc_exl3.c -- CPU oracle of the EXL3 routed-expert linears. Contract and citations: orc_exl3.h.
 * TEST INFRASTRUCTURE, never the product path. Build with -ffp-contract=off: every float operation written here
 * is one rounding.
 */
#include "orc_exl3.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#include "orc_common.h"

#define TILE 16u
#define TILE_VALUES 256u
#define BLOCK 128u

/* ---- format ---- */

uint32_t orc_exl3_bits_x2(uint32_t stored_width)
{
    /* include/anemone/exl3_records.h:86-95 */
    if (stored_width >= 1u && stored_width <= 8u) {
        return 2u * stored_width;
    }
    if (stored_width % 16u == 8u && stored_width < 128u) {
        return stored_width / 8u;
    }
    return 0u;
}

uint32_t orc_exl3_window_end(uint32_t position, uint32_t bits_x2)
{
    /* S(i) = floor((i + 1) bits_x2 / 2): include/anemone/exl3_records.h:6-7,111-119 */
    return (position + 1u) * bits_x2 / 2u;
}

uint64_t orc_exl3_code_bytes(uint32_t inputs, uint32_t outputs, uint32_t stored_width)
{
    /* 16 x 16 tiles of 16 bits_x2 bytes: include/anemone/exl3_records.h:121-128 */
    return (uint64_t)inputs * outputs / 16u * orc_exl3_bits_x2(stored_width);
}

uint64_t orc_exl3_matrix_bytes(uint32_t inputs, uint32_t outputs, uint32_t stored_width)
{
    /* source/exl3.c:25-35: the codes, then fp16 suh[inputs], svh[outputs] */
    return orc_exl3_code_bytes(inputs, outputs, stored_width) + 2ull * ((uint64_t)inputs + outputs);
}

/* ---- codebook ---- */

uint16_t orc_exl3_codebook(uint32_t state)
{
    /* b = byte sum of state * 0x83DCD12D mod 2^32; value = fp16 fma(1024 + b, 0x1EEE, 0xC931), one rounding.
     * 0x1EEE is 1774 / 2^18 and 0xC931 is -10.3828125, so the exact value is (1774 b - 905216) / 2^18. */
    const uint32_t product = (state & 0xFFFFu) * 0x83DCD12Du;
    const uint32_t b = (product & 255u) + ((product >> 8) & 255u) + ((product >> 16) & 255u) + (product >> 24);
    const double exact = orc_half_value((uint16_t)(0x6400u + b)) * orc_half_value(0x1EEEu) + orc_half_value(0xC931u);
    return orc_half_from_double(exact); /* product and sum are exact in double: the one rounding is this */
}

static uint16_t codebook_table[65536];
static float codebook_floats[65536];
static pthread_once_t codebook_once = PTHREAD_ONCE_INIT;

static void codebook_fill(void)
{
    for (uint32_t state = 0; state < 65536u; state++) {
        codebook_table[state] = orc_exl3_codebook(state);
        codebook_floats[state] = orc_half_to_float(codebook_table[state]);
    }
}

/* ---- placement ---- */

void orc_exl3_place(uint32_t position, uint32_t *input, uint32_t *output)
{
    /* weight 8 t + m: input 2 (t % 4) + m % 2 + 8 (m / 2 % 2), output t / 4 + 8 (m / 4) */
    const uint32_t t = position / 8u, m = position % 8u;
    *input = 2u * (t % 4u) + (m & 1u) + 8u * ((m >> 1) & 1u);
    *output = t / 4u + 8u * (m >> 2);
}

uint32_t orc_exl3_position(uint32_t input, uint32_t output)
{
    const uint32_t t = 4u * (output % 8u) + (input % 8u) / 2u;
    const uint32_t m = (input & 1u) + 2u * (input / 8u) + 4u * (output / 8u);
    return 8u * t + m;
}

/* ---- ring ---- */

/* 32 stream bits from bit `at` of a cyclic ring of `word_count` words, stream bit b being bit 31 - b % 32 of word
 * b / 32 */
static uint32_t ring_bits32(const uint32_t *words, uint32_t word_count, uint32_t at)
{
    const uint32_t word = at / 32u, shift = at % 32u;
    uint32_t value = words[word] << shift;
    if (shift != 0u) {
        value |= words[(word + 1u) % word_count] >> (32u - shift);
    }
    return value;
}

void orc_exl3_tile_states(uint32_t bits_x2, const uint32_t *words, uint16_t *states)
{
    const uint32_t ring = TILE_VALUES * bits_x2 / 2u, word_count = ring / 32u;
    for (uint32_t position = 0; position < TILE_VALUES; position++) {
        const uint32_t begin = (orc_exl3_window_end(position, bits_x2) + ring - 16u) % ring;
        states[position] = (uint16_t)(ring_bits32(words, word_count, begin) >> 16);
    }
}

static void matrix_walk(const unsigned char *codes, uint32_t inputs, uint32_t outputs, uint32_t stored_width,
                        uint16_t *out, int decode)
{
    const uint32_t bits_x2 = orc_exl3_bits_x2(stored_width);
    const uint32_t tile_words = TILE_VALUES * bits_x2 / 2u / 32u;
    uint32_t words[128];
    uint16_t states[TILE_VALUES];
    (void)pthread_once(&codebook_once, codebook_fill);
    for (uint32_t kt = 0; kt < inputs / TILE; kt++) {
        for (uint32_t ot = 0; ot < outputs / TILE; ot++) {
            const uint64_t tile = (uint64_t)kt * (outputs / TILE) + ot;
            memcpy(words, codes + tile * tile_words * 4u, tile_words * 4u); /* little-endian host */
            orc_exl3_tile_states(bits_x2, words, states);
            for (uint32_t position = 0; position < TILE_VALUES; position++) {
                uint32_t input, output;
                orc_exl3_place(position, &input, &output);
                out[(uint64_t)(kt * TILE + input) * outputs + ot * TILE + output] =
                    decode ? codebook_table[states[position]] : states[position];
            }
        }
    }
}

void orc_exl3_states(const unsigned char *codes, uint32_t inputs, uint32_t outputs, uint32_t stored_width,
                     uint16_t *states_out)
{
    matrix_walk(codes, inputs, outputs, stored_width, states_out, 0);
}

void orc_exl3_decode_matrix(const unsigned char *codes, uint32_t inputs, uint32_t outputs, uint32_t stored_width,
                            uint16_t *weights_out)
{
    matrix_walk(codes, inputs, outputs, stored_width, weights_out, 1);
}

/* ---- H128 ---- */

void orc_h128_f32(float *values)
{
    /* seven stages, the distance doubling from 1; (lower, upper) -> (lower + upper, lower - upper); then each
     * value times float32(1/sqrt(128)) */
    for (uint32_t distance = 1; distance < BLOCK; distance *= 2u) {
        for (uint32_t index = 0; index < BLOCK; index++) {
            if ((index & distance) == 0u) {
                const float lower = values[index], upper = values[index + distance];
                values[index] = lower + upper;
                values[index + distance] = lower - upper;
            }
        }
    }
    for (uint32_t index = 0; index < BLOCK; index++) {
        values[index] = values[index] * ORC_EXL3_NORM;
    }
}

void orc_h128_f64(const double *values, double *rotated)
{
    /* element (from, to) of the Sylvester matrix is -1 where from & to has an odd number of bits */
    for (uint32_t to = 0; to < BLOCK; to++) {
        double sum = 0.0;
        for (uint32_t from = 0; from < BLOCK; from++) {
            sum += (__builtin_popcount(from & to) & 1) ? -values[from] : values[from];
        }
        rotated[to] = sum / sqrt(128.0);
    }
}

/* ---- exp ---- */

float orc_expf(float x)
{
    /* e^x = 2^k e^r, k = nearest(x log2 e), r = x - k ln2 in two pieces, e^r by a degree-7 polynomial in fma
     * form, scaled by ldexp (one rounding, subnormal results included) */
    if (x != x) {
        return x;
    }
    if (x > 88.8f) {
        return INFINITY;
    }
    if (x < -104.0f) {
        return 0.0f;
    }
    const float k = nearbyintf(x * 1.44269502162933349609375f);
    float r = fmaf(k, -0.693145751953125f, x);
    r = fmaf(k, -1.42860676533018704503775e-06f, r);
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    const float r2 = r * r;
    float y = fmaf(p, r2, r);
    y = y + 1.0f;
    return ldexpf(y, (int)k);
}

/* ---- chain stages ---- */

void orc_exl3_operand(const uint16_t *x_bf16, const uint16_t *suh_fp16, uint32_t width, uint16_t *operand_fp16)
{
    float block[BLOCK];
    for (uint32_t base = 0; base < width; base += BLOCK) {
        for (uint32_t i = 0; i < BLOCK; i++) {
            block[i] = orc_bf16_to_float(x_bf16[base + i]) * orc_half_to_float(suh_fp16[base + i]);
        }
        orc_h128_f32(block);
        for (uint32_t i = 0; i < BLOCK; i++) {
            operand_fp16[base + i] = orc_half_from_float(block[i]);
        }
    }
}

void orc_exl3_product(const uint16_t *weights, uint32_t inputs, uint32_t outputs, const uint16_t *operand_fp16,
                      uint32_t slices, int mode, float *products_out)
{
    const uint32_t tiles = inputs / TILE;
    for (uint32_t output = 0; output < outputs; output++) {
        if (mode == 0) {
            /* a product of two fp16 has 22 significant bits and the exponents span under 80 binades here, so
             * long double (64-bit significand) keeps far more than the float the sum is rounded to */
            long double sum = 0.0L;
            for (uint32_t input = 0; input < inputs; input++) {
                sum += (long double)orc_half_value(weights[(uint64_t)input * outputs + output]) *
                       (long double)orc_half_value(operand_fp16[input]);
            }
            products_out[output] = (float)sum;
        } else {
            float total = 0.0f;
            for (uint32_t slice = 0; slice < slices; slice++) {
                float running = 0.0f;
                const uint32_t end = tiles * (slice + 1u) / slices * TILE;
                for (uint32_t input = tiles * slice / slices * TILE; input < end; input++) {
                    const float product = orc_half_to_float(weights[(uint64_t)input * outputs + output]) *
                                          orc_half_to_float(operand_fp16[input]); /* exact in float */
                    running = running + product;
                }
                total = total + running;
            }
            products_out[output] = total;
        }
    }
}

/* Tile-streaming product in double: one pass over the stored codes, `columns` operand rows at once. */
static void product_codes(const unsigned char *codes, uint32_t inputs, uint32_t outputs, uint32_t stored_width,
                          const float *operands, uint32_t columns, float *products_out)
{
    const uint32_t bits_x2 = orc_exl3_bits_x2(stored_width);
    const uint32_t tile_words = TILE_VALUES * bits_x2 / 2u / 32u;
    const uint32_t out_tiles = outputs / TILE;
    double *sums = calloc((size_t)columns * outputs, sizeof *sums);
    uint16_t states[TILE_VALUES];
    float tile[TILE][TILE]; /* [input][output] */
    uint32_t words[128];
    (void)pthread_once(&codebook_once, codebook_fill);
    for (uint32_t kt = 0; kt < inputs / TILE; kt++) {
        for (uint32_t ot = 0; ot < out_tiles; ot++) {
            memcpy(words, codes + ((uint64_t)kt * out_tiles + ot) * tile_words * 4u, tile_words * 4u);
            orc_exl3_tile_states(bits_x2, words, states);
            for (uint32_t position = 0; position < TILE_VALUES; position++) {
                uint32_t input, output;
                orc_exl3_place(position, &input, &output);
                tile[input][output] = codebook_floats[states[position]];
            }
            for (uint32_t column = 0; column < columns; column++) {
                const float *x = operands + (uint64_t)column * inputs + kt * TILE;
                double *sum = sums + (uint64_t)column * outputs + ot * TILE;
                for (uint32_t input = 0; input < TILE; input++) {
                    const double xv = x[input];
                    for (uint32_t output = 0; output < TILE; output++) {
                        sum[output] += (double)tile[input][output] * xv;
                    }
                }
            }
        }
    }
    for (uint64_t i = 0; i < (uint64_t)columns * outputs; i++) {
        products_out[i] = (float)sums[i];
    }
    free(sums);
}

void orc_exl3_product_codes(const unsigned char *codes, uint32_t inputs, uint32_t outputs, uint32_t stored_width,
                            const uint16_t *operands_fp16, uint32_t columns, float *products_out)
{
    float *operands = malloc((size_t)columns * inputs * sizeof *operands);
    for (uint64_t i = 0; i < (uint64_t)columns * inputs; i++) {
        operands[i] = orc_half_to_float(operands_fp16[i]);
    }
    product_codes(codes, inputs, outputs, stored_width, operands, columns, products_out);
    free(operands);
}

void orc_exl3_activate(const float *gate_products, const float *up_products, const uint16_t *gate_svh,
                       const uint16_t *up_svh, const uint16_t *down_suh, uint32_t inner, float limit,
                       uint16_t *hidden_bf16_out, uint16_t *operand_fp16_out)
{
    float gate[BLOCK], up[BLOCK], next[BLOCK];
    for (uint32_t base = 0; base < inner; base += BLOCK) {
        memcpy(gate, gate_products + base, sizeof gate);
        memcpy(up, up_products + base, sizeof up);
        orc_h128_f32(gate); /* includes the normalisation */
        orc_h128_f32(up);
        for (uint32_t i = 0; i < BLOCK; i++) {
            const float g = gate[i] * orc_half_to_float(gate_svh[base + i]);
            const float u = up[i] * orc_half_to_float(up_svh[base + i]);
            const float bounded_gate = fminf(g, limit);
            const float bounded_up = fminf(fmaxf(u, -limit), limit);
            const float hidden = bounded_gate / (1.0f + orc_expf(-bounded_gate)) * bounded_up;
            if (hidden_bf16_out != NULL) {
                hidden_bf16_out[base + i] = orc_bf16_from_float(hidden);
            }
            next[i] = hidden * orc_half_to_float(down_suh[base + i]);
        }
        orc_h128_f32(next);
        for (uint32_t i = 0; i < BLOCK; i++) {
            operand_fp16_out[base + i] = orc_half_from_float(next[i]);
        }
    }
}

void orc_exl3_finish(const float *down_products, const uint16_t *down_svh, uint32_t width, float route_weight,
                     float *pair_out)
{
    float block[BLOCK];
    for (uint32_t base = 0; base < width; base += BLOCK) {
        memcpy(block, down_products + base, sizeof block);
        orc_h128_f32(block);
        for (uint32_t i = 0; i < BLOCK; i++) {
            const float value = block[i] * orc_half_to_float(down_svh[base + i]);
            pair_out[base + i] = value * route_weight;
        }
    }
}

void orc_exl3_row_sum(const float *pair_outputs, uint32_t rows, uint32_t pairs_per_row, uint32_t width,
                      float *rows_out)
{
    for (uint32_t row = 0; row < rows; row++) {
        for (uint32_t channel = 0; channel < width; channel++) {
            float sum = 0.0f;
            for (uint32_t slot = 0; slot < pairs_per_row; slot++) {
                sum = sum + pair_outputs[((uint64_t)row * pairs_per_row + slot) * width + channel];
            }
            rows_out[(uint64_t)row * width + channel] = sum;
        }
    }
}

void orc_exl3_linear_f64(const unsigned char *matrix, uint32_t inputs, uint32_t outputs, uint32_t stored_width,
                         const double *x, double *y)
{
    const uint16_t *suh = (const uint16_t *)(matrix + orc_exl3_code_bytes(inputs, outputs, stored_width));
    const uint16_t *svh = suh + inputs;
    uint16_t *weights = malloc((size_t)inputs * outputs * sizeof *weights);
    double *rotated = malloc(inputs * sizeof *rotated), *product = malloc(outputs * sizeof *product);
    double block[BLOCK];
    orc_exl3_decode_matrix(matrix, inputs, outputs, stored_width, weights);
    for (uint32_t base = 0; base < inputs; base += BLOCK) {
        for (uint32_t i = 0; i < BLOCK; i++) {
            block[i] = x[base + i] * orc_half_value(suh[base + i]);
        }
        orc_h128_f64(block, rotated + base);
    }
    for (uint32_t output = 0; output < outputs; output++) {
        double sum = 0.0;
        for (uint32_t input = 0; input < inputs; input++) {
            sum += rotated[input] * orc_half_value(weights[(uint64_t)input * outputs + output]);
        }
        product[output] = sum;
    }
    for (uint32_t base = 0; base < outputs; base += BLOCK) {
        orc_h128_f64(product + base, block);
        for (uint32_t i = 0; i < BLOCK; i++) {
            y[base + i] = block[i] * orc_half_value(svh[base + i]);
        }
    }
    free(weights);
    free(rotated);
    free(product);
}

/* ---- the layer ---- */

struct layer_work {
    const uint16_t *x_bf16;
    uint32_t rows, hidden, inner, picks, expert_count;
    const uint32_t *experts;
    const float *weights;
    const unsigned char *const *matrices;
    const uint8_t *widths;
    float limit;
    uint16_t *hidden_out;
    float *pair_out;
    uint32_t next_expert;
    pthread_mutex_t lock;
};

static void layer_expert(struct layer_work *work, uint32_t expert)
{
    uint32_t pairs[512], count = 0;
    const uint32_t pair_total = work->rows * work->picks;
    for (uint32_t pair = 0; pair < pair_total; pair++) {
        if (work->experts[pair] == expert) {
            pairs[count++] = pair;
            if (count == 512u) {
                break;
            }
        }
    }
    /* take the expert's pairs in runs of at most 512: each run is one pass over the three matrices */
    uint32_t done = 0;
    while (count != 0u) {
        const uint32_t H = work->hidden, I = work->inner;
        const unsigned char *gate = work->matrices[expert * 3u + 0u], *up = work->matrices[expert * 3u + 1u],
                            *down = work->matrices[expert * 3u + 2u];
        const uint32_t wg = work->widths[expert * 3u + 0u], wu = work->widths[expert * 3u + 1u],
                       wd = work->widths[expert * 3u + 2u];
        const uint16_t *gate_suh = (const uint16_t *)(gate + orc_exl3_code_bytes(H, I, wg)), *gate_svh = gate_suh + H;
        const uint16_t *up_suh = (const uint16_t *)(up + orc_exl3_code_bytes(H, I, wu)), *up_svh = up_suh + H;
        const uint16_t *down_suh = (const uint16_t *)(down + orc_exl3_code_bytes(I, H, wd)), *down_svh = down_suh + I;
        uint16_t *operands = malloc((size_t)count * (H > I ? H : I) * sizeof *operands);
        float *gate_products = malloc((size_t)count * I * sizeof(float));
        float *up_products = malloc((size_t)count * I * sizeof(float));
        float *down_products = malloc((size_t)count * H * sizeof(float));
        uint16_t *hidden_scratch = malloc((size_t)I * sizeof(uint16_t));
        for (uint32_t c = 0; c < count; c++) {
            orc_exl3_operand(work->x_bf16 + (uint64_t)(pairs[c] / work->picks) * H, gate_suh, H, operands + (uint64_t)c * H);
        }
        orc_exl3_product_codes(gate, H, I, wg, operands, count, gate_products);
        for (uint32_t c = 0; c < count; c++) {
            orc_exl3_operand(work->x_bf16 + (uint64_t)(pairs[c] / work->picks) * H, up_suh, H, operands + (uint64_t)c * H);
        }
        orc_exl3_product_codes(up, H, I, wu, operands, count, up_products);
        for (uint32_t c = 0; c < count; c++) {
            uint16_t *hidden = work->hidden_out != NULL ? work->hidden_out + (uint64_t)pairs[c] * I : hidden_scratch;
            orc_exl3_activate(gate_products + (uint64_t)c * I, up_products + (uint64_t)c * I, gate_svh, up_svh,
                              down_suh, I, work->limit, hidden, operands + (uint64_t)c * I);
        }
        orc_exl3_product_codes(down, I, H, wd, operands, count, down_products);
        for (uint32_t c = 0; c < count; c++) {
            orc_exl3_finish(down_products + (uint64_t)c * H, down_svh, H, work->weights[pairs[c]],
                            work->pair_out + (uint64_t)pairs[c] * H);
        }
        free(operands);
        free(gate_products);
        free(up_products);
        free(down_products);
        free(hidden_scratch);
        /* the next run, if the expert has more than 512 pairs */
        done = pairs[count - 1u] + 1u;
        count = 0;
        for (uint32_t pair = done; pair < pair_total && count < 512u; pair++) {
            if (work->experts[pair] == expert) {
                pairs[count++] = pair;
            }
        }
    }
}

static void *layer_worker(void *argument)
{
    struct layer_work *work = argument;
    for (;;) {
        pthread_mutex_lock(&work->lock);
        const uint32_t expert = work->next_expert++;
        pthread_mutex_unlock(&work->lock);
        if (expert >= work->expert_count) {
            return NULL;
        }
        layer_expert(work, expert);
    }
}

void orc_exl3_moe_layer(const uint16_t *x_bf16, uint32_t rows, uint32_t hidden, uint32_t inner, uint32_t picks,
                        const uint32_t *experts, const float *weights, uint32_t expert_count,
                        const unsigned char *const *matrices, const uint8_t *widths, float limit,
                        float *out_rows, uint16_t *hidden_out, float *pair_out, uint32_t threads)
{
    struct layer_work work = {.x_bf16 = x_bf16, .rows = rows, .hidden = hidden, .inner = inner, .picks = picks,
                              .expert_count = expert_count, .experts = experts, .weights = weights,
                              .matrices = matrices, .widths = widths, .limit = limit, .hidden_out = hidden_out,
                              .next_expert = 0};
    float *own_pairs = NULL;
    pthread_t workers[64];
    if (pair_out == NULL) {
        own_pairs = calloc((size_t)rows * picks * hidden, sizeof(float));
        pair_out = own_pairs;
    }
    work.pair_out = pair_out;
    (void)pthread_once(&codebook_once, codebook_fill);
    pthread_mutex_init(&work.lock, NULL);
    if (threads < 1u) {
        threads = 1u;
    }
    if (threads > 64u) {
        threads = 64u;
    }
    for (uint32_t t = 1; t < threads; t++) {
        pthread_create(&workers[t], NULL, layer_worker, &work);
    }
    (void)layer_worker(&work);
    for (uint32_t t = 1; t < threads; t++) {
        pthread_join(workers[t], NULL);
    }
    pthread_mutex_destroy(&work.lock);
    orc_exl3_row_sum(pair_out, rows, picks, hidden, out_rows);
    free(own_pairs);
}
