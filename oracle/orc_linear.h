/*
 * orc_linear.h -- CPU oracle of the FP4 (E2M1 + E8M0/32, i.e. MXFP4) and FP8 (E4M3) expert linears of the
 * original weights: stored layouts, activation quantizer, block-scaled products, hidden step, row sum.
 *
 * TEST INFRASTRUCTURE: checker of tests/, of the smoke run and of the benchmark's CPU baseline. Never the
 * product path.
 *
 * Restated from (paths relative to the reference tree):
 *   stored layouts (lane order)    include/anemone/weight_format_seam.h:22-46; tests/weight_format_reference.h:10-23
 *   code values                    tests/weight_format_reference.h:24-28
 *   activation quantizer           include/anemone/linear_records.h:36-44; tests/linear_reference.h:22-33
 *   vector lane / operand order    include/anemone/linear_records.h:20-34
 *   product definition             include/anemone/linear_records.h:45-52; tests/linear_reference.h:34-42
 *   tolerance of a card's sum      tests/linear_reference.h:43-58
 *   hidden step                    include/anemone/linear_records.h:96-99; tests/linear_reference.h:59-66
 *   row sum                        tests/linear_reference.h:67-68
 *
 * Pinned by (tests/test_oracle_linear.py): lay-out / read-back round trips written independently of each other,
 * hand-placed weights, the E2M1 / E4M3 / E8M0 value tables, exhaustive nearest-code search for the quantizer,
 * numpy float64 matmul on dequantised tensors, and oracle/_ref (the reference's own C oracles) where present.
 *
 * The second FP8 scaling mode (E4M3 weights with one fp32 scale per 128 x 128 block, activations quantised per
 * row per 128 values with fp32 scales) has no counterpart in the reference: PARITY UNPINNED against the reference
 * by construction, pinned only by closed form (numpy float64 on dequantised tensors).
 */
#ifndef ORC_LINEAR_H
#define ORC_LINEAR_H

#include <stdint.h>

#define ORC_FORMAT_E2M1_SCALED 3 /* enum weight_format_code values of the reference */
#define ORC_FORMAT_E4M3_SCALED 5
#define ORC_FORMAT_E4M3_BLOCK128 6 /* no reference counterpart: E4M3 codes in E4M3_SCALED's lane order, then one float32
                                    * scale for every 128 outputs x 128 inputs, [outputs / 128][inputs / 128] */
/* no reference counterpart either: the two _SCALED formats' weights and scale codes in the lane order of gfx950's matrix
 * instruction. A matrix is tiles of 16 outputs by K steps of 128 inputs, tile after tile, step after step; a step is 64
 * lanes, lane 16 g + o holding output o of the tile.
 *   E2M1_GFX950: 16 bytes a lane; nibble n (0: low) of byte b of word T is input 32 g + 16 n + 2 T + {0, 8, 1, 9}[b] of
 *     the step; behind all tiles the scale codes, the tiles in groups of four: a word a lane a step a group, byte n the
 *     E8M0 code of output o of the group's tile n, inputs 32 g .. + 31.
 *   E4M3_GFX950: 32 bytes a lane, as two halves [half][lane][16]; byte c of word v (half v / 4) is input
 *     64 (v / 4) + 16 g + 8 (c % 2) + 2 (v % 4) + c / 2; the scale codes as E4M3_SCALED's.
 * Inputs a multiple of 128; outputs of 64 (E2M1) or 32 (E4M3). */
#define ORC_FORMAT_E2M1_GFX950 7
#define ORC_FORMAT_E4M3_GFX950 8
/* E4M3_BLOCK128's codes in E4M3_GFX950's lane order, then E4M3_BLOCK128's float32 scales as they are;
 * inputs and outputs a multiple of 128 */
#define ORC_FORMAT_E4M3_BLOCK128_GFX950 9

uint64_t orc_linear_stored_bytes(int format, uint32_t outputs, uint32_t inputs);
uint64_t orc_linear_scale_count(int format, uint32_t outputs, uint32_t inputs);

/* codes [outputs][inputs] one byte a weight; scale_codes E2M1: [outputs][inputs/32], E4M3: [ceil(outputs/32)][inputs/32]
 * -> stored bytes in the kernels' lane order. Returns 0, or -1 for a shape the format does not store. */
int orc_linear_lay_out(int format, uint32_t outputs, uint32_t inputs, const uint8_t *codes,
                       const uint8_t *scale_codes, uint8_t *stored);
/* W[output][input] of a stored matrix: its code, its scale code (an independent walk from the weight to its byte) */
int orc_linear_read(int format, uint32_t outputs, uint32_t inputs, const uint8_t *stored, uint32_t output,
                    uint32_t input, uint32_t *code_out, uint32_t *scale_out);

/* per-32 quantizer: values bf16 [width] -> codes [width] in value order, exponents [width/32] */
int orc_act_quantize(const uint16_t *values_bf16, uint32_t width, uint8_t *codes_out, uint8_t *exponents_out);
/* value order -> the stored lane order of a vector's codes; and the bf16 x 2^100 operands in operand order */
void orc_codes_lane_order(const uint8_t *codes, uint32_t width, uint8_t *stored_out);
void orc_operands_lay_out(const uint8_t *codes, const uint8_t *exponents, uint32_t width, uint16_t *operands_out);

/* y[v][o] for outputs first .. first + count - 1: sum over blocks of 32 inputs, ascending, of (exact block sum) x
 * weight scale x vector scale, in double; magnitude_out (optional) the same over magnitudes.
 * fed_codes [vectors][inputs] E4M3 codes in value order, fed_exponents [vectors][inputs/32]. */
int orc_linear_products(int format, uint32_t outputs, uint32_t inputs, const uint8_t *stored, uint32_t first,
                        uint32_t count, const uint8_t *fed_codes, const uint8_t *fed_exponents, uint32_t vectors,
                        double *sums_out, double *magnitude_out);
/* the tolerance of a card's bf16 output against (sum, magnitude): |c - y| <= ulp_bf16(c)/2 + bound */
int orc_linear_within_tolerance(uint16_t output_bf16, double sum, double magnitude, uint32_t inputs, uint32_t slices);
/* the same with the allowance T for the rounding inside the matrix instructions given: the reference takes 64 for
 * its cards' instructions of 16 products; a card whose instruction adds 128 scaled products has its own */
int orc_linear_within_allowance(uint16_t output_bf16, double sum, double magnitude, uint32_t inputs, uint32_t slices,
                                double allowance);

/* hidden step in double (the definition) and in the kernels' float32 order with gate/up rounded to bf16 first */
double orc_hidden_value(double gate, double up, double limit, double route_weight);
uint16_t orc_hidden_bits(float gate, float up, float limit, float route_weight);
/* float32 sum of bf16 pair outputs [pairs][width] of one row at `column`, ascending slot order from +0 */
float orc_row_sum_bf16(const uint16_t *pair_outputs, uint32_t pairs, uint32_t width, uint32_t column);

/* ---- second FP8 mode: 128 x 128 fp32 weight scales, per-row per-128 fp32 activation scales ---- */
/* activations: scale = max(|v|, 1e-4) / 448 (float32), code = RNE E4M3 of v / scale (float32 division), clamped */
void orc_act_quantize_128(const uint16_t *values_bf16, uint32_t width, uint8_t *codes_out, float *scales_out);
/* W codes [outputs][inputs] plain row-major E4M3, scales fp32 [ceil(outputs/128)][inputs/128];
 * y[v][o] = sum over 128-blocks of (exact block sum) x w_scale x a_scale, in double */
void orc_fp8_block128_products(uint32_t outputs, uint32_t inputs, const uint8_t *w_codes, const float *w_scales,
                               const uint8_t *a_codes, const float *a_scales, uint32_t vectors, double *sums_out);

/* the same for a matrix stored as ORC_FORMAT_E4M3_BLOCK128 and vectors quantized by orc_act_quantize_128
 * (fed_scales float32 [vectors][inputs / 128]): blocks of 128 inputs; any first and count */
int orc_linear_products_128(uint32_t outputs, uint32_t inputs, const uint8_t *stored, uint32_t first, uint32_t count,
                            const uint8_t *fed_codes, const float *fed_scales, uint32_t vectors, double *sums_out,
                            double *magnitude_out);
/* the same for either format of float32 scales (ORC_FORMAT_E4M3_BLOCK128, ORC_FORMAT_E4M3_BLOCK128_GFX950) */
int orc_linear_products_128_of(int format, uint32_t outputs, uint32_t inputs, const uint8_t *stored, uint32_t first,
                               uint32_t count, const uint8_t *fed_codes, const float *fed_scales, uint32_t vectors,
                               double *sums_out, double *magnitude_out);

/* One whole FP4/FP8 routed-expert layer (formats of the reference, per-32 scales), double-precision products with
 * the kernels' rounding points (format 6: float32 scales per 128, quantizer orc_act_quantize_128): quantize x per row, gate/up products -> bf16, hidden step -> bf16, quantize the
 * hidden vector, down product -> bf16 pair output, float32 row sum. matrices [expert_count][3] stored pointers. */
void orc_linear_moe_layer(int format, const uint16_t *x_bf16, uint32_t rows, uint32_t hidden, uint32_t inner,
                          uint32_t picks, const uint32_t *experts, const float *weights, uint32_t expert_count,
                          const uint8_t *const *matrices, float limit, float *out_rows, uint16_t *hidden_out,
                          uint16_t *pair_out, uint32_t threads);

#endif
