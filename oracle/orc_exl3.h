/*
 * orc_exl3.h -- CPU oracle of the EXL3 (trellis, codebook mul1) routed-expert linears.
 *
 * TEST INFRASTRUCTURE: checker of tests/, of the smoke run and of the benchmark's CPU baseline. Never the
 * product path.
 *
 * What is restated, and from where (all paths relative to the reference tree):
 *   format, ring, window end S(i)      include/anemone/exl3_records.h:2-9,100-119
 *   codebook mul1                      tools/measure/trellis_reference.h:13-14,106-127; tests/exl3_reference.c:25-37
 *   position <-> (input, output)       tools/measure/trellis_reference.h:10-11,134-139; tests/exl3_reference.c:39-56
 *   H128, definition and fp32 order    tools/measure/trellis_reference.h:141-168; source/kernel_exl3.cu:104-124
 *   matrix y = (((x.suh)Hb)T)Hb.svh    tools/measure/trellis_reference.h:17-18
 *   chain stages and rounding points   source/kernel_exl3.cu:133-167 (input), :178-293 (product),
 *                                      :314-372 (activate), :374-402 (finish), :406-424 (row sum)
 *   product slice order                tests/exl3_chain_reference.h:5-12
 *
 * Pinned by (tests/test_oracle_exl3.py): the reference's known-answer state digests per width
 * (tests/exl3_widths_test.c:67-88), codebook state 0 = 0xC2E8 and the closed form over all 65,536 states, the
 * all-zero K3 tile x ones = -884.0, the position bijection, H.H = I and the double-precision definition of H128,
 * an independent Python bit walk of the ring, and oracle/_ref (the reference's own C oracles built in place)
 * wherever that library is present.
 *
 * One deliberate restatement: exp() of the SwiGLU is `orc_expf`, a fixed sequence of binary32 operations (the
 * reference says "the card's expf", any implementation within the usual ulp bound); the HIP kernels run the same
 * sequence so the hidden vector is bit-defined. orc_expf is pinned against libm to 1 ulp over a sweep.
 */
#ifndef ORC_EXL3_H
#define ORC_EXL3_H

#include <stdint.h>

#define ORC_EXL3_NORM 0.08838834764831845f /* float32(1 / sqrt(128)) */

/* bits_x2 (twice K) of a stored width: K for whole K = 1..8, 16 K for a half K; 0 if the value is no width */
uint32_t orc_exl3_bits_x2(uint32_t stored_width);
/* S(i): ring bit where the 16-bit window of position i ends */
uint32_t orc_exl3_window_end(uint32_t position, uint32_t bits_x2);
/* stored bytes of an inputs x outputs matrix: codes + fp16 suh[inputs] + fp16 svh[outputs] */
uint64_t orc_exl3_matrix_bytes(uint32_t inputs, uint32_t outputs, uint32_t stored_width);
uint64_t orc_exl3_code_bytes(uint32_t inputs, uint32_t outputs, uint32_t stored_width);

uint16_t orc_exl3_codebook(uint32_t state);                     /* state -> fp16 bits */
uint32_t orc_exl3_position(uint32_t input, uint32_t output);    /* place in tile -> ring position */
void orc_exl3_place(uint32_t position, uint32_t *input, uint32_t *output);
/* the 256 states of one tile in ring order; words: the tile's little-endian uint32 words */
void orc_exl3_tile_states(uint32_t bits_x2, const uint32_t *words, uint16_t *states);
/* whole matrix: states or fp16 weights as [inputs][outputs] */
void orc_exl3_states(const unsigned char *codes, uint32_t inputs, uint32_t outputs, uint32_t stored_width,
                     uint16_t *states_out);
void orc_exl3_decode_matrix(const unsigned char *codes, uint32_t inputs, uint32_t outputs, uint32_t stored_width,
                            uint16_t *weights_out);

/* one block of 128: kernels' fp32 order (in place, includes the 1/sqrt(128)), and the definition in double */
void orc_h128_f32(float *values);
void orc_h128_f64(const double *values, double *rotated);

float orc_expf(float x);

/* X5: operand row = fp16(H128(bf16 x . fp16 suh) * norm); width a multiple of 128 */
void orc_exl3_operand(const uint16_t *x_bf16, const uint16_t *suh_fp16, uint32_t width, uint16_t *operand_fp16);

/* X6: product of decoded weights [inputs][outputs] (fp16 bits) with one fp16 operand row.
 * mode 0: every product and the whole sum exact in double, rounded once to float (the ideal the kernels are
 *         held to within tolerance);
 * mode 1: float32, `slices` contiguous runs of K tiles each summed in ascending input order from +0, then the
 *         slice sums added in order from +0 (one plain-C order of the reference's slice rule). */
void orc_exl3_product(const uint16_t *weights, uint32_t inputs, uint32_t outputs, const uint16_t *operand_fp16,
                      uint32_t slices, int mode, float *products_out);
/* the same straight from the stored codes, without materialising the matrix (mode 0 arithmetic); columns rows of
 * operands [columns][inputs] -> products [columns][outputs] */
void orc_exl3_product_codes(const unsigned char *codes, uint32_t inputs, uint32_t outputs, uint32_t stored_width,
                            const uint16_t *operands_fp16, uint32_t columns, float *products_out);

/* X7: gate/up products -> bf16 hidden and the down operand */
void orc_exl3_activate(const float *gate_products, const float *up_products, const uint16_t *gate_svh,
                       const uint16_t *up_svh, const uint16_t *down_suh, uint32_t inner, float limit,
                       uint16_t *hidden_bf16_out, uint16_t *operand_fp16_out);
/* X8: down products -> weighted pair output */
void orc_exl3_finish(const float *down_products, const uint16_t *down_svh, uint32_t width, float route_weight,
                     float *pair_out);
void orc_exl3_row_sum(const float *pair_outputs, uint32_t rows, uint32_t pairs_per_row, uint32_t width,
                      float *rows_out);

/* One whole linear y = (((x.suh)Hb)T)Hb.svh in double precision from the stored matrix: the definition, for the
 * single-matrix configuration. x as doubles [inputs], y [outputs]. */
void orc_exl3_linear_f64(const unsigned char *matrix, uint32_t inputs, uint32_t outputs, uint32_t stored_width,
                         const double *x, double *y);

/* The routed experts of one layer for `rows` rows of `picks` routes each (pair = row * picks + slot).
 *   x_bf16        [rows][hidden]
 *   experts       [rows][picks] expert of each pair, weights [rows][picks] its route weight
 *   matrices      [expert_count][3] pointers to the stored gate, up, down matrices (gate/up hidden x inner,
 *                 down inner x hidden); widths [expert_count][3] their stored widths
 *   out_rows      [rows][hidden] float32: sum over slots, ascending, of the finished pair outputs
 *   hidden_out    optional [rows*picks][inner] bf16; pair_out optional [rows*picks][hidden] float32
 *   threads       worker threads (>= 1); experts are the unit of work
 * Products use mode 0 arithmetic. */
void orc_exl3_moe_layer(const uint16_t *x_bf16, uint32_t rows, uint32_t hidden, uint32_t inner, uint32_t picks,
                        const uint32_t *experts, const float *weights, uint32_t expert_count,
                        const unsigned char *const *matrices, const uint8_t *widths, float limit,
                        float *out_rows, uint16_t *hidden_out, float *pair_out, uint32_t threads);

#endif
