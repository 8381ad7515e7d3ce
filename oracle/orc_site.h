/*
 * orc_site.h -- CPU oracle of the step ahead of the routed experts: the launches a block's site front stands for, the
 * dense product (the mix project and the router's scores) and the hyper-connection mix finish.
 *
 * TEST INFRASTRUCTURE: the checker of tests and of the smoke run; never the product path.
 *
 * Restated from the definitions the reference's records give (include/anemone/dense_linear_records.h:10-18,
 * include/anemone/hyper_connection_records.h:10-22; the kernels' statement source/kernel_dense_linear.cu:100-175 and
 * source/kernel_hyper_connection.cu:40-125, source/kernel_hyper_connection.cuh): float32 arithmetic, every operation
 * rounded on its own except the fused multiply-adds the definitions write (a chain's fmaf(weight, value, chain), the
 * squares' fmaf(value, value, q), the finish's fmaf(m, s, b)).
 *   dense product  thread t of 256 takes the chunks t, t + 256, ... of 8 inputs; its chain of an output and a row runs
 *                  from +0 in ascending input order; a group of 32 threads adds its chains by exchanges at distance 16
 *                  down to 1 (lane l adds lane l ^ d's), then the 8 groups' sums are added from +0 in ascending order.
 *                  With ORC_DENSE_ROW_SCALE the sum is multiplied by r(q (1 / input_size) + epsilon), q the row's
 *                  squares added in the same order. A float32 output is the value times output_scale; a bfloat16 one
 *                  is rounded, multiplied and rounded again.
 *   mix finish     pre_k = sigmoid(fmaf(m_k, s_0, b_k)) + 1e-6; post_k = 2 sigmoid(fmaf(m_4+k, s_1, b_4+k)); comb the
 *                  4 x 4 of fmaf(m_8+e, s_2, b_8+e), each row less its largest, exponentiated, divided by its row's
 *                  sum (+ 1e-6 on the quotient), then by its column's sum + 1e-6, then nineteen more rounds of rows
 *                  and columns (sum + 1e-6); a line's four values added (x_0 + x_2) + (x_1 + x_3). The collapse with
 *                  the CARRIED pre p: h_d = bfloat16((((0 + p_0 X_0d) + p_1 X_1d) + p_2 X_2d) + p_3 X_3d); q the sum
 *                  of h_d h_d (thread t its eight from +0, product and sum rounded apart, then 32-lane exchanges and
 *                  one more over the groups' sums, zeros behind them); hidden_d = bfloat16(w_d (h_d r(q (1 / width) +
 *                  1e-20))). The site's pre then replaces the carried one.
 * Where the reference says "the card's expf" and "the card's rsqrtf" this build fixes the function: e^x is orc_expf
 * (the fixed float32 sequence of orc_exl3.h, within 2 places of the nearest) and r(x) the float32 nearest x^-1/2.
 * Pinned by the reference's own host oracles built into oracle/_ref from its sources: the collapse, the norm's operand
 * and the normed row bit for bit (test_hyper_collapse, test_hyper_norm_operand, test_hyper_norm_with with the factor
 * test_hyper_reciprocal_root gives), pre and post within TEST_HYPER_SINKHORN_PLACES (4) float32 places and comb within
 * TEST_HYPER_COMB_TOLERANCE (2^-20) of test_hyper_sinkhorn (tests/hyper_connection_reference.h:13-29), the dense
 * product inside test_dense_output_holds' bound of test_dense_reference (tests/dense_linear_reference.h:14-21); and
 * by what the definitions fix: inputs of small integers and powers of two make every sum exact whatever the order.
 */
#ifndef ORC_SITE_H
#define ORC_SITE_H

#include <stdint.h>

#define ORC_DENSE_BFLOAT16 0u
#define ORC_DENSE_FLOAT32 1u
#define ORC_DENSE_ROW_SCALE 1u
#define ORC_MIXES 24u

/* the float32 nearest 1 / sqrt(operand), of a positive normal float32 */
float orc_reciprocal_root(float operand);

/* weights [output_size][input_size] of weight_type; rows bfloat16 [row_count][input_size]; output [row_count]
 * [output_size] of output_type. input_size a multiple of 8. Returns 0, or -1 for an argument it does not take. */
int orc_dense_linear(uint32_t weight_type, const void *weights, uint32_t output_size, uint32_t input_size, uint32_t flags,
                     float epsilon, float output_scale, uint32_t output_type, const uint16_t *rows, uint32_t row_count,
                     void *output);

/* pre, post [4] and comb [4][4] of one row's 24 mixes, scale [3] and base [24] */
void orc_hyper_sinkhorn(const float *mixes, const float *scale, const float *base, float *pre_out, float *post_out, float *comb_out);

/* One row's mix finish. streams bfloat16 [4][width]; carried_pre [4]: read (the collapse's weights), then written (the
 * site's); norm_weight bfloat16 [width]; post_out [4]; comb_out [4][4]; hidden_out bfloat16 [width]; width a multiple
 * of 256, at most 8192. */
void orc_hyper_mix_finish(const uint16_t *streams, float *carried_pre, const float *mixes, const float *scale, const float *base,
                          const uint16_t *norm_weight, uint32_t width, float *post_out, float *comb_out, uint16_t *hidden_out);

/* the pieces, for the pins: the collapse, the norm's operand q (1 / width) + 1e-20, the normed row of a factor */
void orc_hyper_collapse(const uint16_t *streams, const float *pre, uint32_t width, uint16_t *collapsed_out);
float orc_hyper_norm_operand(const uint16_t *collapsed, uint32_t width);
void orc_hyper_norm_with(const uint16_t *collapsed, const uint16_t *weight, float factor, uint32_t width, uint16_t *normed_out);

#endif
