/*
 * orc_join.h -- CPU oracle of the step behind the routed experts: the FFN site's join (a row's routed sum, the
 * shared expert's output added to it, and the hyper-connection post of the four residual streams).
 *
 * TEST INFRASTRUCTURE: the checker of tests, of the smoke run and of the benchmark's CPU baseline; never the product
 * path.
 *
 * Restated from the definitions the reference's records give (include/anemone/hyper_connection_records.h:27-29,
 * include/anemone/expert_fused_records.h:31-41; the kernels' statement source/kernel_hyper_connection.cuh:62-85,
 * source/kernel_expert_join.cuh:35-57): float32 arithmetic, every product and sum rounded on its own (no fused
 * multiply-add), a bfloat16 rounded to nearest with a tie to even and a not-a-number to 0x7FC0:
 *   s_d   = the float32 sum of the row's pair outputs, from +0 in ascending slot order;
 *   y_d   = bfloat16(s_d + shared_d);
 *   X'_kd = bfloat16(post_k y_d + ((((0 + c_0k X_0d) + c_1k X_1d) + c_2k X_2d) + c_3k X_3d)), of the streams X as they
 *           were before any is written; comb is [source j][target k].
 * Pinned by: the reference's own host oracle test_hyper_post (tests/hyper_connection_reference.c, built into
 * oracle/_ref from its sources) bit for bit at its fixed width of 5,120, with and without routed sums; and by what
 * the definition fixes on hand-made cases (identity comb with post 0 leaves the streams; a single non-zero comb entry
 * moves one stream; powers of two make every step exact).
 */
#ifndef ORC_JOIN_H
#define ORC_JOIN_H

#include <stdint.h>

#define ORC_STREAMS 4u

/* One row's post. streams, streams_out: bfloat16 [4][width] (may be the same array); post [4]; comb [4][4];
 * output bfloat16 [width]; routed_sums float32 [width], or NULL where the post adds none. */
void orc_hyper_post(const uint16_t *streams, const float *post, const float *comb, const uint16_t *output,
                    const float *routed_sums, uint32_t width, uint16_t *streams_out);

/* The join of `rows` rows. pair_output bfloat16 [rows * pairs_per_row][width]; shared_output bfloat16 [rows][width];
 * streams bfloat16 [rows][4][width], in place; post [rows][4]; comb [rows][4][4]; row_sums_out float32 [rows][width],
 * or NULL. */
void orc_expert_join(const uint16_t *pair_output, const uint16_t *shared_output, uint16_t *streams, const float *post,
                     const float *comb, float *row_sums_out, uint32_t rows, uint32_t pairs_per_row, uint32_t width);

/* The hidden step of the shared expert (route weight 1): gate, up, hidden bfloat16 [count] */
void orc_trunk_hidden(const uint16_t *gate, const uint16_t *up, float limit, uint32_t count, uint16_t *hidden_out);

#endif
