/*
 * kernel_hyper_connection.hip -- the FFN site's post and join on gfx950: what follows the routed experts of a layer.
 * Entry names, records and arithmetic follow the reference (source/kernel_hyper_connection.cu:204-226, 249-271;
 * source/kernel_hyper_connection.cuh:62-85; source/kernel_expert_join.cuh:35-57;
 * include/anemone/hyper_connection_records.h:27-29; include/anemone/expert_fused_records.h:31-41):
 *   - hyper_post_entry: stream k of a row becomes bfloat16(post_k y_d + ((((0 + c_0k X_0d) + c_1k X_1d) + c_2k X_2d) +
 *     c_3k X_3d)) of the four streams X as they were before any is written, in place; with is_combined 1, y_d is first
 *     bfloat16(s_d + y_d) of the routed experts' float32 sums s;
 *   - expert_join: expert_row_sum_entry (the float32 sum of a row's pair outputs from +0 in ascending slot order,
 *     stored where the record names an array for it) and behind it that post with the combine, in one launch.
 *   - hyper_mix_finish: the step ahead of the sublayer (below, with its own comment).
 * Every product and sum is rounded on its own (no fused multiply-add); a bfloat16 is rounded to nearest with a tie to
 * even, a not-a-number to 0x7FC0.
 *
 * Work mapping: a thread takes HYPER_VALUES_PER_THREAD = 8 consecutive values of one row (one 16-byte load of each
 * array); grid (width / (8 block[0]), rows). The streams' width is what the grid covers: the reference fixes it at its
 * model's 5,120 (it checks blockDim.x gridDim.x against that); here any multiple of 8 block[0]. Every load of a thread
 * is asked for before the first is used: the kernel moves (pairs_per_row + 9) x 2 bytes a value and computes little.
 */
#include "kernel_registry.h"
#include "hyper_device.cuh"

extern "C" __global__ void __launch_bounds__(HYPER_PIECE_THREADS) hyper_post_entry(struct hyper_post_arguments arguments, unsigned char *arena)
{
    const uint64_t row = blockIdx.y, row_threads = (uint64_t)gridDim.x * blockDim.x, thread = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const float *post = (const float *)(arena + arguments.post_offset) + row * MODEL_STREAMS;
    const float *comb = (const float *)(arena + arguments.comb_offset) + row * MODEL_STREAMS * MODEL_STREAMS;
    uint4_t *streams = (uint4_t *)(arena + arguments.streams_offset) + row * MODEL_STREAMS * row_threads + thread;
    float output[HYPER_VALUES_PER_THREAD];
    join_unpack(((const uint4_t *)(arena + arguments.output_offset))[row * row_threads + thread], output);
    if (arguments.is_combined != 0u) {
        const float4_t *sums = (const float4_t *)(arena + arguments.sums_offset) + (row * row_threads + thread) * 2u;
        const float4_t low = sums[0], high = sums[1];
#pragma unroll
        for (uint32_t v = 0; v < HYPER_VALUES_PER_THREAD; v++) {
            output[v] = bf16_to_float(float_to_bf16(__fadd_rn(v < 4u ? low[v % 4u] : high[v % 4u], output[v])));
        }
    }
    join_post_values(output, post, comb, streams, row_threads);
}
ANEMONE_KERNEL(KERNEL_FILE_HYPER_CONNECTION, hyper_post_entry, hyper_post_arguments);

extern "C" __global__ void __launch_bounds__(HYPER_PIECE_THREADS) expert_join(struct expert_join_arguments arguments, unsigned char *arena)
{
    const uint64_t row = blockIdx.y, row_threads = (uint64_t)gridDim.x * blockDim.x, thread = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    float shared_output[HYPER_VALUES_PER_THREAD];
    join_unpack(((const uint4_t *)(arena + arguments.shared_output_offset))[row * row_threads + thread], shared_output);
    join_values((const uint4_t *)(arena + arguments.pair_output_offset) + row * arguments.pairs_per_row * row_threads + thread,
                arguments.pairs_per_row, shared_output, (const float *)(arena + arguments.post_offset) + row * MODEL_STREAMS,
                (const float *)(arena + arguments.comb_offset) + row * MODEL_STREAMS * MODEL_STREAMS,
                (uint4_t *)(arena + arguments.streams_offset) + row * MODEL_STREAMS * row_threads + thread,
                arguments.row_sums_offset == EXPERT_JOIN_NO_ROW_SUMS
                    ? nullptr
                    : (float4_t *)(arena + arguments.row_sums_offset) + (row * row_threads + thread) * 2u,
                row_threads);
}
ANEMONE_KERNEL(KERNEL_FILE_HYPER_CONNECTION, expert_join, expert_join_arguments);

/* ---- the mix finish: what stands between a site's mix project and its sublayer ----
 * include/anemone/hyper_connection_records.h:10-22 and source/kernel_hyper_connection.cu:40-125,
 * source/kernel_hyper_connection.cuh of the reference. A row's block: the collapse of the four streams with the CARRIED
 * pre p, h_d = bfloat16((((0 + p_0 X_0d) + p_1 X_1d) + p_2 X_2d) + p_3 X_3d); q, the sum of the h_d h_d in a fixed tree
 * (a thread its eight from +0, a group of 32 threads by exchanges at distance 16 down to 1, one group the groups' sums
 * with zeros behind them); hidden_d = bfloat16(w_d (h_d r(q (1 / width) + 1e-20))), r the float32 nearest the reciprocal
 * square root (the reference takes its card's rsqrtf); and Sinkhorn of the row's 24 mixes, which writes post and comb and
 * replaces the carried pre with the site's once every thread has read it (behind the block's barrier). e^x is det_expf
 * (the reference takes its card's expf), every division IEEE, a line's four values added (x_0 + x_2) + (x_1 + x_3). */
extern "C" __global__ void __launch_bounds__(HYPER_FINISH_MOST_THREADS) hyper_mix_finish(struct hyper_finish_arguments arguments, unsigned char *arena)
{
    __shared__ float group_sums[32];
    hyper_mix_finish_body(arguments, arena, blockIdx.y, threadIdx.x, blockDim.x, group_sums);
}
ANEMONE_KERNEL(KERNEL_FILE_HYPER_CONNECTION, hyper_mix_finish, hyper_finish_arguments);
