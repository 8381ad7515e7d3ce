/*
 * kernel_dense_linear.hip -- the dense products of a step of 1 to 8 rows on gfx950: y = W x for a matrix as the
 * checkpoint stores it (bfloat16 or float32, row-major) and bfloat16 rows: a site's mix project (float32
 * [24][4 width], with the row's scale) and the router's scores of the site front's order. Entry names, record and
 * arithmetic follow the reference (include/anemone/dense_linear_records.h:10-30, source/kernel_dense_linear.cu:40-175):
 *   - thread t of 256 takes the chunks t, t + 256, ... of 8 inputs; its chain of an output and a row runs from +0 in
 *     ascending input order, fmaf(weight, value, chain), both widened exactly;
 *   - a group of 32 threads adds its chains by exchanges at distance 16 down to 1, then the 8 groups' sums are added
 *     from +0 in ascending order;
 *   - DENSE_ROW_SCALE: the sum times r(q (1 / input_size) + epsilon), q the row's squares (fmaf(value, value, q)) added
 *     in the same order; r is the float32 nearest the reciprocal square root (the reference takes its card's rsqrtf);
 *   - a float32 output is the value times output_scale; a bfloat16 one is rounded, multiplied and rounded again.
 * DENSE_STEP_ROWS and DENSE_CONE_ROWS (the head's and the prefill cone's rows) are not built: the host refuses them.
 * More than 8 rows: the rows in groups of 8 on grid[1] (dense_linear_<type>_8_wide, 8 outputs a block, or the 8-row
 * instance of 4 outputs where the outputs do not divide).
 *
 * Work mapping: a wavefront holds two of the definition's groups of 32 (an exchange at a distance below 32 stays inside
 * its half). A step's matrices are 2 to 4 MB: the launch is a few round trips to memory, not a stream, so what counts is
 * how many blocks there are and how many loads each keeps in flight. A block takes the rows ROWS blockIdx.y .. + ROWS - 1
 * (the reference's launches have one row of blocks; here the host may give a matrix of few outputs, the mix project's 24,
 * a block a row and an output, the one-row instance on a grid (outputs, rows): 192 blocks in place of 24, the same
 * operations for every output); the chunk loop of the one-row instance is unrolled four times.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernel_registry.h"
#include "dense_device.cuh"

/* a kernel's block: its outputs and rows by the grid. Blocks go to the card's 8 dies in turn by their linear index, and
 * each die has its own L2. The blocks that share a group of rows (one an output group) are renumbered to follow each other
 * on one die, so that the rows come from memory once and from that die's L2 for the other output groups: a bijection of
 * the grid when its row groups divide by 8, the plain numbering otherwise. Which block computes an output changes nothing
 * in its bits. */
template <uint32_t TYPE, uint32_t ROWS, uint32_t OUTPUTS>
__device__ static __forceinline__ void dense_linear(const struct dense_linear_arguments &arguments, unsigned char *arena)
{
    __shared__ dense_group_sums<ROWS, OUTPUTS> lds;
    uint32_t output_group = blockIdx.x, row_group = blockIdx.y;
    if constexpr (ROWS != 1u) {
        if (gridDim.y % DENSE_DIES == 0u) {
            const uint32_t linear = blockIdx.x + gridDim.x * blockIdx.y, place = linear / DENSE_DIES;
            output_group = place % gridDim.x;
            row_group = place / gridDim.x * DENSE_DIES + linear % DENSE_DIES;
        }
    }
    dense_linear_body<TYPE, ROWS, OUTPUTS>(arguments, arena, (const uint16_t *)(arena + arguments.rows_offset), output_group * OUTPUTS,
                                           row_group * ROWS, threadIdx.x, true, lds);
}

#define DENSE_STAMP(name, type, rows, outputs, form)                                                                                  \
    extern "C" __global__ void __launch_bounds__(DENSE_THREADS_VALUE)                                                                 \
        dense_linear_##name##_##rows##form(struct dense_linear_arguments arguments, unsigned char *arena)                             \
    {                                                                                                                                 \
        dense_linear<type, rows, outputs>(arguments, arena);                                                                          \
    }                                                                                                                                 \
    ANEMONE_KERNEL(KERNEL_FILE_DENSE_LINEAR, dense_linear_##name##_##rows##form, dense_linear_arguments);
DENSE_STAMP(bfloat16, DENSE_BFLOAT16, 1, DENSE_OUTPUTS_PER_BLOCK, )
DENSE_STAMP(bfloat16, DENSE_BFLOAT16, 8, DENSE_OUTPUTS_PER_BLOCK, )
DENSE_STAMP(float32, DENSE_FLOAT32, 1, DENSE_OUTPUTS_PER_BLOCK, )
DENSE_STAMP(float32, DENSE_FLOAT32, 8, DENSE_OUTPUTS_PER_BLOCK, )
DENSE_STAMP(bfloat16, DENSE_BFLOAT16, 1, 1u, _narrow)
DENSE_STAMP(bfloat16, DENSE_BFLOAT16, 8, 1u, _narrow)
DENSE_STAMP(float32, DENSE_FLOAT32, 1, 1u, _narrow)
DENSE_STAMP(float32, DENSE_FLOAT32, 8, 1u, _narrow)
/* a step of more rows (a prefill chunk's): groups of 8 rows on grid[1], a block 8 outputs of its group, so that a group's
 * rows are read once for eight outputs; every output's bits are those of the launch of 8 rows of its group
 * (dense_linear_<type>_wide_<O> of the reference, include/anemone/dense_linear_records.h:31-37) */
DENSE_STAMP(bfloat16, DENSE_BFLOAT16, 8, DENSE_WIDE_OUTPUTS, _wide)
DENSE_STAMP(float32, DENSE_FLOAT32, 8, DENSE_WIDE_OUTPUTS, _wide)
