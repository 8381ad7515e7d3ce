/*
 * kernel_calibrate.hip -- a plain copy inside the arena, of a known size: the yardstick the memory-traffic counters
 * of a profile are scaled by (a counter's reading for this kernel against the bytes it is known to move). No
 * counterpart in the reference; not on the routed-expert path.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernel_registry.h"

struct arena_copy_arguments {
    uint64_t source_offset;
    uint64_t destination_offset;
    uint64_t byte_count; /* a multiple of 16 */
};
static_assert(sizeof(struct arena_copy_arguments) == 24, "arena_copy_arguments ABI");

typedef uint32_t copy_word __attribute__((ext_vector_type(4)));

extern "C" __global__ void arena_copy(struct arena_copy_arguments arguments, unsigned char *arena)
{
    const copy_word *source = (const copy_word *)(arena + arguments.source_offset);
    copy_word *destination = (copy_word *)(arena + arguments.destination_offset);
    const uint64_t words = arguments.byte_count / 16u;
    for (uint64_t word = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; word < words; word += (uint64_t)gridDim.x * blockDim.x) {
        destination[word] = source[word];
    }
}
ANEMONE_KERNEL("kernel_calibrate", arena_copy, arena_copy_arguments);
