/* prepare_common.c -- contract: prepare_common.h. */
#include "prepare_common.h"

#include <inttypes.h>
#include <string.h>

uint64_t product_or_most(uint64_t a, uint64_t b)
{
    if (a != 0 && b > UINT64_MAX / a) {
        return UINT64_MAX;
    }
    return a * b;
}

bool ranges_are_valid(const char *what, const struct checked_range *ranges, uint32_t count, uint64_t arena_bytes)
{
    for (uint32_t i = 0; i < count; i++) {
        const uint64_t at = ranges[i].range.byte_offset, size = ranges[i].range.byte_count;
        if (at % LINEAR_OFFSET_ALIGNMENT_BYTES != 0) {
            REFUSE("%s: %s begins at byte %" PRIu64 ", not on a multiple of %u", what, ranges[i].name, at,
                   LINEAR_OFFSET_ALIGNMENT_BYTES);
            return false;
        }
        if (at > arena_bytes || size > arena_bytes - at) {
            REFUSE("%s: %s (%" PRIu64 " bytes at %" PRIu64 ") leaves the arena of %" PRIu64 " bytes", what,
                   ranges[i].name, size, at, arena_bytes);
            return false;
        }
        if (ranges[i].exact ? size != ranges[i].touched : (ranges[i].touched == UINT64_MAX || size < ranges[i].touched)) {
            REFUSE("%s: %s holds %" PRIu64 " bytes where %s%" PRIu64 " are needed", what, ranges[i].name, size,
                   ranges[i].exact ? "exactly " : "", ranges[i].touched);
            return false;
        }
    }
    for (uint32_t i = 0; i < count; i++) {
        for (uint32_t j = i + 1; j < count; j++) {
            const struct linear_range *a = &ranges[i].range, *b = &ranges[j].range;
            if (a->byte_offset < b->byte_offset + b->byte_count && b->byte_offset < a->byte_offset + a->byte_count) {
                REFUSE("%s: %s and %s share a byte", what, ranges[i].name, ranges[j].name);
                return false;
            }
        }
    }
    return true;
}

void launch_fill(struct kernel_launch *launch, uint32_t kernel, uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                 uint32_t threads, uint32_t shared_bytes, const void *record, uint32_t record_bytes)
{
    memset(launch, 0, sizeof *launch);
    launch->kernel = kernel;
    launch->grid[0] = grid_x;
    launch->grid[1] = grid_y;
    launch->grid[2] = grid_z;
    launch->block[0] = threads;
    launch->block[1] = 1;
    launch->block[2] = 1;
    launch->dynamic_shared_byte_count = shared_bytes;
    launch->argument_byte_count = record_bytes;
    launch->branch = LAUNCH_CHAIN;
    memcpy(launch->argument, record, record_bytes);
}
