/*
 * prepare_common.h -- what every prepare function shares: the refusal line, the range rules and the one way a
 * launch is filled. Private to anemone_amd/host.
 *
 * Range rules (the reference's, source/prepare_common.c:49-107): a range begins on a multiple of
 * LINEAR_OFFSET_ALIGNMENT_BYTES, lies inside the arena (64-bit arithmetic, no wrap), holds at least the bytes the
 * launches touch (a matrix: exactly its stored bytes), and no two ranges of one description share a byte.
 */
#ifndef PREPARE_COMMON_H
#define PREPARE_COMMON_H

#include <stdbool.h>
#include <stdint.h>
#include <stdio.h>

#include "anemone_ops.h"

#define REFUSE(...)                                  \
    do {                                             \
        (void)fprintf(stderr, "anemone: " __VA_ARGS__); \
        (void)fputc('\n', stderr);                   \
    } while (0)

struct checked_range {
    const char *name;
    struct linear_range range;
    uint64_t touched; /* bytes the launches read or write from its first byte on; UINT64_MAX fits no range */
    bool exact;       /* a matrix occupies exactly its bytes */
};

bool ranges_are_valid(const char *what, const struct checked_range *ranges, uint32_t count, uint64_t arena_bytes);

/* every byte of the launch: grid (x, y, z), block (threads, 1, 1), the record, zero behind it */
void launch_fill(struct kernel_launch *launch, uint32_t kernel, uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                 uint32_t threads, uint32_t shared_bytes, const void *record, uint32_t record_bytes);

/* a * b, or UINT64_MAX where the product leaves 64 bits */
uint64_t product_or_most(uint64_t a, uint64_t b);

/* exl3_tc.c: why the fused EXL3 launches do not take a layer of these sizes, NULL when they do */
const char *exl3_tc_geometry_refusal(uint32_t hidden, uint32_t intermediate);

#endif
