/*
 * kernel_registry.h -- how a kernel file tells the backend which entries it holds.
 *
 * The reference's backend loads one module per kernel file and reads each entry's argument sizes from the module
 * (source/backend_cuda_launch.c:160-186). Here the kernels are linked into the library; every kernel file lists
 * its entries with ANEMONE_KERNEL(file, function, record), which records the names, the host handle of the
 * function and sizeof(record) in a table built before main. kernel_prepare checks a request against that table:
 * the function exists in that file and its record has exactly argument_byte_count bytes.
 */
#ifndef KERNEL_REGISTRY_H
#define KERNEL_REGISTRY_H

#include <stdint.h>

extern "C" void anemone_register_kernel(const char *file, const char *function, const void *host_function,
                                        uint32_t record_bytes);

#define ANEMONE_KERNEL(file, function, record)                                                                 \
    static const int anemone_registered_##function =                                                           \
        (anemone_register_kernel(file, #function, (const void *)&function, (uint32_t)sizeof(struct record)), 0)

#endif
