/*
 * anemone_backend.h -- the C ABI of libanemone_hip.so: the status codes, the backend table of one MI355X ("card")
 * and the prepared launch. Plain C: pointers, sizes and fixed-width integers only.
 *
 * This is the drop-in boundary. The reference engine reaches a card only through `struct backend_operations`
 * (include/anemone/backend_seam.h:206-308) bound once at load; its one instance is `backend_cuda_value`
 * (backend_seam.h:310). This library exports `backend_hip_value`, the same table with the same member order, over
 * the HIP runtime and hand-written gfx950 kernels. Every member keeps the reference's contract
 * (backend_seam.h:4-117): a record and an arena pointer per kernel, one arena per card allocated at card_open,
 * launches prepared at load and queued in order, failure as a status with outputs untouched.
 *
 * Members this build leaves NULL (a caller answers STATUS_UNSUPPORTED, backend_seam.h:113-115): digest,
 * exchange_*, peer_*, mark_*, staging_retire -- multi-card and storage features outside the routed-expert path.
 */
#ifndef ANEMONE_BACKEND_H
#define ANEMONE_BACKEND_H

#include <stdbool.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MUST_CHECK __attribute__((warn_unused_result))

/* include/anemone/status.h:23-35, same values */
typedef enum result_status {
    STATUS_OK = 0,
    STATUS_INVALID_ARGUMENT,
    STATUS_OUT_OF_MEMORY,
    STATUS_INPUT_OUTPUT_ERROR,
    STATUS_CORRUPT_PACK,
    STATUS_DEVICE_ERROR,
    STATUS_TIMED_OUT,
    STATUS_UNSUPPORTED,
    STATUS_BUSY_VALUE,
    STATUS_INJECTED_FAULT,
    STATUS_COUNT
} result_status;
const char *status_text(result_status status); /* include/anemone/status.h:38 */

/* include/anemone/weight_format_seam.h:58-73, same values */
enum weight_format_code {
    WEIGHT_FORMAT_NONE = 0,
    WEIGHT_FORMAT_FLOAT16 = 1,
    WEIGHT_FORMAT_EXL3 = 2,
    WEIGHT_FORMAT_E2M1_SCALED = 3,
    WEIGHT_FORMAT_INT4_SCALED = 4,
    WEIGHT_FORMAT_E4M3_SCALED = 5,
    WEIGHT_FORMAT_COUNT = 6, /* the reference's formats end here */
    /* extension, no counterpart in the reference: E4M3 codes in E4M3_SCALED's lane order [out/16][in/32][lane][16], then
     * one float32 scale for every 128 outputs x 128 inputs, [out/128][in/128]; its vectors are quantized 128 values a
     * float32 scale */
    WEIGHT_FORMAT_E4M3_BLOCK128 = 6,
    /* extensions, no counterpart in the reference: the two formats above whose name ends in _SCALED, the same weights and
     * scale codes, laid out in the lane order of gfx950's own matrix instruction (v_mfma_scale_f32_16x16x128_f8f6f4 on
     * wavefronts of 64) as the reference's are in the order of its cards' (include/anemone/weight_format_seam.h:22-46: "a
     * new format is a new entry here, its kernels in every backend, and its reference decode among the tests"). Made at
     * load time from the reference's bytes by weight_format_gfx950_pack (anemone_ops.h), which also states the lay-out. */
    WEIGHT_FORMAT_E2M1_GFX950 = 7,
    WEIGHT_FORMAT_E4M3_GFX950 = 8,
    /* and E4M3_BLOCK128 likewise: its codes in E4M3_GFX950's order, its float32 scales where they are */
    WEIGHT_FORMAT_E4M3_BLOCK128_GFX950 = 9
};

#define BACKEND_MAXIMUM_CARDS 16
#define BACKEND_MAXIMUM_KERNELS 256
#define BACKEND_NO_KERNEL UINT32_MAX
#define BACKEND_MAXIMUM_GRAPHS 512
#define BACKEND_MAXIMUM_UPLOADS_IN_FLIGHT 16
#define BACKEND_STAGING_ALIGNMENT_BYTES 4096
#define BACKEND_MAXIMUM_STAGING_BLOCKS 256
#define LAUNCH_DIMENSIONS 3
#define LAUNCH_ARGUMENT_BYTES 192
#define CARD_NAME_CAPACITY 96
#define CARD_BUS_ADDRESS_CAPACITY 32
/* the reference's classes are 80, 120, 1200 (backend_seam.h:152-162); this backend describes its cards as: */
#define ARITHMETIC_CLASS_GFX950 950u
#define BACKEND_HIP_MEMORY_RESERVED_BYTES (512ull << 20)

struct card_description_record { /* backend_seam.h:165-179 */
    char name[CARD_NAME_CAPACITY];
    char bus_address[CARD_BUS_ADDRESS_CAPACITY];
    uint32_t arithmetic_class;
    uint32_t link_generation;
    uint32_t link_lane_count;
    uint32_t reserved_zero;
    uint64_t memory_total_bytes;
    uint64_t memory_free_bytes;
    uint64_t memory_reserved_bytes;
};

struct device_card;

/* backend_seam.h:184-195 of the reference: where a launch stands in a captured graph. CHAIN: behind the launch before
 * it. A run of SIDE launches stands behind the launch before the run (the fork), each behind the one before it;
 * SIDE_MORE is another side run, of one launch, behind the same fork; RESUME stands behind the fork, not the side runs;
 * JOIN behind the launch before it and every side run's last. A list's first launch may open a side run: its fork is
 * then the graph's root. launch_run runs a list in its serial order whatever the branches say. */
#define LAUNCH_CHAIN 0u
#define LAUNCH_SIDE 1u
#define LAUNCH_RESUME 2u
#define LAUNCH_JOIN 3u
#define LAUNCH_SIDE_MORE 4u
#define LAUNCH_MOST_SIDE_RUNS 4u
struct kernel_launch { /* backend_seam.h:196-204 */
    uint32_t kernel;
    uint32_t grid[LAUNCH_DIMENSIONS];
    uint32_t block[LAUNCH_DIMENSIONS];
    uint32_t dynamic_shared_byte_count;
    uint32_t argument_byte_count;
    uint32_t branch;
    unsigned char argument[LAUNCH_ARGUMENT_BYTES];
};

struct backend_operations { /* backend_seam.h:206-308, member for member */
    const char *name;
    MUST_CHECK result_status (*card_count)(uint32_t *card_count_out);
    MUST_CHECK result_status (*card_describe)(uint32_t card_index, struct card_description_record *description_out);
    MUST_CHECK result_status (*card_open)(uint32_t card_index, uint64_t arena_byte_count,
                                          struct device_card **card_out);
    void (*card_close)(struct device_card *card, uint64_t wait_limit_nanoseconds);
    MUST_CHECK result_status (*staging_allocate)(uint64_t byte_count, void **page_locked_memory_out);
    void (*staging_free)(void *page_locked_memory);
    MUST_CHECK result_status (*upload_begin)(struct device_card *card, uint64_t arena_byte_offset,
                                             const void *page_locked_source, uint64_t byte_count,
                                             uint64_t *upload_ticket_out);
    MUST_CHECK result_status (*upload_wait)(struct device_card *card, uint64_t upload_ticket,
                                            uint64_t wait_limit_nanoseconds);
    MUST_CHECK result_status (*digest)(struct device_card *card, uint64_t arena_byte_offset, uint64_t byte_count,
                                       uint64_t wait_limit_nanoseconds, uint64_t *digest_out);
    MUST_CHECK result_status (*download_begin)(struct device_card *card, uint64_t arena_byte_offset,
                                               void *page_locked_destination, uint64_t byte_count,
                                               uint64_t *download_ticket_out);
    MUST_CHECK result_status (*kernel_prepare)(struct device_card *card, const char *kernel_file_name,
                                               const char *function_name, uint32_t argument_byte_count,
                                               uint32_t *kernel_out);
    MUST_CHECK result_status (*launch_run)(struct device_card *card, const struct kernel_launch *launches,
                                           uint32_t launch_count);
    MUST_CHECK result_status (*launch_wait)(struct device_card *card, uint64_t wait_limit_nanoseconds);
    bool (*format_supported)(uint32_t card_index, enum weight_format_code format);
    MUST_CHECK result_status (*exchange_allocate)(uint64_t byte_count, void **exchange_out);
    void (*exchange_free)(void *exchange);
    MUST_CHECK result_status (*exchange_attach)(struct device_card *card, const void *exchange,
                                                uint64_t address_word_offset);
    MUST_CHECK result_status (*peer_attach)(struct device_card *accessor, struct device_card *owner,
                                            const char *gate_record_path, uint64_t address_word_offset);
    MUST_CHECK result_status (*graph_capture)(struct device_card *card, const struct kernel_launch *launches,
                                              uint32_t launch_count, uint32_t *graph_out);
    MUST_CHECK result_status (*graph_run)(struct device_card *card, uint32_t graph);
    MUST_CHECK result_status (*mark_record)(struct device_card *card, uint32_t mark);
    MUST_CHECK result_status (*mark_follow)(struct device_card *card, struct device_card *owner, uint32_t mark);
    void (*staging_retire)(void *page_locked_memory);
    MUST_CHECK result_status (*peer_connect)(struct device_card *accessor, struct device_card *owner,
                                             uint64_t owner_offset, uint64_t address_word_offset);
    MUST_CHECK result_status (*measure_begin)(struct device_card *card);
    MUST_CHECK result_status (*measure_end)(struct device_card *card);
    MUST_CHECK result_status (*measure_elapsed_us)(struct device_card *card, uint64_t wait_limit_nanoseconds,
                                                   double *microseconds_out);
};

/* replaces `extern const struct backend_operations backend_cuda_value` (backend_seam.h:310) */
extern const struct backend_operations backend_hip_value;

/* The table's functions by name, for bindings that cannot read a struct of function pointers (ctypes, cgo):
 * each is the member of the same name of backend_hip_value. */
MUST_CHECK result_status backend_hip_card_count(uint32_t *card_count_out);
MUST_CHECK result_status backend_hip_card_describe(uint32_t card_index, struct card_description_record *out);
MUST_CHECK result_status backend_hip_card_open(uint32_t card_index, uint64_t arena_byte_count,
                                               struct device_card **card_out);
void backend_hip_card_close(struct device_card *card, uint64_t wait_limit_nanoseconds);
MUST_CHECK result_status backend_hip_staging_allocate(uint64_t byte_count, void **page_locked_memory_out);
void backend_hip_staging_free(void *page_locked_memory);
MUST_CHECK result_status backend_hip_upload_begin(struct device_card *card, uint64_t arena_byte_offset,
                                                  const void *page_locked_source, uint64_t byte_count,
                                                  uint64_t *upload_ticket_out);
MUST_CHECK result_status backend_hip_upload_wait(struct device_card *card, uint64_t upload_ticket,
                                                 uint64_t wait_limit_nanoseconds);
MUST_CHECK result_status backend_hip_download_begin(struct device_card *card, uint64_t arena_byte_offset,
                                                    void *page_locked_destination, uint64_t byte_count,
                                                    uint64_t *download_ticket_out);
MUST_CHECK result_status backend_hip_kernel_prepare(struct device_card *card, const char *kernel_file_name,
                                                    const char *function_name, uint32_t argument_byte_count,
                                                    uint32_t *kernel_out);
MUST_CHECK result_status backend_hip_launch_run(struct device_card *card, const struct kernel_launch *launches,
                                                uint32_t launch_count);
MUST_CHECK result_status backend_hip_launch_wait(struct device_card *card, uint64_t wait_limit_nanoseconds);
bool backend_hip_format_supported(uint32_t card_index, enum weight_format_code format);
MUST_CHECK result_status backend_hip_graph_capture(struct device_card *card, const struct kernel_launch *launches,
                                                   uint32_t launch_count, uint32_t *graph_out);
MUST_CHECK result_status backend_hip_graph_run(struct device_card *card, uint32_t graph);
MUST_CHECK result_status backend_hip_measure_begin(struct device_card *card);
MUST_CHECK result_status backend_hip_measure_end(struct device_card *card);
MUST_CHECK result_status backend_hip_measure_elapsed_us(struct device_card *card, uint64_t wait_limit_nanoseconds,
                                                        double *microseconds_out);

/* No counterpart in the reference (its card tests time with their own helper, tests/card_timing.h): queues the
 * launches as launch_run does with a device timestamp between consecutive launches, waits for them, and writes the
 * duration of each launch in microseconds to microseconds_out[launch_count]. For benchmarks and profiles. */
MUST_CHECK result_status backend_hip_launch_run_timed(struct device_card *card,
                                                      const struct kernel_launch *launches, uint32_t launch_count,
                                                      double *microseconds_out);
/* How many kernels the library was built with, and the i-th one's names and record size: what kernel_prepare checks
 * a request against (the reference reads the same from the module, source/backend_cuda_launch.c:160-186). */
uint32_t backend_hip_kernel_table_count(void);
MUST_CHECK result_status backend_hip_kernel_table_entry(uint32_t index, const char **file_out,
                                                        const char **function_out, uint32_t *record_bytes_out);
/* Adds one kernel to that table: every kernel file of the library does so for its entries before main, and a second
 * library of kernels linked against this one (the build's libanemone_probe.so: a plain copy, an instruction-rate probe
 * and exhaustive arithmetic checks, which are measurement and tests and stay out of the drop-in library) does so when it
 * is loaded. host_function is the kernel's host-side handle; the strings must outlive the table. No counterpart in the
 * reference, which finds its kernels in module images (source/backend_cuda_kernel_images.h:18-26). */
void anemone_register_kernel(const char *file, const char *function, const void *host_function, uint32_t record_bytes);

#ifdef __cplusplus
}
#endif
#endif
