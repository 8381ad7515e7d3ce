/*
 * backend_hip.cpp -- `backend_hip_value`: the reference's backend table (include/anemone/backend_seam.h:206-308)
 * over the HIP runtime for MI355X. Host code only; the kernels live in the kernel_*.hip files of this library and
 * announce themselves through kernel_registry.h.
 *
 * One card = one HIP device, one stream, one arena (hipMalloc at card_open; no other allocation on the card
 * afterwards). Uploads, downloads and launches are queued on the card's stream in call order. A ticket is the
 * card's copy sequence number; each unfinished copy holds one of BACKEND_MAXIMUM_UPLOADS_IN_FLIGHT events.
 * Failure is a status: a HIP error makes the card sticky (STATUS_DEVICE_ERROR, no new work), nothing aborts.
 * Every call of one card is serialised by the card's mutex.
 */
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "anemone_backend.h"
#include "kernel_registry.h"

namespace {

struct kernel_entry {
    const char *file;
    const char *function;
    const void *host_function;
    uint32_t record_bytes;
};

std::vector<kernel_entry> &kernel_table()
{
    static std::vector<kernel_entry> table; /* built by the kernel files' static registrations */
    return table;
}

struct copy_slot {
    hipEvent_t event;
    uint64_t ticket; /* 0: free */
};

struct staging_block {
    void *memory;
    uint64_t bytes;
};

std::mutex staging_mutex;
std::vector<staging_block> staging_blocks;

void log_error(const char *what, const char *detail)
{
    std::fprintf(stderr, "anemone backend_hip: %s: %s\n", what, detail);
}

} // namespace

struct device_card {
    int device;
    hipStream_t stream;
    unsigned char *arena;
    uint64_t arena_bytes;
    std::mutex mutex;
    bool failed;
    /* prepared kernels: handle = index */
    std::vector<uint32_t> prepared; /* indices into kernel_table() */
    /* copies */
    uint64_t next_ticket, finished_ticket;
    copy_slot slots[BACKEND_MAXIMUM_UPLOADS_IN_FLIGHT];
    /* graphs; the streams and events that carry a graph's side runs while it is captured */
    std::vector<hipGraphExec_t> graphs;
    hipStream_t side_streams[LAUNCH_MOST_SIDE_RUNS];
    hipEvent_t fork_event, side_events[LAUNCH_MOST_SIDE_RUNS];
    /* one timing interval */
    hipEvent_t measure_start, measure_stop;
    int measure_state; /* 0 idle, 1 begun, 2 ended */
    int max_threads, max_shared;
};

namespace {

std::mutex open_mutex;
device_card *open_cards[BACKEND_MAXIMUM_CARDS];

bool card_fail(device_card *card, const char *what, hipError_t error)
{
    if (error == hipSuccess) {
        return false;
    }
    card->failed = true;
    log_error(what, hipGetErrorString(error));
    return true;
}

bool range_in_staging(const void *memory, uint64_t bytes)
{
    std::lock_guard<std::mutex> guard(staging_mutex);
    const unsigned char *p = (const unsigned char *)memory;
    for (const staging_block &block : staging_blocks) {
        const unsigned char *base = (const unsigned char *)block.memory;
        if (p >= base && bytes <= block.bytes && (uint64_t)(p - base) <= block.bytes - bytes) {
            return true;
        }
    }
    return false;
}

/* retire every copy whose event has passed; tickets finish in order */
void copies_poll(device_card *card)
{
    for (;;) {
        copy_slot *oldest = nullptr;
        for (copy_slot &slot : card->slots) {
            if (slot.ticket != 0 && (oldest == nullptr || slot.ticket < oldest->ticket)) {
                oldest = &slot;
            }
        }
        if (oldest == nullptr) {
            return;
        }
        const hipError_t state = hipEventQuery(oldest->event);
        if (state == hipErrorNotReady) {
            return;
        }
        if (card_fail(card, "a copy failed", state)) {
            return;
        }
        card->finished_ticket = oldest->ticket;
        oldest->ticket = 0;
    }
}

result_status copy_begin(device_card *card, uint64_t offset, void *host, uint64_t bytes, bool upload,
                         uint64_t *ticket_out)
{
    if (card == nullptr || host == nullptr || ticket_out == nullptr || bytes == 0 || offset > card->arena_bytes ||
        bytes > card->arena_bytes - offset || !range_in_staging(host, bytes)) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(card->mutex);
    if (card->failed) {
        return STATUS_DEVICE_ERROR;
    }
    copies_poll(card);
    copy_slot *slot = nullptr;
    for (copy_slot &candidate : card->slots) {
        if (candidate.ticket == 0) {
            slot = &candidate;
            break;
        }
    }
    if (slot == nullptr) {
        return STATUS_BUSY_VALUE;
    }
    if (card_fail(card, "hipSetDevice", hipSetDevice(card->device))) {
        return STATUS_DEVICE_ERROR;
    }
    const hipError_t copied =
        upload ? hipMemcpyAsync(card->arena + offset, host, bytes, hipMemcpyHostToDevice, card->stream)
               : hipMemcpyAsync(host, card->arena + offset, bytes, hipMemcpyDeviceToHost, card->stream);
    if (card_fail(card, "hipMemcpyAsync", copied) ||
        card_fail(card, "hipEventRecord", hipEventRecord(slot->event, card->stream))) {
        return STATUS_DEVICE_ERROR;
    }
    slot->ticket = card->next_ticket++;
    *ticket_out = slot->ticket;
    return STATUS_OK;
}

/* every launch checked before any is queued (backend_seam.h:72-76) */
result_status launches_check(device_card *card, const kernel_launch *launches, uint32_t count)
{
    for (uint32_t index = 0; index < count; index++) {
        const kernel_launch &launch = launches[index];
        if (launch.kernel >= card->prepared.size()) {
            log_error("launch", "a kernel handle that was not prepared on this card");
            return STATUS_INVALID_ARGUMENT;
        }
        const kernel_entry &entry = kernel_table()[card->prepared[launch.kernel]];
        uint64_t threads = 1;
        for (uint32_t d = 0; d < LAUNCH_DIMENSIONS; d++) {
            if (launch.grid[d] == 0 || launch.block[d] == 0) {
                log_error(entry.function, "a grid or block dimension of zero");
                return STATUS_INVALID_ARGUMENT;
            }
            threads *= launch.block[d];
        }
        if (launch.argument_byte_count != entry.record_bytes || launch.argument_byte_count > LAUNCH_ARGUMENT_BYTES ||
            threads > (uint64_t)card->max_threads || launch.dynamic_shared_byte_count > (uint32_t)card->max_shared) {
            log_error(entry.function, "a record size, block size or shared memory size the card refuses");
            return STATUS_INVALID_ARGUMENT;
        }
        for (uint32_t byte = launch.argument_byte_count; byte < LAUNCH_ARGUMENT_BYTES; byte++) {
            if (launch.argument[byte] != 0) {
                log_error(entry.function, "bytes behind the record are not zero");
                return STATUS_INVALID_ARGUMENT;
            }
        }
    }
    /* the branches: side runs open behind a fork (a launch on the main line, or the root), at most
     * LAUNCH_MOST_SIDE_RUNS of them; the main line goes on with RESUME or JOIN, never with a CHAIN behind a side launch */
    uint32_t open_runs = 0;
    bool last_is_side = false;
    for (uint32_t index = 0; index < count; index++) {
        const uint32_t branch = launches[index].branch;
        bool fine = true;
        switch (branch) {
        case LAUNCH_CHAIN:
            fine = !last_is_side;
            last_is_side = false;
            break;
        case LAUNCH_SIDE:
            if (!last_is_side) {
                fine = open_runs == 0; /* one fork at a time: further runs behind it are SIDE_MORE */
                open_runs++;
            }
            last_is_side = true;
            break;
        case LAUNCH_SIDE_MORE:
            fine = open_runs != 0 && open_runs < LAUNCH_MOST_SIDE_RUNS && last_is_side;
            open_runs++;
            last_is_side = true;
            break;
        case LAUNCH_RESUME:
            fine = open_runs != 0 && last_is_side;
            last_is_side = false;
            break;
        case LAUNCH_JOIN:
            fine = open_runs != 0;
            open_runs = 0;
            last_is_side = false;
            break;
        default:
            fine = false;
        }
        if (!fine) {
            log_error("launch", "a branch that does not fit the launches before it");
            return STATUS_INVALID_ARGUMENT;
        }
    }
    return STATUS_OK;
}

hipError_t launch_on(device_card *card, const kernel_launch &launch, hipStream_t stream)
{
    const kernel_entry &entry = kernel_table()[card->prepared[launch.kernel]];
    /* the record travels by value: the runtime copies record_bytes from the launch's own bytes */
    void *arguments[2] = {(void *)launch.argument, (void *)&card->arena};
    return hipLaunchKernel(entry.host_function, dim3(launch.grid[0], launch.grid[1], launch.grid[2]),
                           dim3(launch.block[0], launch.block[1], launch.block[2]), arguments,
                           launch.dynamic_shared_byte_count, stream);
}

hipError_t launch_one(device_card *card, const kernel_launch &launch)
{
    return launch_on(card, launch, card->stream);
}

/* A checked list under capture on the card's stream: side runs go to side streams that wait for the fork's event, a
 * JOIN (and the list's end) makes the main line wait for theirs. Every stream keeps the default priority. */
hipError_t capture_branches(device_card *card, const kernel_launch *launches, uint32_t count)
{
    hipError_t status = hipSuccess;
    uint32_t open_runs = 0;
    bool last_is_side = false;
    auto join = [&]() {
        for (uint32_t run = 0; run < open_runs && status == hipSuccess; run++) {
            status = hipEventRecord(card->side_events[run], card->side_streams[run]);
            if (status == hipSuccess) {
                status = hipStreamWaitEvent(card->stream, card->side_events[run], 0);
            }
        }
        open_runs = 0;
    };
    for (uint32_t index = 0; index < count && status == hipSuccess; index++) {
        const kernel_launch &launch = launches[index];
        switch (launch.branch) {
        case LAUNCH_SIDE:
        case LAUNCH_SIDE_MORE:
            if (!last_is_side || launch.branch == LAUNCH_SIDE_MORE) { /* a new run behind the fork */
                if (open_runs == 0) {
                    status = hipEventRecord(card->fork_event, card->stream);
                }
                if (status == hipSuccess) {
                    status = hipStreamWaitEvent(card->side_streams[open_runs], card->fork_event, 0);
                }
                open_runs++;
            }
            if (status == hipSuccess) {
                status = launch_on(card, launch, card->side_streams[open_runs - 1u]);
            }
            last_is_side = true;
            break;
        case LAUNCH_JOIN:
            join();
            /* fall through: the launch itself stands on the main line */
        default: /* CHAIN, RESUME: the main line, which stands at the fork while side runs are open */
            if (status == hipSuccess) {
                status = launch_on(card, launch, card->stream);
            }
            last_is_side = false;
            break;
        }
    }
    if (status == hipSuccess) {
        join(); /* a capture ends with every stream back on the main line */
    }
    return status;
}

result_status wait_for(device_card *card, hipEvent_t event, uint64_t limit_ns)
{
    const auto deadline = std::chrono::steady_clock::now() + std::chrono::nanoseconds(limit_ns);
    for (;;) {
        const hipError_t state = hipEventQuery(event);
        if (state == hipSuccess) {
            return STATUS_OK;
        }
        if (state != hipErrorNotReady) {
            (void)card_fail(card, "a wait found the card failed", state);
            return STATUS_DEVICE_ERROR;
        }
        if (std::chrono::steady_clock::now() >= deadline) {
            return STATUS_TIMED_OUT;
        }
        std::this_thread::yield();
    }
}

} // namespace

extern "C" result_status exl3_tc_static_scratch_resolve(void); /* kernel_exl3_tc.hip; private to the library */

extern "C" {

void anemone_register_kernel(const char *file, const char *function, const void *host_function,
                             uint32_t record_bytes)
{
    kernel_table().push_back(kernel_entry{file, function, host_function, record_bytes});
}

uint32_t backend_hip_kernel_table_count(void)
{
    return (uint32_t)kernel_table().size();
}

result_status backend_hip_kernel_table_entry(uint32_t index, const char **file_out, const char **function_out,
                                             uint32_t *record_bytes_out)
{
    if (index >= kernel_table().size() || file_out == nullptr || function_out == nullptr ||
        record_bytes_out == nullptr) {
        return STATUS_INVALID_ARGUMENT;
    }
    *file_out = kernel_table()[index].file;
    *function_out = kernel_table()[index].function;
    *record_bytes_out = kernel_table()[index].record_bytes;
    return STATUS_OK;
}

result_status backend_hip_card_count(uint32_t *card_count_out)
{
    if (card_count_out == nullptr) {
        return STATUS_INVALID_ARGUMENT;
    }
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess) {
        (void)hipGetLastError();
        count = 0; /* a machine without cards answers 0 */
    }
    if (count > BACKEND_MAXIMUM_CARDS) {
        return STATUS_UNSUPPORTED;
    }
    *card_count_out = (uint32_t)count;
    return STATUS_OK;
}

result_status backend_hip_card_describe(uint32_t card_index, struct card_description_record *out)
{
    uint32_t count = 0;
    if (out == nullptr || backend_hip_card_count(&count) != STATUS_OK || card_index >= count) {
        return STATUS_INVALID_ARGUMENT;
    }
    hipDeviceProp_t properties;
    if (hipGetDeviceProperties(&properties, (int)card_index) != hipSuccess) {
        return STATUS_DEVICE_ERROR;
    }
    struct card_description_record description;
    std::memset(&description, 0, sizeof description);
    std::snprintf(description.name, sizeof description.name, "%.*s", (int)sizeof description.name - 1, properties.name);
    std::snprintf(description.bus_address, sizeof description.bus_address, "%04x:%02x:%02x.0",
                  (unsigned)properties.pciDomainID, (unsigned)properties.pciBusID, (unsigned)properties.pciDeviceID);
    description.arithmetic_class =
        std::strncmp(properties.gcnArchName, "gfx950", 6) == 0 ? ARITHMETIC_CLASS_GFX950 : 0u;
    size_t free_bytes = 0, total_bytes = 0;
    if (hipSetDevice((int)card_index) != hipSuccess || hipMemGetInfo(&free_bytes, &total_bytes) != hipSuccess) {
        return STATUS_DEVICE_ERROR;
    }
    description.memory_total_bytes = total_bytes;
    description.memory_free_bytes = free_bytes;
    description.memory_reserved_bytes = BACKEND_HIP_MEMORY_RESERVED_BYTES;
    *out = description;
    return STATUS_OK;
}

result_status backend_hip_card_open(uint32_t card_index, uint64_t arena_byte_count, struct device_card **card_out)
{
    uint32_t count = 0;
    if (card_out == nullptr || arena_byte_count == 0 || backend_hip_card_count(&count) != STATUS_OK ||
        card_index >= count) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(open_mutex);
    if (open_cards[card_index] != nullptr) {
        return STATUS_INVALID_ARGUMENT; /* a card is opened once */
    }
    device_card *card = new (std::nothrow) device_card();
    if (card == nullptr) {
        return STATUS_OUT_OF_MEMORY;
    }
    card->device = (int)card_index;
    card->arena_bytes = arena_byte_count;
    card->failed = false;
    card->next_ticket = 1;
    card->finished_ticket = 0;
    card->measure_state = 0;
    hipDeviceProp_t properties;
    if (hipSetDevice(card->device) != hipSuccess ||
        hipGetDeviceProperties(&properties, card->device) != hipSuccess) {
        delete card;
        return STATUS_DEVICE_ERROR;
    }
    card->max_threads = properties.maxThreadsPerBlock;
    /* what a block may take with the limit raised at kernel_prepare: the whole LDS of a compute unit on gfx950 */
    card->max_shared = (int)(properties.maxSharedMemoryPerMultiProcessor > properties.sharedMemPerBlock
                                 ? properties.maxSharedMemoryPerMultiProcessor
                                 : properties.sharedMemPerBlock);
    if (hipMalloc((void **)&card->arena, arena_byte_count) != hipSuccess) {
        (void)hipGetLastError();
        delete card;
        return STATUS_OUT_OF_MEMORY;
    }
    bool ok = hipStreamCreateWithFlags(&card->stream, hipStreamNonBlocking) == hipSuccess;
    ok = ok && exl3_tc_static_scratch_resolve() == STATUS_OK; /* the library's array on this device: found once, here */
    for (copy_slot &slot : card->slots) {
        slot.ticket = 0;
        ok = ok && hipEventCreateWithFlags(&slot.event, hipEventDisableTiming) == hipSuccess;
    }
    ok = ok && hipEventCreate(&card->measure_start) == hipSuccess && hipEventCreate(&card->measure_stop) == hipSuccess;
    ok = ok && hipEventCreateWithFlags(&card->fork_event, hipEventDisableTiming) == hipSuccess;
    for (uint32_t run = 0; run < LAUNCH_MOST_SIDE_RUNS; run++) {
        ok = ok && hipStreamCreateWithFlags(&card->side_streams[run], hipStreamNonBlocking) == hipSuccess &&
             hipEventCreateWithFlags(&card->side_events[run], hipEventDisableTiming) == hipSuccess;
    }
    if (!ok) {
        (void)hipFree(card->arena);
        delete card;
        return STATUS_DEVICE_ERROR;
    }
    open_cards[card_index] = card;
    *card_out = card;
    return STATUS_OK;
}

void backend_hip_card_close(struct device_card *card, uint64_t wait_limit_nanoseconds)
{
    if (card == nullptr) {
        return;
    }
    {
        std::lock_guard<std::mutex> guard(card->mutex);
        (void)hipSetDevice(card->device);
        /* unfinished work is waited for up to the limit; past it one line is logged and the drain goes on (the arena
         * cannot be freed under a running launch) */
        const auto deadline = std::chrono::steady_clock::now() + std::chrono::nanoseconds(wait_limit_nanoseconds);
        while (hipStreamQuery(card->stream) == hipErrorNotReady) {
            if (std::chrono::steady_clock::now() >= deadline) {
                log_error("card_close", "work unfinished at the wait limit: draining the stream");
                break;
            }
            std::this_thread::sleep_for(std::chrono::microseconds(50));
        }
        if (hipStreamSynchronize(card->stream) != hipSuccess) {
            log_error("card_close", "the drain failed: the card and its arena are retained");
            return;
        }
        for (hipGraphExec_t graph : card->graphs) {
            (void)hipGraphExecDestroy(graph);
        }
        for (copy_slot &slot : card->slots) {
            (void)hipEventDestroy(slot.event);
        }
        (void)hipEventDestroy(card->measure_start);
        (void)hipEventDestroy(card->measure_stop);
        for (uint32_t run = 0; run < LAUNCH_MOST_SIDE_RUNS; run++) {
            (void)hipStreamDestroy(card->side_streams[run]);
            (void)hipEventDestroy(card->side_events[run]);
        }
        (void)hipEventDestroy(card->fork_event);
        (void)hipStreamDestroy(card->stream);
        (void)hipFree(card->arena);
    }
    {
        std::lock_guard<std::mutex> guard(open_mutex);
        open_cards[card->device] = nullptr;
    }
    delete card;
}

result_status backend_hip_staging_allocate(uint64_t byte_count, void **page_locked_memory_out)
{
    if (byte_count == 0 || page_locked_memory_out == nullptr) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(staging_mutex);
    if (staging_blocks.size() >= BACKEND_MAXIMUM_STAGING_BLOCKS) {
        return STATUS_BUSY_VALUE;
    }
    void *memory = nullptr;
    if (hipHostMalloc(&memory, byte_count, hipHostMallocPortable) != hipSuccess) {
        (void)hipGetLastError();
        return STATUS_OUT_OF_MEMORY;
    }
    staging_blocks.push_back(staging_block{memory, byte_count});
    *page_locked_memory_out = memory;
    return STATUS_OK;
}

void backend_hip_staging_free(void *page_locked_memory)
{
    if (page_locked_memory == nullptr) {
        return;
    }
    std::lock_guard<std::mutex> guard(staging_mutex);
    for (size_t index = 0; index < staging_blocks.size(); index++) {
        if (staging_blocks[index].memory == page_locked_memory) {
            (void)hipHostFree(page_locked_memory);
            staging_blocks.erase(staging_blocks.begin() + (long)index);
            return;
        }
    }
    log_error("staging_free", "an address that is not the start of a block: left alone");
}

result_status backend_hip_upload_begin(struct device_card *card, uint64_t arena_byte_offset,
                                       const void *page_locked_source, uint64_t byte_count,
                                       uint64_t *upload_ticket_out)
{
    return copy_begin(card, arena_byte_offset, (void *)page_locked_source, byte_count, true, upload_ticket_out);
}

result_status backend_hip_download_begin(struct device_card *card, uint64_t arena_byte_offset,
                                         void *page_locked_destination, uint64_t byte_count,
                                         uint64_t *download_ticket_out)
{
    return copy_begin(card, arena_byte_offset, page_locked_destination, byte_count, false, download_ticket_out);
}

result_status backend_hip_upload_wait(struct device_card *card, uint64_t upload_ticket,
                                      uint64_t wait_limit_nanoseconds)
{
    if (card == nullptr || upload_ticket == 0) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(card->mutex);
    if (upload_ticket >= card->next_ticket) {
        return STATUS_INVALID_ARGUMENT;
    }
    const auto deadline = std::chrono::steady_clock::now() + std::chrono::nanoseconds(wait_limit_nanoseconds);
    for (;;) {
        if (card->failed) {
            return STATUS_DEVICE_ERROR;
        }
        copies_poll(card);
        if (card->finished_ticket >= upload_ticket) {
            return STATUS_OK;
        }
        if (std::chrono::steady_clock::now() >= deadline) {
            return STATUS_TIMED_OUT;
        }
        std::this_thread::yield();
    }
}

result_status backend_hip_kernel_prepare(struct device_card *card, const char *kernel_file_name,
                                         const char *function_name, uint32_t argument_byte_count,
                                         uint32_t *kernel_out)
{
    if (card == nullptr || kernel_file_name == nullptr || function_name == nullptr || kernel_out == nullptr) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(card->mutex);
    bool file_known = false;
    const std::vector<kernel_entry> &table = kernel_table();
    for (uint32_t index = 0; index < table.size(); index++) {
        if (std::strcmp(table[index].file, kernel_file_name) != 0) {
            continue;
        }
        file_known = true;
        if (std::strcmp(table[index].function, function_name) != 0) {
            continue;
        }
        if (table[index].record_bytes != argument_byte_count) {
            log_error(function_name, "the record does not have the size the kernel takes");
            return STATUS_INVALID_ARGUMENT;
        }
        for (uint32_t handle = 0; handle < card->prepared.size(); handle++) {
            if (card->prepared[handle] == index) {
                *kernel_out = handle; /* the same kernel again gives the same handle */
                return STATUS_OK;
            }
        }
        if (card->prepared.size() >= BACKEND_MAXIMUM_KERNELS) {
            log_error(function_name, "more kernels than a card prepares");
            return STATUS_INVALID_ARGUMENT;
        }
        /* as the reference's backend does behind its parameter check (source/backend_cuda_launch.c:160-186): raise
         * the kernel's limit of dynamic shared memory to what the card holds; a refusal shows at the launch that asks */
        if (hipSetDevice(card->device) == hipSuccess) {
            (void)hipFuncSetAttribute(table[index].host_function, hipFuncAttributeMaxDynamicSharedMemorySize, card->max_shared);
            (void)hipGetLastError();
        }
        card->prepared.push_back(index);
        *kernel_out = (uint32_t)card->prepared.size() - 1u;
        return STATUS_OK;
    }
    if (!file_known) {
        log_error(kernel_file_name, "no build of this kernel file for gfx950");
        return STATUS_UNSUPPORTED;
    }
    log_error(function_name, "no such function in its kernel file");
    return STATUS_INVALID_ARGUMENT;
}

result_status backend_hip_launch_run(struct device_card *card, const struct kernel_launch *launches,
                                     uint32_t launch_count)
{
    if (card == nullptr || (launches == nullptr && launch_count != 0)) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(card->mutex);
    if (card->failed) {
        return STATUS_DEVICE_ERROR;
    }
    const result_status checked = launches_check(card, launches, launch_count);
    if (checked != STATUS_OK) {
        return checked;
    }
    if (card_fail(card, "hipSetDevice", hipSetDevice(card->device))) {
        return STATUS_DEVICE_ERROR;
    }
    for (uint32_t index = 0; index < launch_count; index++) {
        if (card_fail(card, "hipLaunchKernel", launch_one(card, launches[index]))) {
            return STATUS_DEVICE_ERROR;
        }
    }
    return STATUS_OK;
}

result_status backend_hip_launch_run_timed(struct device_card *card, const struct kernel_launch *launches,
                                           uint32_t launch_count, double *microseconds_out)
{
    if (card == nullptr || launches == nullptr || launch_count == 0 || microseconds_out == nullptr) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(card->mutex);
    if (card->failed) {
        return STATUS_DEVICE_ERROR;
    }
    const result_status checked = launches_check(card, launches, launch_count);
    if (checked != STATUS_OK) {
        return checked;
    }
    if (card_fail(card, "hipSetDevice", hipSetDevice(card->device))) {
        return STATUS_DEVICE_ERROR;
    }
    std::vector<hipEvent_t> events;
    events.reserve(launch_count + 1u);
    for (uint32_t index = 0; index <= launch_count; index++) {
        hipEvent_t event;
        if (card_fail(card, "hipEventCreate", hipEventCreate(&event))) {
            for (hipEvent_t created : events) {
                (void)hipEventDestroy(created);
            }
            return STATUS_DEVICE_ERROR;
        }
        events.push_back(event);
    }
    result_status status = STATUS_OK;
    for (uint32_t index = 0; index < launch_count && status == STATUS_OK; index++) {
        if (card_fail(card, "hipEventRecord", hipEventRecord(events[index], card->stream)) ||
            card_fail(card, "hipLaunchKernel", launch_one(card, launches[index]))) {
            status = STATUS_DEVICE_ERROR;
        }
    }
    if (status == STATUS_OK && (card_fail(card, "hipEventRecord", hipEventRecord(events[launch_count], card->stream)) ||
                                card_fail(card, "hipEventSynchronize", hipEventSynchronize(events[launch_count])))) {
        status = STATUS_DEVICE_ERROR;
    }
    for (uint32_t index = 0; index < launch_count && status == STATUS_OK; index++) {
        float milliseconds = 0.0f;
        if (card_fail(card, "hipEventElapsedTime", hipEventElapsedTime(&milliseconds, events[index], events[index + 1u]))) {
            status = STATUS_DEVICE_ERROR;
        }
        microseconds_out[index] = 1000.0 * (double)milliseconds;
    }
    for (hipEvent_t event : events) {
        (void)hipEventDestroy(event);
    }
    return status;
}

result_status backend_hip_launch_wait(struct device_card *card, uint64_t wait_limit_nanoseconds)
{
    if (card == nullptr) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(card->mutex);
    if (card->failed) {
        return STATUS_DEVICE_ERROR;
    }
    const auto deadline = std::chrono::steady_clock::now() + std::chrono::nanoseconds(wait_limit_nanoseconds);
    for (;;) {
        const hipError_t state = hipStreamQuery(card->stream);
        if (state == hipSuccess) {
            return STATUS_OK;
        }
        if (state != hipErrorNotReady) {
            (void)card_fail(card, "launch_wait found the card failed", state);
            return STATUS_DEVICE_ERROR;
        }
        if (std::chrono::steady_clock::now() >= deadline) {
            return STATUS_TIMED_OUT;
        }
        std::this_thread::yield();
    }
}

bool backend_hip_format_supported(uint32_t card_index, enum weight_format_code format)
{
    uint32_t count = 0;
    if (backend_hip_card_count(&count) != STATUS_OK || card_index >= count) {
        return false;
    }
    return format == WEIGHT_FORMAT_EXL3 || format == WEIGHT_FORMAT_E2M1_SCALED || format == WEIGHT_FORMAT_E4M3_SCALED ||
           format == WEIGHT_FORMAT_E4M3_BLOCK128;
}

result_status backend_hip_graph_capture(struct device_card *card, const struct kernel_launch *launches,
                                        uint32_t launch_count, uint32_t *graph_out)
{
    if (card == nullptr || launches == nullptr || launch_count == 0 || graph_out == nullptr) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(card->mutex);
    if (card->failed) {
        return STATUS_DEVICE_ERROR;
    }
    const result_status checked = launches_check(card, launches, launch_count);
    if (checked != STATUS_OK) {
        return checked;
    }
    if (card->graphs.size() >= BACKEND_MAXIMUM_GRAPHS) {
        return STATUS_BUSY_VALUE;
    }
    if (card_fail(card, "hipSetDevice", hipSetDevice(card->device)) ||
        card_fail(card, "hipStreamBeginCapture", hipStreamBeginCapture(card->stream, hipStreamCaptureModeThreadLocal))) {
        return STATUS_DEVICE_ERROR;
    }
    const hipError_t launched = capture_branches(card, launches, launch_count); /* kernels only: no memset node enters a graph */
    hipGraph_t graph = nullptr;
    const hipError_t ended = hipStreamEndCapture(card->stream, &graph);
    if (card_fail(card, "a launch under capture", launched) || card_fail(card, "hipStreamEndCapture", ended)) {
        return STATUS_DEVICE_ERROR;
    }
    hipGraphExec_t executable = nullptr;
    const hipError_t instantiated = hipGraphInstantiate(&executable, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (card_fail(card, "hipGraphInstantiate", instantiated)) {
        return STATUS_DEVICE_ERROR;
    }
    card->graphs.push_back(executable);
    *graph_out = (uint32_t)card->graphs.size() - 1u;
    return STATUS_OK;
}

result_status backend_hip_graph_run(struct device_card *card, uint32_t graph)
{
    if (card == nullptr) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(card->mutex);
    if (card->failed) {
        return STATUS_DEVICE_ERROR;
    }
    if (graph >= card->graphs.size()) {
        return STATUS_INVALID_ARGUMENT;
    }
    if (card_fail(card, "hipSetDevice", hipSetDevice(card->device)) ||
        card_fail(card, "hipGraphLaunch", hipGraphLaunch(card->graphs[graph], card->stream))) {
        return STATUS_DEVICE_ERROR;
    }
    return STATUS_OK;
}

result_status backend_hip_measure_begin(struct device_card *card)
{
    if (card == nullptr) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(card->mutex);
    if (card->failed) {
        return STATUS_DEVICE_ERROR;
    }
    if (card->measure_state != 0) {
        return STATUS_BUSY_VALUE;
    }
    if (card_fail(card, "hipEventRecord", hipEventRecord(card->measure_start, card->stream))) {
        return STATUS_DEVICE_ERROR;
    }
    card->measure_state = 1;
    return STATUS_OK;
}

result_status backend_hip_measure_end(struct device_card *card)
{
    if (card == nullptr) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(card->mutex);
    if (card->failed) {
        return STATUS_DEVICE_ERROR;
    }
    if (card->measure_state != 1) {
        return STATUS_INVALID_ARGUMENT;
    }
    if (card_fail(card, "hipEventRecord", hipEventRecord(card->measure_stop, card->stream))) {
        return STATUS_DEVICE_ERROR;
    }
    card->measure_state = 2;
    return STATUS_OK;
}

result_status backend_hip_measure_elapsed_us(struct device_card *card, uint64_t wait_limit_nanoseconds,
                                             double *microseconds_out)
{
    if (card == nullptr || microseconds_out == nullptr) {
        return STATUS_INVALID_ARGUMENT;
    }
    std::lock_guard<std::mutex> guard(card->mutex);
    if (card->failed) {
        return STATUS_DEVICE_ERROR;
    }
    if (card->measure_state != 2) {
        return STATUS_INVALID_ARGUMENT;
    }
    const result_status waited = wait_for(card, card->measure_stop, wait_limit_nanoseconds);
    if (waited != STATUS_OK) {
        return waited; /* a timeout keeps the interval live for another ask */
    }
    float milliseconds = 0.0f;
    if (card_fail(card, "hipEventElapsedTime", hipEventElapsedTime(&milliseconds, card->measure_start, card->measure_stop))) {
        return STATUS_DEVICE_ERROR;
    }
    card->measure_state = 0;
    *microseconds_out = 1000.0 * (double)milliseconds;
    return STATUS_OK;
}

const struct backend_operations backend_hip_value = {
    "hip-gfx950",
    backend_hip_card_count,
    backend_hip_card_describe,
    backend_hip_card_open,
    backend_hip_card_close,
    backend_hip_staging_allocate,
    backend_hip_staging_free,
    backend_hip_upload_begin,
    backend_hip_upload_wait,
    nullptr, /* digest */
    backend_hip_download_begin,
    backend_hip_kernel_prepare,
    backend_hip_launch_run,
    backend_hip_launch_wait,
    backend_hip_format_supported,
    nullptr, /* exchange_allocate */
    nullptr, /* exchange_free */
    nullptr, /* exchange_attach */
    nullptr, /* peer_attach */
    backend_hip_graph_capture,
    backend_hip_graph_run,
    nullptr, /* mark_record */
    nullptr, /* mark_follow */
    nullptr, /* staging_retire */
    nullptr, /* peer_connect */
    backend_hip_measure_begin,
    backend_hip_measure_end,
    backend_hip_measure_elapsed_us,
};

} /* extern "C" */
