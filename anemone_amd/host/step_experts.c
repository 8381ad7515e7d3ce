/*
 * step_experts.c -- a step's expert pauses. A layer may keep some of its routed experts in host memory; between the
 * layer's router and its expert launches the ones the step needs are brought into slots of the card. Written from the
 * contract of the reference's include/anemone/model_seam.h:193-214 (what a tag is, where a slot lies, that a held expert
 * does not go up again); the reference's step driver holds the slots' state itself (source/step_experts.c:27-168), here it
 * is the caller's struct expert_slots.
 *
 * expert_pause_plan is the walk over a job table in host memory and touches no card: it reads every job first and refuses
 * a table with a broken job whole; then the slots whose expert a job names are set aside, and in the table's order each
 * hosted job is pointed at the slot of its expert, which is the one that holds it or else the first slot from the cursor
 * on that no job of this pause reads (the expert is then owed an upload and the cursor moves behind that slot).
 * expert_pause_run is the pause on a card over the backend's copies.
 */
#include <string.h>

#include "prepare_common.h"

/* a card's slots a pause can name at once: the walk keeps one bit a slot on its stack */
#define PAUSE_MOST_SLOTS 4096u
#define NO_SLOT UINT32_MAX

enum job_kind { JOB_STAYS, JOB_HOSTED, JOB_BROKEN };

/* What a job's three offsets say. A hosted job's are one value, slots_offset + 16 i with i among the pause's host
 * experts; a job that stays has all three below slots_offset (or no rows); anything between the two is broken. */
static enum job_kind job_kind_of(const struct expert_pause *pause, const struct expert_job_record *job, uint32_t *host_expert_out)
{
    const uint64_t floor = pause->slots_offset;
    const bool any_above = job->gate_offset >= floor || job->up_offset >= floor || job->down_offset >= floor;
    if (job->row_count == 0 || !any_above) {
        return JOB_STAYS;
    }
    if (job->gate_offset < floor || job->up_offset != job->gate_offset || job->down_offset != job->gate_offset) {
        return JOB_BROKEN;
    }
    const uint64_t distance = job->gate_offset - floor;
    if (distance % LINEAR_OFFSET_ALIGNMENT_BYTES != 0 || distance / LINEAR_OFFSET_ALIGNMENT_BYTES >= pause->host_expert_count) {
        return JOB_BROKEN;
    }
    *host_expert_out = (uint32_t)(distance / LINEAR_OFFSET_ALIGNMENT_BYTES);
    return JOB_HOSTED;
}

/* the card's slots as the walk sees them: who is in a slot, and one bit a slot for "a job of this pause reads it" */
struct slot_view {
    uint64_t *fields;
    uint32_t count;
    uint64_t in_use[PAUSE_MOST_SLOTS / 64u];
};

static uint64_t *occupant(const struct slot_view *view, uint32_t slot)
{
    return &view->fields[(uint64_t)slot * EXPERT_SLOT_FIELDS];
}

static uint32_t slot_of_expert(const struct slot_view *view, uint64_t expert)
{
    for (uint32_t slot = 0; slot < view->count; slot++) {
        if (*occupant(view, slot) == expert + 1u) {
            return slot;
        }
    }
    return NO_SLOT;
}

static bool in_use(const struct slot_view *view, uint32_t slot)
{
    return (view->in_use[slot / 64u] >> (slot % 64u)) & 1u;
}

static void take(struct slot_view *view, uint32_t slot)
{
    view->in_use[slot / 64u] |= (uint64_t)1 << (slot % 64u);
}

/* the first slot from the cursor on, round the ring once, that no job of this pause reads */
static uint32_t spare_slot_from(const struct slot_view *view, uint32_t cursor)
{
    for (uint32_t step = 0; step < view->count; step++) {
        const uint32_t slot = (cursor + step) % view->count;
        if (!in_use(view, slot)) {
            return slot;
        }
    }
    return NO_SLOT;
}

result_status expert_pause_plan(const struct expert_pause *pause, struct expert_job_record *jobs, uint64_t job_count,
                                struct expert_slots *slots, struct expert_pause_upload *uploads_out, uint32_t *upload_count_out,
                                uint32_t *tag_count_out)
{
    if (pause == NULL || slots == NULL || slots->fields == NULL || uploads_out == NULL || upload_count_out == NULL || tag_count_out == NULL ||
        (job_count != 0 && jobs == NULL)) {
        REFUSE("expert_pause_plan: every pointer is needed");
        return STATUS_INVALID_ARGUMENT;
    }
    if (slots->slot_count == 0 || slots->slot_count > PAUSE_MOST_SLOTS || slots->slot_count != pause->slot_count ||
        slots->next_slot >= slots->slot_count) {
        REFUSE("expert_pause_plan: the state holds %u slots (cursor %u), the pause speaks of %u; 1..%u are served", slots->slot_count,
               slots->next_slot, pause->slot_count, PAUSE_MOST_SLOTS);
        return STATUS_INVALID_ARGUMENT;
    }
    if (job_count > slots->slot_count || pause->expert_byte_count > pause->slot_byte_count) {
        REFUSE("expert_pause_plan: %llu jobs must find room in %u slots and %llu bytes of an expert in a slot's %llu",
               (unsigned long long)job_count, slots->slot_count, (unsigned long long)pause->expert_byte_count,
               (unsigned long long)pause->slot_byte_count);
        return STATUS_INVALID_ARGUMENT;
    }
    /* 1. read every job before anything moves: a table with a broken job leaves the slots and the table as they were */
    uint32_t hosted = 0, host_expert = 0;
    for (uint64_t j = 0; j < job_count; j++) {
        const enum job_kind kind = job_kind_of(pause, &jobs[j], &host_expert);
        if (kind == JOB_BROKEN) {
            REFUSE("expert_pause_plan: the offsets of job %llu (%llu, %llu, %llu) are not below the slots at %llu and are no tag of the "
                   "layer's %u host experts either (card %u)",
                   (unsigned long long)j, (unsigned long long)jobs[j].gate_offset, (unsigned long long)jobs[j].up_offset,
                   (unsigned long long)jobs[j].down_offset, (unsigned long long)pause->slots_offset, pause->host_expert_count, pause->card);
            return STATUS_DEVICE_ERROR;
        }
        hosted += kind == JOB_HOSTED;
    }
    struct slot_view view = {slots->fields, slots->slot_count, {0}};
    const uint64_t stamp = slots->pause_mark + 1u;
    /* 2. the experts already in a slot keep it: those slots are out of the spare ones' ring for this pause */
    for (uint64_t j = 0; j < job_count && hosted != 0; j++) {
        if (job_kind_of(pause, &jobs[j], &host_expert) == JOB_HOSTED) {
            const uint32_t slot = slot_of_expert(&view, (uint64_t)pause->first_host_expert + host_expert);
            if (slot != NO_SLOT) {
                take(&view, slot);
            }
        }
    }
    /* 3. in the table's order every hosted job gets its slot, a spare one from the cursor on where its expert is in none */
    uint32_t owed = 0, cursor = slots->next_slot;
    for (uint64_t j = 0; j < job_count && hosted != 0; j++) {
        struct expert_job_record *job = &jobs[j];
        if (job_kind_of(pause, job, &host_expert) != JOB_HOSTED) {
            continue;
        }
        const uint64_t expert = (uint64_t)pause->first_host_expert + host_expert;
        uint32_t slot = slot_of_expert(&view, expert);
        if (slot == NO_SLOT) {
            slot = spare_slot_from(&view, cursor);
            if (slot == NO_SLOT) { /* not reached while a table has no more jobs than the card slots */
                REFUSE("expert_pause_plan: all %u slots of card %u are read by this pause's jobs", view.count, pause->card);
                for (uint32_t u = 0; u < owed; u++) {
                    *occupant(&view, uploads_out[u].slot) = 0;
                }
                return STATUS_DEVICE_ERROR;
            }
            cursor = (slot + 1u) % view.count;
            *occupant(&view, slot) = expert + 1u;
            take(&view, slot);
            uploads_out[owed].slot = slot;
            uploads_out[owed].host_expert = host_expert;
            owed++;
        }
        occupant(&view, slot)[1] = stamp;
        const uint64_t slot_base = pause->slots_offset + (uint64_t)slot * pause->slot_byte_count;
        job->gate_offset = slot_base + pause->matrix_offsets[0];
        job->up_offset = slot_base + pause->matrix_offsets[1];
        job->down_offset = slot_base + pause->matrix_offsets[2];
    }
    slots->pause_mark = stamp;
    slots->next_slot = cursor;
    *upload_count_out = owed;
    *tag_count_out = hosted;
    return STATUS_OK;
}

/* waits for the tickets held, oldest first */
static result_status tickets_wait(const struct backend_operations *backend, struct device_card *card, const uint64_t *tickets, uint32_t count,
                                  uint64_t limit)
{
    result_status status = STATUS_OK;
    for (uint32_t index = 0; index < count; index++) {
        const result_status waited = backend->upload_wait(card, tickets[index], limit);
        status = status != STATUS_OK ? status : waited;
    }
    return status;
}

result_status expert_pause_run(const struct backend_operations *backend, struct device_card *card, const struct expert_pause *pause,
                               uint32_t row_count, struct expert_slots *slots, void *jobs_staging, const unsigned char *expert_copies,
                               uint64_t wait_limit_nanoseconds, uint32_t *upload_count_out)
{
    static const char what[] = "an expert pause";
    if (backend == NULL || backend->download_begin == NULL || backend->upload_begin == NULL || backend->upload_wait == NULL || card == NULL ||
        pause == NULL || slots == NULL || jobs_staging == NULL || (expert_copies == NULL && pause->host_expert_count != 0)) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t job_count = (uint64_t)pause->jobs_per_row * row_count;
    if (job_count == 0 || job_count > slots->slot_count) {
        REFUSE("%s: %llu jobs for %u slots", what, (unsigned long long)job_count, slots->slot_count);
        return STATUS_INVALID_ARGUMENT;
    }
    struct expert_job_record *jobs = (struct expert_job_record *)jobs_staging;
    uint64_t ticket = 0;
    /* the job table comes back; the card's launches queued before the pause (its router) are finished when it has */
    result_status status = backend->download_begin(card, pause->jobs_offset, jobs, job_count * sizeof *jobs, &ticket);
    if (status == STATUS_OK) {
        status = backend->upload_wait(card, ticket, wait_limit_nanoseconds);
    }
    if (status != STATUS_OK) {
        return status;
    }
    struct expert_pause_upload uploads[LINEAR_MAXIMUM_ROWS * ROUTER_MOST_PICKS];
    if (job_count > sizeof uploads / sizeof uploads[0]) {
        REFUSE("%s: %llu jobs are more than a thin step's", what, (unsigned long long)job_count);
        return STATUS_INVALID_ARGUMENT;
    }
    uint32_t upload_count = 0, tag_count = 0;
    status = expert_pause_plan(pause, jobs, job_count, slots, uploads, &upload_count, &tag_count);
    if (status != STATUS_OK) {
        return status;
    }
    /* the experts go up, at most BACKEND_MAXIMUM_UPLOADS_IN_FLIGHT copies on their way at once; then the job table */
    uint64_t tickets[BACKEND_MAXIMUM_UPLOADS_IN_FLIGHT];
    uint32_t held = 0;
    for (uint32_t index = 0; index < upload_count && status == STATUS_OK; index++) {
        if (held == BACKEND_MAXIMUM_UPLOADS_IN_FLIGHT) {
            status = tickets_wait(backend, card, tickets, held, wait_limit_nanoseconds);
            held = 0;
        }
        if (status == STATUS_OK) {
            status = backend->upload_begin(card, pause->slots_offset + (uint64_t)uploads[index].slot * pause->slot_byte_count,
                                           expert_copies + (uint64_t)uploads[index].host_expert * pause->expert_byte_count,
                                           pause->expert_byte_count, &tickets[held]);
            held += status == STATUS_OK ? 1u : 0u;
        }
    }
    if (status == STATUS_OK && tag_count != 0) {
        if (held == BACKEND_MAXIMUM_UPLOADS_IN_FLIGHT) {
            status = tickets_wait(backend, card, tickets, held, wait_limit_nanoseconds);
            held = 0;
        }
        if (status == STATUS_OK) {
            status = backend->upload_begin(card, pause->jobs_offset, jobs, job_count * sizeof *jobs, &tickets[held]);
            held += status == STATUS_OK ? 1u : 0u;
        }
    }
    const result_status waited = tickets_wait(backend, card, tickets, held, wait_limit_nanoseconds);
    status = status != STATUS_OK ? status : waited;
    if (status != STATUS_OK) {
        /* a copy that did not begin or did not finish: none of this pause's slots is taken to hold its expert whole (the
         * walk named them before any copy), so a later pause brings the expert up again */
        for (uint32_t index = 0; index < upload_count; index++) {
            slots->fields[(uint64_t)uploads[index].slot * EXPERT_SLOT_FIELDS] = 0;
        }
    }
    if (upload_count_out != NULL) {
        *upload_count_out = upload_count;
    }
    return status;
}

/* ---- the page-locked copies a card's pauses upload from ------------------------------------------------------------ */

/* the bytes of a pause's copies, or UINT64_MAX where they leave 64 bits */
static uint64_t pause_copy_bytes(const struct expert_pause *pause)
{
    return product_or_most(pause->expert_byte_count, pause->host_expert_count);
}

result_status expert_host_copies_attach(const struct backend_operations *backend, const struct expert_pause *pauses, uint32_t pause_count,
                                        const uint64_t *host_expert_offsets, uint64_t host_expert_count, const void *host_arena,
                                        uint64_t host_byte_count, uint64_t table_staging_bytes, uint64_t most_bytes,
                                        struct expert_host_copies *copies_out, uint64_t *pause_offsets_out)
{
    if (backend == NULL || backend->staging_allocate == NULL || copies_out == NULL || (pause_count != 0 && (pauses == NULL || pause_offsets_out == NULL))) {
        REFUSE("expert_host_copies_attach: a backend that allocates page-locked memory, the pauses and both outputs are needed");
        return STATUS_INVALID_ARGUMENT;
    }
    /* first the sizes and every source range, so that a refusal has allocated and written nothing */
    uint64_t total = 0;
    for (uint32_t p = 0; p < pause_count; p++) {
        const struct expert_pause *pause = &pauses[p];
        const uint64_t bytes = pause_copy_bytes(pause);
        const uint64_t last = (uint64_t)pause->first_host_expert + pause->host_expert_count;
        if (pause->host_expert_count == 0 || pause->expert_byte_count == 0 || bytes == UINT64_MAX || last > host_expert_count ||
            host_expert_offsets == NULL || host_arena == NULL) {
            REFUSE("expert_host_copies_attach: pause %u speaks of host experts %u..%llu of %llu, %llu bytes each: none, or not all, are in the "
                   "table of the host arena", p, pause->first_host_expert, (unsigned long long)last, (unsigned long long)host_expert_count,
                   (unsigned long long)pause->expert_byte_count);
            return STATUS_INVALID_ARGUMENT;
        }
        for (uint64_t e = pause->first_host_expert; e < last; e++) {
            if (host_expert_offsets[e] > host_byte_count || pause->expert_byte_count > host_byte_count - host_expert_offsets[e]) {
                REFUSE("expert_host_copies_attach: host expert %llu (%llu bytes at %llu) ends behind the host arena's %llu bytes",
                       (unsigned long long)e, (unsigned long long)pause->expert_byte_count, (unsigned long long)host_expert_offsets[e],
                       (unsigned long long)host_byte_count);
                return STATUS_INVALID_ARGUMENT;
            }
        }
        if (bytes > UINT64_MAX - total) {
            return STATUS_OUT_OF_MEMORY;
        }
        total += bytes;
    }
    const uint64_t table_at = (total + 255u) / 256u * 256u;
    if (table_staging_bytes > UINT64_MAX - table_at || table_at + table_staging_bytes > most_bytes) {
        REFUSE("expert_host_copies_attach: %llu bytes of experts and %llu of a job table are above the %llu the caller allows",
               (unsigned long long)total, (unsigned long long)table_staging_bytes, (unsigned long long)most_bytes);
        return STATUS_OUT_OF_MEMORY;
    }
    struct expert_host_copies made = {NULL, table_at + table_staging_bytes, table_at};
    if (made.byte_count != 0) {
        void *block = NULL;
        const result_status status = backend->staging_allocate(made.byte_count, &block);
        if (status != STATUS_OK) {
            return status;
        }
        if (block == NULL) {
            return STATUS_OUT_OF_MEMORY;
        }
        made.block = block;
    }
    uint64_t at = 0;
    for (uint32_t p = 0; p < pause_count; p++) {
        const struct expert_pause *pause = &pauses[p];
        pause_offsets_out[p] = at;
        for (uint32_t e = 0; e < pause->host_expert_count; e++, at += pause->expert_byte_count) {
            memcpy(made.block + at, (const unsigned char *)host_arena + host_expert_offsets[(uint64_t)pause->first_host_expert + e],
                   (size_t)pause->expert_byte_count);
        }
    }
    *copies_out = made;
    return STATUS_OK;
}

void expert_host_copies_detach(const struct backend_operations *backend, struct expert_host_copies *copies)
{
    if (backend == NULL || copies == NULL) {
        return;
    }
    if (copies->block != NULL && backend->staging_free != NULL) {
        backend->staging_free(copies->block);
    }
    copies->block = NULL;
    copies->byte_count = copies->table_staging_offset = 0;
}
