/*
 * step_experts.c -- a step's expert pauses: the routed experts a layer keeps in host memory go into the card's slots
 * between the layer's router and its experts. Host code over the backend's copies; what happens, its order and its
 * refusals follow the reference (include/anemone/model_seam.h:193-214; source/step_experts.c:27-168, whose driver-held
 * state is here a struct of the caller's, expert_slots).
 *
 * A job names a host expert i of its layer by three offsets equal to slots_offset + 16 i (a tag). At a pause the job
 * table comes back from the card; a first walk marks every slot that holds an expert some job names; a second gives
 * each such job that slot, or else the next slot in turn that no job of this pause marked, into which the expert's
 * bytes go up, and points the job's three offsets into the slot; the job table goes up again where a tag was in it. A
 * job of a tag marks one slot at most and a card has at least as many slots as a step has jobs, so an unmarked slot is
 * always left. expert_pause_plan is the walk alone (no card), expert_pause_run the pause on a card.
 */
#include <string.h>

#include "prepare_common.h"

#define TAG_BYTES LINEAR_OFFSET_ALIGNMENT_BYTES
#define SLOT_PASSES 2u /* the slots that hold their expert; then the others' */

static uint32_t slot_holding(const struct expert_slots *slots, uint64_t expert)
{
    uint32_t slot = 0;
    while (slot < slots->slot_count && slots->fields[(uint64_t)slot * EXPERT_SLOT_FIELDS] != expert + 1u) {
        slot++;
    }
    return slot;
}

result_status expert_pause_plan(const struct expert_pause *pause, struct expert_job_record *jobs, uint64_t job_count,
                                struct expert_slots *slots, struct expert_pause_upload *uploads_out, uint32_t *upload_count_out,
                                uint32_t *tag_count_out)
{
    static const char what[] = "an expert pause";
    if (pause == NULL || (jobs == NULL && job_count != 0) || slots == NULL || slots->fields == NULL || uploads_out == NULL ||
        upload_count_out == NULL || tag_count_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    if (slots->slot_count == 0 || slots->slot_count != pause->slot_count || slots->next_slot >= slots->slot_count ||
        job_count > slots->slot_count || pause->expert_byte_count > pause->slot_byte_count) {
        REFUSE("%s: %u slots of the card for the pause's %u, no more jobs (%llu) than slots, an expert no larger than a slot", what,
               slots->slot_count, pause->slot_count, (unsigned long long)job_count);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t mark = ++slots->pause_mark;
    uint32_t uploads = 0, tags = 0;
    for (uint32_t pass = 0; pass < SLOT_PASSES; pass++) {
        for (uint64_t index = 0; index < job_count; index++) {
            struct expert_job_record *job = &jobs[index];
            const uint64_t base = pause->slots_offset;
            if (job->row_count == 0 || (job->gate_offset < base && job->up_offset < base && job->down_offset < base)) {
                continue; /* empty, or an expert on the card */
            }
            const uint64_t tag = (job->gate_offset - base) / TAG_BYTES; /* where the job holds one */
            if (job->gate_offset < base || (job->gate_offset - base) % TAG_BYTES != 0 || tag >= pause->host_expert_count ||
                job->up_offset != job->gate_offset || job->down_offset != job->gate_offset) {
                REFUSE("%s: job %llu names neither an expert on card %u nor one of the %u in host memory", what,
                       (unsigned long long)index, pause->card, pause->host_expert_count);
                return STATUS_DEVICE_ERROR;
            }
            uint32_t slot = slot_holding(slots, pause->first_host_expert + tag);
            if (slot < slots->slot_count) { /* the first walk marks it, the second finds it marked */
                slots->fields[(uint64_t)slot * EXPERT_SLOT_FIELDS + 1u] = mark;
            }
            if (pass == 0) {
                continue;
            }
            if (slot == slots->slot_count) {
                slot = slots->next_slot;
                for (uint32_t tried = 1; tried < slots->slot_count && slots->fields[(uint64_t)slot * EXPERT_SLOT_FIELDS + 1u] == mark; tried++) {
                    slot = (slot + 1u) % slots->slot_count;
                }
                slots->next_slot = (slot + 1u) % slots->slot_count;
                if (slots->fields[(uint64_t)slot * EXPERT_SLOT_FIELDS + 1u] == mark) {
                    REFUSE("%s: none of the %u slots of card %u is free", what, slots->slot_count, pause->card);
                    for (uint32_t named = 0; named < uploads; named++) { /* nothing went up: these hold no expert */
                        slots->fields[(uint64_t)uploads_out[named].slot * EXPERT_SLOT_FIELDS] = 0;
                    }
                    return STATUS_DEVICE_ERROR;
                }
                uploads_out[uploads++] = (struct expert_pause_upload){slot, (uint32_t)tag};
                slots->fields[(uint64_t)slot * EXPERT_SLOT_FIELDS] = pause->first_host_expert + tag + 1u;
                slots->fields[(uint64_t)slot * EXPERT_SLOT_FIELDS + 1u] = mark;
            }
            const uint64_t at = base + (uint64_t)slot * pause->slot_byte_count;
            job->gate_offset = at + pause->matrix_offsets[0];
            job->up_offset = at + pause->matrix_offsets[1];
            job->down_offset = at + pause->matrix_offsets[EXPERT_PAUSE_MATRICES - 1u];
            tags++;
        }
    }
    *upload_count_out = uploads;
    *tag_count_out = tags;
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
