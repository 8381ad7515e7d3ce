/*
 * site_front.c -- load-time preparation of the fused fronts of a block's sites: one launch in place of a site's mix
 * project, mix finish and quantization (and, for the FFN front, the router's scores and select between them). Entry
 * points and refusal rules follow the reference's source/site_front.c (include/anemone/site_front.h:7-21, 38-75).
 *
 *   launch        kernel             grid                                                          block
 *   site front    site_front_<R>     (rows + site_front_mix_blocks, 1, 1)                          width / 8
 *   FFN front     ffn_front_<R>      (rows + site_front_mix_blocks + site_front_score_blocks, 1, 1)  width / 8
 *   input front   input_front_<R>    (rows, 1, 1)                                                  width / 8
 *   coefficients  coefficient_front_<R>  (site_front_mix_blocks, 1, 1)                             width / 8
 * The input front and then the coefficient front are the site front in two launches of one stream.
 * R = 1 for one row, 8 for 2 to 8 rows. The width is a multiple of 1,024 from 2,048 to SITE_FRONT_MOST_WIDTH (a block holds
 * at least one quarter of 256 threads for the dense products and at most 640 threads). The scratch's counters are zero
 * before the first launch (whoever owns the arena clears it once); every launch leaves them zero; launches that share a
 * scratch run one after the other.
 */
#include <stddef.h>
#include <string.h>

#include "prepare_common.h"

#define FRONT_DEFAULT_WIDTH 5120u
#define FRONT_LEAST_WIDTH 2048u
#define FRONT_WIDTH_STEP 1024u /* the mix finish's and the post's */

result_status site_front_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                         struct site_front_kernels *kernels_out)
{
    if (backend == NULL || backend->kernel_prepare == NULL || card == NULL || kernels_out == NULL) {
        REFUSE("the kernels of the site fronts: a missing argument");
        return STATUS_INVALID_ARGUMENT;
    }
    static const char *const names[SITE_FRONT_INSTANCES] = {"site_front_1", "site_front_8", "ffn_front_1", "ffn_front_8",
                                                               "input_front_1", "input_front_8", "coefficient_front_1", "coefficient_front_8"};
    struct site_front_kernels kernels;
    for (uint32_t instance = 0; instance < SITE_FRONT_INSTANCES; instance++) {
        kernels.fronts[instance] = BACKEND_NO_KERNEL;
        const result_status status =
            backend->kernel_prepare(card, KERNEL_FILE_SITE_FRONT, names[instance], sizeof(struct site_front_arguments), &kernels.fronts[instance]);
        if (status != STATUS_OK) {
            REFUSE("the kernels of the site fronts: %s is not prepared: %s", names[instance], status_text(status));
            return status;
        }
    }
    *kernels_out = kernels;
    return STATUS_OK;
}

/* a positive float32 as fp16 bits, or 0 where fp16 does not hold it exactly */
static uint32_t exact_half_bits(float value)
{
    uint32_t bits;
    memcpy(&bits, &value, sizeof bits);
    const int32_t exponent = (int32_t)((bits >> 23) & 255u) - 127 + 15;
    if ((bits >> 31) != 0u || exponent <= 0 || exponent >= 31 || (bits & 0x1FFFu) != 0u) {
        return 0u;
    }
    return ((uint32_t)exponent << 10) | ((bits >> 13) & 1023u);
}

result_status site_front_prepare(const struct site_front_description *description, uint64_t arena_byte_count,
                                 const struct router_kernels_record *router_kernels, const struct site_front_kernels *kernels,
                                 struct kernel_launch *launch_out)
{
    static const char what[] = "a site front";
    if (description == NULL || kernels == NULL || launch_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    if (description->kind >= SITE_FRONT_KINDS) {
        REFUSE("%s: kind %u is outside the enumeration", what, description->kind);
        return STATUS_INVALID_ARGUMENT;
    }
    const bool ffn = description->kind == SITE_FRONT_KIND_FFN;
    if ((description->router != NULL) != ffn || (router_kernels != NULL) != ffn) {
        REFUSE("%s: a router and its kernels are given together, exactly for the FFN front", what);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t width = description->reserved_zero != 0u ? description->reserved_zero : FRONT_DEFAULT_WIDTH, rows = description->row_count;
    if (rows == 0u || rows > LINEAR_MAXIMUM_ROWS || width < FRONT_LEAST_WIDTH || width > SITE_FRONT_MOST_WIDTH || width % FRONT_WIDTH_STEP != 0u) {
        REFUSE("%s: 1 to %u rows of a width in whole %u from %u to %u", what, LINEAR_MAXIMUM_ROWS, FRONT_WIDTH_STEP, FRONT_LEAST_WIDTH, SITE_FRONT_MOST_WIDTH);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t instance = description->kind * SITE_FRONT_ROW_FORMS + (rows > 1u ? 1u : 0u);
    if (kernels->fronts[instance] == BACKEND_NO_KERNEL) {
        REFUSE("%s: its kernel is not prepared", what);
        return STATUS_INVALID_ARGUMENT;
    }
    struct site_front_arguments record;
    memset(&record, 0, sizeof record);
    record.select.row_count = rows;
    uint32_t experts = 0;
    if (ffn) {
        /* whatever router_select_prepare refuses of the router; its record is the front's select */
        struct kernel_launch select_launch;
        const result_status selected = router_select_prepare(description->router, arena_byte_count, router_kernels, &select_launch);
        if (selected != STATUS_OK) {
            return selected;
        }
        struct router_select_arguments select;
        memcpy(&select, select_launch.argument, sizeof select);
        const uint32_t scale_bits = exact_half_bits(select.route_scale);
        if (select.row_count != rows || select.expert_count > 1023u || select.expert_count % SITE_FRONT_SCORE_OUTPUTS != 0u || scale_bits == 0u) {
            REFUSE("%s: the routed experts' rows are the front's, at most 1,023 experts in whole %u, a route scale fp16 holds exactly", what,
                   SITE_FRONT_SCORE_OUTPUTS);
            return STATUS_INVALID_ARGUMENT;
        }
        experts = select.expert_count;
        record.select.step_offset = select.step_offset;
        record.select.scores_offset = select.scores_offset;
        record.select.bias_offset = select.bias_offset;
        record.select.expert_offsets_offset = select.expert_offsets_offset;
        record.select.affinities_offset = select.affinities_offset;
        record.select.jobs_offset = select.jobs_offset;
        record.select.weights_offset = select.weights_offset;
        record.select.gate_up_last_offset = select.gate_up_last_offset;
        record.select.down_last_offset = select.down_last_offset;
        record.select.reference_order_and_shape =
            site_front_shape_word(select.reference_order, select.expert_count, select.pick_count, select.affinity_kind, scale_bits);
    }
    const uint64_t row_values = (uint64_t)rows * width;
    struct checked_range ranges[24] = {
        {"the streams", description->streams, row_values * MODEL_STREAMS * 2u, false},
        {"the carried pre", description->carried_pre, (uint64_t)rows * MODEL_STREAMS * 4u, false},
        {"the mix weights", description->mix_weights, (uint64_t)MODEL_MIXES * MODEL_STREAMS * width * 4u, true},
        {"the scale", description->scale, HYPER_SCALES * 4u, true},
        {"the base", description->base, MODEL_MIXES * 4u, true},
        {"the norm's weight", description->norm_weight, (uint64_t)width * 2u, true},
        {"post", description->post, (uint64_t)rows * MODEL_STREAMS * 4u, false},
        {"comb", description->comb, (uint64_t)rows * MODEL_STREAMS * MODEL_STREAMS * 4u, false},
        {"the hidden rows", description->hidden, row_values * 2u, false},
        {"the codes", description->codes, row_values, false},
        {"the exponents", description->exponents, row_values / 32u, false},
        {"the operands", description->operands, row_values * 2u, false},
        {"the scratch", description->scratch, SITE_FRONT_SCRATCH_BYTES, false},
    };
    uint32_t count = 13u;
    if (ffn) {
        /* the router's ranges share no byte with the description's (its own were checked among themselves above) */
        const struct router_description *router = description->router;
        const struct checked_range more[] = {
            {"the router's weights", description->router_weights, (uint64_t)experts * width * 2u, true},
            {"the step block", router->step, sizeof(struct step_block), false},
            {"the router scores", router->scores, (uint64_t)rows * experts * 4u, false},
            {"the bias", router->bias, (uint64_t)experts * 4u, false},
            {"the expert offsets", router->offsets, (uint64_t)experts * MODEL_EXPERT_MATRICES * 8u, false},
            {"the affinities", router->affinities, (uint64_t)rows * experts * 4u, false},
            {"the job table", router->experts->jobs, (uint64_t)router->experts->job_count * sizeof(struct expert_job_record), false},
        };
        memcpy(&ranges[count], more, sizeof more);
        count += (uint32_t)(sizeof more / sizeof more[0]);
    }
    if (!ranges_are_valid(what, ranges, count, arena_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    record.streams_offset = description->streams.byte_offset;
    record.pre_offset = description->carried_pre.byte_offset;
    record.scale_offset = description->scale.byte_offset;
    record.base_offset = description->base.byte_offset;
    record.post_offset = description->post.byte_offset;
    record.comb_offset = description->comb.byte_offset;
    record.norm_weight_offset = description->norm_weight.byte_offset;
    record.hidden_offset = description->hidden.byte_offset;
    record.mix_weights_offset = description->mix_weights.byte_offset;
    record.codes_offset = description->codes.byte_offset;
    record.exponents_offset = description->exponents.byte_offset;
    record.operands_offset = description->operands.byte_offset;
    record.scratch_offset = description->scratch.byte_offset;
    record.router_weights_offset = ffn ? description->router_weights.byte_offset : 0u;
    const uint32_t blocks = description->kind == SITE_FRONT_KIND_INPUT          ? rows
                            : description->kind == SITE_FRONT_KIND_COEFFICIENTS ? site_front_mix_blocks(width)
                                                                                : rows + site_front_mix_blocks(width) +
                                                                                      (ffn ? site_front_score_blocks(width, experts) : 0u);
    launch_fill(launch_out, kernels->fronts[instance], blocks, 1, 1, width / HYPER_VALUES_PER_THREAD, 0, &record, sizeof record);
    return STATUS_OK;
}

result_status site_front_check(const struct backend_operations *backend, struct device_card *card, struct linear_range scratch,
                               void *staging, uint64_t wait_limit_nanoseconds, uint32_t *gave_up_out)
{
    if (backend == NULL || backend->download_begin == NULL || backend->upload_begin == NULL || backend->upload_wait == NULL || card == NULL ||
        staging == NULL || scratch.byte_count < SITE_FRONT_SCRATCH_BYTES || scratch.byte_offset % LINEAR_OFFSET_ALIGNMENT_BYTES != 0) {
        REFUSE("site_front_check: a backend with copies, a card, the front's scratch range and 8 page-locked bytes are needed");
        return STATUS_INVALID_ARGUMENT;
    }
    /* the two words behind the mixes: departed (zero again once a launch has ended) and gave_up */
    const uint64_t tail = scratch.byte_offset + offsetof(struct site_front_scratch, departed);
    uint32_t *words = staging;
    uint64_t ticket = 0;
    result_status status = backend->download_begin(card, tail, words, 2 * sizeof *words, &ticket);
    if (status == STATUS_OK) {
        status = backend->upload_wait(card, ticket, wait_limit_nanoseconds);
    }
    if (status != STATUS_OK) {
        return status;
    }
    const uint32_t gave_up = words[1];
    if (gave_up_out != NULL) {
        *gave_up_out = gave_up;
    }
    if (gave_up == 0) {
        return STATUS_OK;
    }
    REFUSE("site_front_check: %u blocks of a fused front gave their wait up: the outputs of that launch are not whole", gave_up);
    words[1] = 0; /* the count is read once: the next launch begins on a clean scratch */
    status = backend->upload_begin(card, tail, words, 2 * sizeof *words, &ticket);
    if (status == STATUS_OK) {
        status = backend->upload_wait(card, ticket, wait_limit_nanoseconds);
    }
    return status != STATUS_OK ? status : STATUS_DEVICE_ERROR;
}
