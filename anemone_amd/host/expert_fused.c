/*
 * expert_fused.c -- load-time preparation of the producer: gate with up and the quantization of the hidden vectors
 * in one launch. Entry points and refusal rules follow the reference's source/expert_fused.c:114-204 and
 * include/anemone/expert_fused.h:37-60; the join and the shared join of that header are the layer's next step and
 * are not built (their handles are BACKEND_NO_KERNEL).
 *
 *   launch      kernel                          grid                                   block
 *   producer    expert_gate_up_quantize_<S>     (ceil(outputs / strip), jobs + 1, 1)   64 S
 * strip = 64 outputs of E2M1 weights, 32 of E4M3; the last row of blocks takes the pairs that stand in no job.
 */
#include <stdio.h>
#include <string.h>

#include "prepare_common.h"

static const uint32_t slice_counts[LINEAR_SLICE_INSTANCES] = {1u, 2u, 4u, 8u, 16u};
#define BUILT_INSTANCES 4u

result_status expert_fused_kernels_prepare(const struct backend_operations *backend, struct device_card *card,
                                           uint32_t arithmetic_class, struct expert_fused_kernels *kernels_out)
{
    if (backend == NULL || backend->kernel_prepare == NULL || card == NULL || kernels_out == NULL ||
        arithmetic_class != ARITHMETIC_CLASS_GFX950) {
        REFUSE("the kernels of the fused experts: a missing argument, or a class other than %u", ARITHMETIC_CLASS_GFX950);
        return STATUS_INVALID_ARGUMENT;
    }
    struct expert_fused_kernels kernels;
    memset(&kernels, 0xFF, sizeof kernels); /* every handle BACKEND_NO_KERNEL */
    for (uint32_t instance = 0; instance < BUILT_INSTANCES; instance++) {
        char name[56];
        (void)snprintf(name, sizeof name, "%s%u", KERNEL_EXPERT_GATE_UP_QUANTIZE_STEM, slice_counts[instance]);
        result_status status = backend->kernel_prepare(card, KERNEL_FILE_EXPERT_LINEAR, name, sizeof(struct expert_gate_up_quantize_arguments),
                                                       &kernels.gate_up_quantize[instance]);
        if (status == STATUS_OK) {
            (void)snprintf(name, sizeof name, "%se4m3_%u", KERNEL_EXPERT_GATE_UP_QUANTIZE_STEM, slice_counts[instance]);
            status = backend->kernel_prepare(card, KERNEL_FILE_EXPERT_LINEAR, name, sizeof(struct expert_gate_up_quantize_arguments),
                                             &kernels.gate_up_quantize_e4m3[instance]);
        }
        if (status != STATUS_OK) {
            REFUSE("the kernels of the fused experts: %s is not prepared: %s", name, status_text(status));
            return status;
        }
    }
    *kernels_out = kernels;
    return STATUS_OK;
}

static bool ranges_share_a_byte(struct linear_range a, struct linear_range b)
{
    return a.byte_count != 0 && b.byte_count != 0 && a.byte_offset < b.byte_offset + b.byte_count &&
           b.byte_offset < a.byte_offset + a.byte_count;
}

result_status expert_producer_prepare(const struct linear_routed_experts_description *description,
                                      struct linear_range arrivals, uint64_t arena_byte_count,
                                      const struct linear_kernels_record *linear_kernels,
                                      const struct expert_fused_kernels *kernels, struct kernel_launch *launch_out)
{
    static const char what[] = "the producer";
    if (description == NULL || linear_kernels == NULL || kernels == NULL || launch_out == NULL) {
        REFUSE("%s: a missing argument", what);
        return STATUS_INVALID_ARGUMENT;
    }
    /* what the routed experts' prepare refuses is refused here, behind its one error line; its launches are discarded */
    struct kernel_launch discarded[LINEAR_ROUTED_EXPERTS_LAUNCH_COUNT];
    const result_status checked = linear_routed_experts_prepare(description, arena_byte_count, linear_kernels, discarded);
    if (checked != STATUS_OK) {
        return checked;
    }
    const uint64_t pairs = (uint64_t)description->row_count * description->pairs_per_row;
    const uint32_t outputs = description->gate_up_shape.output_size;
    if (description->row_count > LINEAR_MAXIMUM_ROWS || pairs > EXPERT_PRODUCER_MOST_PAIRS || outputs % 32u != 0) {
        REFUSE("%s: at most %u rows and %u pairs, outputs a multiple of 32", what, LINEAR_MAXIMUM_ROWS, EXPERT_PRODUCER_MOST_PAIRS);
        return STATUS_INVALID_ARGUMENT;
    }
    const uint64_t arrival_bytes = (uint64_t)description->job_count * (outputs / 32u) * 4u;
    const struct linear_range *others[] = {&description->jobs, &description->expert_weights, &description->codes, &description->exponents,
                                           &description->operands, &description->hidden, &description->hidden_codes,
                                           &description->hidden_exponents, &description->hidden_operands, &description->pair_output,
                                           &description->row_output};
    bool shares = false;
    for (uint32_t i = 0; i < sizeof others / sizeof others[0]; i++) {
        shares = shares || ranges_share_a_byte(arrivals, *others[i]);
    }
    if (arrivals.byte_offset % LINEAR_OFFSET_ALIGNMENT_BYTES != 0 || arrivals.byte_count < arrival_bytes ||
        arrivals.byte_offset > arena_byte_count || arrivals.byte_count > arena_byte_count - arrivals.byte_offset || shares) {
        REFUSE("%s: the arrival counters: %llu bytes on a multiple of %u inside the arena, sharing no byte with another range", what,
               (unsigned long long)arrival_bytes, LINEAR_OFFSET_ALIGNMENT_BYTES);
        return STATUS_INVALID_ARGUMENT;
    }
    const bool bytes = description->weight_format == WEIGHT_FORMAT_E4M3_SCALED;
    uint32_t instance = 0;
    while (instance < BUILT_INSTANCES && slice_counts[instance] != description->gate_up_slice_count) {
        instance++;
    }
    const uint32_t kernel = instance == BUILT_INSTANCES ? BACKEND_NO_KERNEL
                            : bytes                     ? kernels->gate_up_quantize_e4m3[instance]
                                                        : kernels->gate_up_quantize[instance];
    if (kernel == BACKEND_NO_KERNEL) {
        REFUSE("%s: the kernel of %u slices is not prepared", what, description->gate_up_slice_count);
        return STATUS_INVALID_ARGUMENT;
    }
    const struct expert_gate_up_quantize_arguments record = {
        description->jobs.byte_offset, description->codes.byte_offset, description->exponents.byte_offset,
        description->operands.byte_offset, description->hidden.byte_offset, description->hidden_codes.byte_offset,
        description->hidden_exponents.byte_offset, description->hidden_operands.byte_offset, arrivals.byte_offset,
        outputs, description->gate_up_shape.input_size, (uint32_t)pairs, description->pairs_per_row, description->activation_limit, 0};
    const uint32_t strip = bytes ? 32u : 64u;
    launch_fill(launch_out, kernel, (outputs + strip - 1u) / strip, description->job_count + 1u, 1,
                64u * description->gate_up_slice_count, 0, &record, sizeof record);
    return STATUS_OK;
}
