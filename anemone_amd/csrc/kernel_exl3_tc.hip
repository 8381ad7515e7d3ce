/*
 * kernel_exl3_tc.hip -- the routed experts of one EXL3 layer for a decode-sized step (1 to 64 rows) on gfx950, from
 * the router's job table: five launches (operands, gate/up products, activation, down products, combine), the
 * counterpart of the reference's tensor-core MoE (source/kernel_exl3_tc.cu, include/anemone/exl3_tc_records.h).
 *
 * The arithmetic is the chain's (kernel_exl3.hip): fp16 operands from a float32 Hadamard transform, the codebook's
 * weights (see EXACT_WEIGHTS), float32 MFMA sums, SwiGLU in float32, the weighted pair outputs added in slot order. What
 * differs is the work mapping: every (job, matrix, strip of eight output tiles, K slice) is an independent wavefront item
 * that streams its bytes once, from memory straight into the registers of the lanes that decode them; K-slice partial sums are kept apart in the workspace and added in slice order by the next
 * launch, so a result does not depend on scheduling, on the other rows of the step or on the grid.
 *
 * Workspace (exl3_tc_workspace_bytes): fp16 operands [2][pairs][hidden], reused as [pairs][intermediate] for the
 * down operands; float32 gate/up partials [GATE_UP_SLICES][2][pairs][intermediate]; float32 down partials
 * [DOWN_SLICES][pairs][hidden].
 */
#include "exl3_stream_device.cuh"
#include "kernel_registry.h"
#include "anemone_ops.h"

#include <mutex>
#include <stdio.h>
#include <string.h>

#define STRIP_PAIRS (EXL3_TC_STRIP_OUTPUTS / 32u) /* a strip: pairs of adjacent output tiles */
/* false: the matrix instruction takes the codebook values before their scale and bias (1024 + b), which enter once a
 * sum; the weights' own rounding to fp16 is then left out of the product (within the products' stated tolerance) */
#define EXACT_WEIGHTS true
#define PRODUCT_WAVES 4u
#define PRODUCT_THREADS (PRODUCT_WAVES * WAVE)
#define COMBINE_THREADS (ROUTER_MOST_PICKS * WAVE) /* a wavefront a slot of the row */

struct tc_shape {
    uint32_t hidden, intermediate, picks, pairs;
};

__device__ static __forceinline__ tc_shape tc_shape_of(const struct exl3_tc_record &record)
{
    tc_shape shape;
    shape.hidden = record.hidden != 0u ? record.hidden : EXL3_TC_DEFAULT_HIDDEN;
    shape.intermediate = record.intermediate;
    shape.picks = record.pairs_per_row != 0u ? record.pairs_per_row : EXL3_TC_DEFAULT_PAIRS_PER_ROW;
    shape.pairs = record.row_count * shape.picks;
    return shape;
}

__device__ static __forceinline__ uint32_t tc_bits_x2(const struct exl3_tc_record &record, const unsigned char *arena,
                                                      uint32_t expert, uint32_t matrix)
{
    if (record.widths_offset == 0u) {
        return record.bits_x2;
    }
    if (expert >= record.expert_count) {
        return 0u; /* beyond the table: no width, which every launch treats as a matrix it cannot decode */
    }
    return exl3_bits_x2(exl3_width_of(((const uint32_t *)(arena + record.widths_offset))[expert], matrix));
}

/* launch 0: grid (hidden / 128, job_capacity, 2), block 64 */
extern "C" __global__ void exl3_tc_operands(struct exl3_tc_record record, unsigned char *arena)
{
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + record.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const tc_shape shape = tc_shape_of(record);
    const uint32_t lane = threadIdx.x, projection = blockIdx.z, channel = blockIdx.x * EXL3_TRANSFORM + lane;
    const uint64_t matrix = projection == 0u ? job->gate_offset : job->up_offset;
    const uint16_t *suh = (const uint16_t *)(arena + matrix + exl3_code_bytes(shape.hidden, shape.intermediate,
                                                                               tc_bits_x2(record, arena, job->expert, projection)));
    const float s0 = half_bits_to_float(suh[channel]), s1 = half_bits_to_float(suh[channel + WAVE]);
    const uint16_t *rows = (const uint16_t *)(arena + record.hidden_offset);
    uint16_t *operands = (uint16_t *)(arena + record.workspace_offset);
    for (uint32_t column = 0; column < job->row_count; column++) {
        const uint32_t pair = job->pair_index[column];
        const uint64_t row = pair / shape.picks;
        float v0 = __fmul_rn(bf16_to_float(rows[row * shape.hidden + channel]), s0);
        float v1 = __fmul_rn(bf16_to_float(rows[row * shape.hidden + channel + WAVE]), s1);
        wave_hadamard128(v0, v1, lane);
        uint16_t *out = operands + ((uint64_t)projection * shape.pairs + pair) * shape.hidden;
        out[channel] = float_to_half_bits(__fmul_rn(v0, EXL3_NORMALIZATION));
        out[channel + WAVE] = float_to_half_bits(__fmul_rn(v1, EXL3_NORMALIZATION));
    }
}
ANEMONE_KERNEL(EXL3_TC_KERNEL_FILE, exl3_tc_operands, exl3_tc_record);

/* one wavefront item: a strip of EXL3_TC_STRIP_OUTPUTS outputs by one K slice of one matrix of one job */
template <uint32_t bits_x2>
__device__ static __forceinline__ void tc_item(const uint32_t *codes, uint32_t inputs, uint32_t outputs,
                                               uint32_t strip, uint32_t slice, uint32_t slices,
                                               const struct expert_job_record *job, const half_t *operands,
                                               float *partials, uint32_t lane)
{
    const uint32_t column = lane % 16u;
    const bool live = column < job->row_count;
    /* a column that is not live reads the first column's operand: its sums are not stored */
    const uint32_t pair = job->pair_index[live ? column : 0u];
    const uint32_t steps = inputs / (4u * EXL3_TILE); /* a slice is a whole number of steps of four K tiles */
    float4_t accumulator[STRIP_PAIRS][2];
    exl3_stream_product<bits_x2, STRIP_PAIRS, EXACT_WEIGHTS>(codes, outputs / EXL3_TILE, strip * 2u * STRIP_PAIRS, 4u * (steps * slice / slices),
                                                             4u * (steps * (slice + 1u) / slices), operands + (uint64_t)pair * inputs, lane,
                                                             accumulator);
    if (live) {
        float *out = partials + (uint64_t)pair * outputs;
#pragma unroll
        for (uint32_t p = 0; p < STRIP_PAIRS; p++) {
#pragma unroll
            for (uint32_t h = 0; h < 2u; h++) {
                *(float4_t *)(out + exl3_stream_output(strip * 2u * STRIP_PAIRS, p, h, lane)) = accumulator[p][h];
            }
        }
    }
}

/* launches 1 and 3: grid (outputs / EXL3_TC_STRIP_OUTPUTS, job_capacity, matrices * slices / 4), block 256: the block's four
 * wavefronts take four consecutive (matrix, slice) items of one strip (a strip of fewer than four items: the items of
 * adjacent strips, the grid's x that many times smaller and its z 1). pass 0: gate and up; pass 1: down. A slice is
 * a whole number of steps of four K tiles. */
__device__ static __forceinline__ void tc_products_block(const struct exl3_tc_record &record, unsigned char *arena, uint32_t block_x,
                                                         uint32_t block_y, uint32_t block_z, uint32_t lane, uint32_t wave)
{
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + record.jobs_offset) + block_y;
    if (job->row_count == 0u) {
        return;
    }
    const tc_shape shape = tc_shape_of(record);
    const bool down = record.pass != 0u;
    const uint32_t slices = down ? EXL3_TC_DOWN_SLICES : EXL3_TC_GATE_UP_SLICES;
    /* a strip's items: projection * slices + slice; fewer than a block's wavefronts: the block takes adjacent strips */
    const uint32_t strip_items = (down ? 1u : 2u) * slices;
    const uint32_t place = block_z * PRODUCT_WAVES + wave;
    const uint32_t item = strip_items >= PRODUCT_WAVES ? place : place % strip_items;
    const uint32_t strip = strip_items >= PRODUCT_WAVES ? block_x : block_x * (PRODUCT_WAVES / strip_items) + place / strip_items;
    const uint32_t projection = item / slices, slice = item % slices;
    const uint32_t inputs = down ? shape.intermediate : shape.hidden;
    const uint32_t outputs = down ? shape.hidden : shape.intermediate;
    const uint64_t matrix = down ? job->down_offset : projection == 0u ? job->gate_offset : job->up_offset;
    const uint32_t bits_x2 = tc_bits_x2(record, arena, job->expert, down ? 2u : projection);
    unsigned char *workspace = arena + record.workspace_offset;
    const half_t *operands = (const half_t *)workspace + (down ? 0u : (uint64_t)projection * shape.pairs * inputs);
    float *partials;
    if (down) {
        partials = (float *)(workspace + exl3_tc_operand_bytes(shape.pairs, shape.hidden) +
                             exl3_tc_gate_up_bytes(shape.pairs, shape.intermediate)) +
                   (uint64_t)slice * shape.pairs * outputs;
    } else {
        partials = (float *)(workspace + exl3_tc_operand_bytes(shape.pairs, shape.hidden)) +
                   ((uint64_t)slice * 2u + projection) * shape.pairs * outputs;
    }
    const uint32_t *codes = (const uint32_t *)(arena + matrix);
    switch (bits_x2) {
    case 4u: tc_item<4u>(codes, inputs, outputs, strip, slice, slices, job, operands, partials, lane); break;
    case 5u: tc_item<5u>(codes, inputs, outputs, strip, slice, slices, job, operands, partials, lane); break;
    case 6u: tc_item<6u>(codes, inputs, outputs, strip, slice, slices, job, operands, partials, lane); break;
    case 8u: tc_item<8u>(codes, inputs, outputs, strip, slice, slices, job, operands, partials, lane); break;
    default:
        /* a width this build does not decode (the prepare function refuses the one width of a record; a table's widths
         * are the caller's): zeros, so that the launches behind this one add nothing stale */
        if (lane % 16u < job->row_count) {
            float *out = partials + (uint64_t)job->pair_index[lane % 16u] * outputs;
#pragma unroll
            for (uint32_t p = 0; p < STRIP_PAIRS; p++) {
#pragma unroll
                for (uint32_t h = 0; h < 2u; h++) {
                    *(float4_t *)(out + exl3_stream_output(strip * 2u * STRIP_PAIRS, p, h, lane)) = (float4_t){0.0f, 0.0f, 0.0f, 0.0f};
                }
            }
        }
        break;
    }
}

extern "C" __global__ void __launch_bounds__(PRODUCT_THREADS, 4)
    exl3_tc_products(struct exl3_tc_record record, unsigned char *arena)
{
    tc_products_block(record, arena, blockIdx.x, blockIdx.y, blockIdx.z, threadIdx.x % WAVE, __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE));
}
ANEMONE_KERNEL(EXL3_TC_KERNEL_FILE, exl3_tc_products, exl3_tc_record);

/* launch 2: grid (intermediate / 128, job_capacity), block 64 */
extern "C" __global__ void exl3_tc_activate(struct exl3_tc_record record, unsigned char *arena)
{
    const struct expert_job_record *job = (const struct expert_job_record *)(arena + record.jobs_offset) + blockIdx.y;
    if (job->row_count == 0u) {
        return;
    }
    const tc_shape shape = tc_shape_of(record);
    const uint32_t lane = threadIdx.x, channel = blockIdx.x * EXL3_TRANSFORM + lane;
    const uint32_t H = shape.hidden, I = shape.intermediate;
    const uint16_t *gate_svh = (const uint16_t *)(arena + job->gate_offset + exl3_code_bytes(H, I, tc_bits_x2(record, arena, job->expert, 0u))) + H;
    const uint16_t *up_svh = (const uint16_t *)(arena + job->up_offset + exl3_code_bytes(H, I, tc_bits_x2(record, arena, job->expert, 1u))) + H;
    const uint16_t *down_suh = (const uint16_t *)(arena + job->down_offset + exl3_code_bytes(I, H, tc_bits_x2(record, arena, job->expert, 2u)));
    const float gs[2] = {half_bits_to_float(gate_svh[channel]), half_bits_to_float(gate_svh[channel + WAVE])};
    const float us[2] = {half_bits_to_float(up_svh[channel]), half_bits_to_float(up_svh[channel + WAVE])};
    const float ds[2] = {half_bits_to_float(down_suh[channel]), half_bits_to_float(down_suh[channel + WAVE])};
    const float limit = record.activation_limit;
    unsigned char *workspace = arena + record.workspace_offset;
    const float *partials = (const float *)(workspace + exl3_tc_operand_bytes(shape.pairs, H));
    for (uint32_t column = 0; column < job->row_count; column++) {
        const uint32_t pair = job->pair_index[column];
        float g[2] = {0.0f, 0.0f}, u[2] = {0.0f, 0.0f};
        for (uint32_t slice = 0; slice < EXL3_TC_GATE_UP_SLICES; slice++) { /* in slice order from +0 */
            const float *gate = partials + ((uint64_t)slice * 2u * shape.pairs + pair) * I;
            const float *up = partials + (((uint64_t)slice * 2u + 1u) * shape.pairs + pair) * I;
            g[0] = __fadd_rn(g[0], gate[channel]);
            g[1] = __fadd_rn(g[1], gate[channel + WAVE]);
            u[0] = __fadd_rn(u[0], up[channel]);
            u[1] = __fadd_rn(u[1], up[channel + WAVE]);
        }
        wave_hadamard128(g[0], g[1], lane);
        wave_hadamard128(u[0], u[1], lane);
        float v[2];
#pragma unroll
        for (uint32_t i = 0; i < 2u; i++) {
            const float gate = __fmul_rn(__fmul_rn(g[i], EXL3_NORMALIZATION), gs[i]);
            const float up = __fmul_rn(__fmul_rn(u[i], EXL3_NORMALIZATION), us[i]);
            const float bounded_gate = limit > 0.0f ? fminf(gate, limit) : gate;
            const float bounded_up = limit > 0.0f ? fminf(fmaxf(up, -limit), limit) : up;
            const float hidden = __fmul_rn(det_silu(bounded_gate), bounded_up);
            v[i] = __fmul_rn(hidden, ds[i]);
        }
        wave_hadamard128(v[0], v[1], lane);
        uint16_t *operand = (uint16_t *)workspace + (uint64_t)pair * I;
        operand[channel] = float_to_half_bits(__fmul_rn(v[0], EXL3_NORMALIZATION));
        operand[channel + WAVE] = float_to_half_bits(__fmul_rn(v[1], EXL3_NORMALIZATION));
    }
}
ANEMONE_KERNEL(EXL3_TC_KERNEL_FILE, exl3_tc_activate, exl3_tc_record);

/* launch 4: grid (hidden / 128, row_count), block 64 x ROUTER_MOST_PICKS: wavefront s takes the row's pair of slot s
 * (its down sums in slice order, the output transform, the output scales, the route weight); wavefront 0 then adds the
 * slots' values in slot order. A wavefront runs one instruction at a time: eight slots side by side are an eighth of
 * the instructions one wavefront would run for the row. */
extern "C" __global__ void __launch_bounds__(COMBINE_THREADS) exl3_tc_combine(struct exl3_tc_record record, unsigned char *arena)
{
    __shared__ float values[ROUTER_MOST_PICKS][EXL3_TRANSFORM];
    __shared__ uint32_t is_held[ROUTER_MOST_PICKS];
    const tc_shape shape = tc_shape_of(record);
    const uint32_t lane = threadIdx.x % WAVE, slot = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t channel = blockIdx.x * EXL3_TRANSFORM + lane, row = blockIdx.y;
    const uint32_t H = shape.hidden, I = shape.intermediate;
    const struct expert_job_record *jobs = (const struct expert_job_record *)(arena + record.jobs_offset);
    const unsigned char *workspace = arena + record.workspace_offset;
    const float *partials = (const float *)(workspace + exl3_tc_operand_bytes(shape.pairs, H) + exl3_tc_gate_up_bytes(shape.pairs, I));
    bool held = false;
    float y0 = 0.0f, y1 = 0.0f;
    if (slot < shape.picks) {
        const uint32_t pair = row * shape.picks + slot;
        /* the pair's sums are asked for first: they are inside the workspace whether a job holds the pair or not */
        float partial0[EXL3_TC_DOWN_SLICES], partial1[EXL3_TC_DOWN_SLICES];
#pragma unroll
        for (uint32_t slice = 0; slice < EXL3_TC_DOWN_SLICES; slice++) {
            const float *down = partials + ((uint64_t)slice * shape.pairs + pair) * H;
            partial0[slice] = down[channel];
            partial1[slice] = down[channel + WAVE];
        }
        /* the job and column that hold the pair: every lane looks at the jobs lane, lane + 64, ... (what it needs of a
         * job in four 16-byte loads asked for together); a pair is held at most once */
        static_assert(LINEAR_MAXIMUM_ROWS == 8u && offsetof(struct expert_job_record, down_offset) == 16u &&
                          offsetof(struct expert_job_record, pair_index) == 32u && sizeof(struct expert_job_record) == 96u,
                      "a job from its down offset on is five loads of 16 bytes");
        uint64_t down_offset = 0;
        uint32_t expert = 0;
        float weight = 0.0f;
        for (uint32_t base = 0; base < record.job_capacity && !held; base += WAVE) {
            const uint32_t index = base + lane;
            bool mine = false;
            uint64_t my_offset = 0;
            uint32_t my_expert = 0;
            float my_weight = 0.0f;
            if (index < record.job_capacity) {
                const uint4_t *job = (const uint4_t *)(jobs + index);
                const uint4_t head = job[1], low = job[2], high = job[3], weights_low = job[4], weights_high = job[5];
                const uint32_t count = head.z;
                const uint32_t indexes[LINEAR_MAXIMUM_ROWS] = {low.x, low.y, low.z, low.w, high.x, high.y, high.z, high.w};
                const uint32_t weights[LINEAR_MAXIMUM_ROWS] = {weights_low.x, weights_low.y, weights_low.z, weights_low.w,
                                                               weights_high.x, weights_high.y, weights_high.z, weights_high.w};
#pragma unroll
                for (uint32_t column = 0; column < LINEAR_MAXIMUM_ROWS; column++) {
                    const bool here = column < count && indexes[column] == pair;
                    mine = mine || here;
                    my_weight = here ? __uint_as_float(weights[column]) : my_weight;
                }
                my_offset = ((uint64_t)head.y << 32) | head.x;
                my_expert = head.w;
            }
            const uint64_t holders = __builtin_amdgcn_ballot_w64(mine);
            if (holders != 0ull) { /* the same in every lane */
                const int holder = __builtin_ctzll(holders);
                held = true;
                down_offset = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(my_offset >> 32), holder) << 32) |
                              (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)my_offset, holder);
                expert = (uint32_t)__builtin_amdgcn_readlane((int)my_expert, holder);
                weight = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(my_weight), holder));
            }
        }
        if (held) {
            const uint16_t *svh = (const uint16_t *)(arena + down_offset + exl3_code_bytes(I, H, tc_bits_x2(record, arena, expert, 2u))) + I;
            const float scale0 = half_bits_to_float(svh[channel]), scale1 = half_bits_to_float(svh[channel + WAVE]);
            float v0 = 0.0f, v1 = 0.0f;
#pragma unroll
            for (uint32_t slice = 0; slice < EXL3_TC_DOWN_SLICES; slice++) { /* in slice order from +0 */
                v0 = __fadd_rn(v0, partial0[slice]);
                v1 = __fadd_rn(v1, partial1[slice]);
            }
            wave_hadamard128(v0, v1, lane);
            y0 = __fmul_rn(__fmul_rn(__fmul_rn(v0, EXL3_NORMALIZATION), scale0), weight);
            y1 = __fmul_rn(__fmul_rn(__fmul_rn(v1, EXL3_NORMALIZATION), scale1), weight);
        }
    }
    values[slot][lane] = y0;
    values[slot][lane + WAVE] = y1;
    if (lane == 0u) {
        is_held[slot] = held ? 1u : 0u;
    }
    __syncthreads();
    if (slot != 0u) {
        return;
    }
    float sum0 = 0.0f, sum1 = 0.0f;
    for (uint32_t other = 0; other < shape.picks; other++) {
        if (is_held[other] != 0u) { /* a pair no job holds (a row beyond the live ones) adds nothing */
            sum0 = __fadd_rn(sum0, values[other][lane]);
            sum1 = __fadd_rn(sum1, values[other][lane + WAVE]);
        }
    }
    if (record.shared_sum != 0u) {
        /* the sum joins the shared expert's bfloat16 row, in place: bfloat16(sum + row), one rounding of the float32
         * addition's result (source/kernel_exl3_tc.cu:468-471 of the reference); output_offset is not written */
        uint16_t *shared = (uint16_t *)(arena + record.shared_offset) + (uint64_t)row * H;
        shared[channel] = float_to_bf16(__fadd_rn(sum0, bf16_to_float(shared[channel])));
        shared[channel + WAVE] = float_to_bf16(__fadd_rn(sum1, bf16_to_float(shared[channel + WAVE])));
        return;
    }
    float *out = (float *)(arena + record.output_offset) + (uint64_t)row * H;
    out[channel] = sum0;
    out[channel + WAVE] = sum1;
}
ANEMONE_KERNEL(EXL3_TC_KERNEL_FILE, exl3_tc_combine, exl3_tc_record);

/* ---- the fused decode for callers that cannot allocate: the workspace in an array of the library's own ---- */

/* Every device the library runs on holds its own copy of this array, at its own address, until the process ends. The
 * name stands for the array in host code only as a symbol: its device address is asked for once a device. */
static __device__ __align__(256) unsigned char scratch[EXL3_TC_STATIC_SCRATCH_BYTES];

#define STATIC_MOST_DEVICES 64

static result_status static_scratch_of(unsigned char **address_out)
{
    static std::mutex guard;
    static unsigned char *address_of[STATIC_MOST_DEVICES];
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= STATIC_MOST_DEVICES) {
        (void)fprintf(stderr, "anemone: exl3_tc_run_static: no current device among the first %d\n", STATIC_MOST_DEVICES);
        return STATUS_DEVICE_ERROR;
    }
    std::lock_guard<std::mutex> held(guard);
    if (address_of[device] == nullptr) {
        unsigned char *address = nullptr;
        const hipError_t asked = hipGetSymbolAddress((void **)&address, HIP_SYMBOL(scratch));
        if (asked != hipSuccess || address == nullptr) {
            (void)fprintf(stderr, "anemone: exl3_tc_run_static: hipGetSymbolAddress: %s\n", hipGetErrorString(asked));
            return STATUS_DEVICE_ERROR;
        }
        address_of[device] = address;
    }
    *address_out = address_of[device];
    return STATUS_OK;
}

/* card_open's part of the set-up: the array's address on the card's device (current when this is called) is asked for
 * there, so that the code object is loaded and the address known before the first step; a call of exl3_tc_run_static on
 * a device no card was opened on still resolves it itself, once, and that one call is not one to make under capture */
extern "C" result_status exl3_tc_static_scratch_resolve(void)
{
    unsigned char *address = nullptr;
    return static_scratch_of(&address);
}

/* kernel_prepare of a table that launches nothing: the four kernels of this file by number */
static const char *const static_kernel_names[] = {"exl3_tc_operands", "exl3_tc_products", "exl3_tc_activate", "exl3_tc_combine"};

static result_status static_kernel_prepare(struct device_card *, const char *file, const char *function, uint32_t record_bytes,
                                           uint32_t *kernel_out)
{
    if (strcmp(file, EXL3_TC_KERNEL_FILE) != 0 || record_bytes != sizeof(struct exl3_tc_record)) {
        return STATUS_INVALID_ARGUMENT;
    }
    for (uint32_t index = 0; index < 4u; index++) {
        if (strcmp(function, static_kernel_names[index]) == 0) {
            *kernel_out = index;
            return STATUS_OK;
        }
    }
    return STATUS_INVALID_ARGUMENT;
}

extern "C" result_status exl3_tc_run_static(const struct exl3_tc_record *record, void *arena_device, uint64_t arena_byte_count,
                                            void *stream)
{
    if (record == nullptr || arena_device == nullptr) {
        (void)fprintf(stderr, "anemone: exl3_tc_run_static: a missing argument\n");
        return STATUS_INVALID_ARGUMENT;
    }
    const uint32_t hidden = record->hidden != 0u ? record->hidden : EXL3_TC_DEFAULT_HIDDEN;
    const uint32_t picks = record->pairs_per_row != 0u ? record->pairs_per_row : EXL3_TC_DEFAULT_PAIRS_PER_ROW;
    const uint64_t pairs = (uint64_t)record->row_count * picks;
    if (record->row_count > EXL3_TC_MOST_ROWS || picks > ROUTER_MOST_PICKS || hidden > (1u << 20) || record->intermediate > (1u << 20) ||
        exl3_tc_workspace_bytes(pairs, hidden, record->intermediate) > EXL3_TC_STATIC_SCRATCH_BYTES) {
        (void)fprintf(stderr, "anemone: exl3_tc_run_static: a step of %u rows of %u pairs, hidden %u, intermediate %u needs a workspace "
                              "above the library's %u bytes\n", record->row_count, picks, hidden, record->intermediate,
                      EXL3_TC_STATIC_SCRATCH_BYTES);
        return STATUS_INVALID_ARGUMENT;
    }
    unsigned char *workspace = nullptr;
    const result_status found = static_scratch_of(&workspace);
    if (found != STATUS_OK) {
        return found;
    }
    struct backend_operations table;
    memset(&table, 0, sizeof table);
    table.kernel_prepare = static_kernel_prepare;
    struct exl3_tc_record stamped = *record;
    stamped.workspace_offset = 0u; /* checked for its alignment alone; the launches get the array's own offset below */
    struct kernel_launch launches[EXL3_TC_LAUNCHES];
    int placeholder = 0;
    const result_status prepared = exl3_tc_prepare_detached(&stamped, arena_byte_count, &table, (struct device_card *)&placeholder, launches);
    if (prepared != STATUS_OK) {
        return prepared;
    }
    /* arena + offset is computed in 64 bits on the card: the difference of the two addresses names the array from the
     * arena whichever lies higher */
    const uint64_t offset = (uint64_t)(uintptr_t)workspace - (uint64_t)(uintptr_t)arena_device;
    typedef void (*entry)(struct exl3_tc_record, unsigned char *);
    const entry entries[4] = {exl3_tc_operands, exl3_tc_products, exl3_tc_activate, exl3_tc_combine};
    for (uint32_t index = 0; index < EXL3_TC_LAUNCHES; index++) {
        struct exl3_tc_record argument;
        memcpy(&argument, launches[index].argument, sizeof argument);
        argument.workspace_offset = offset;
        hipLaunchKernelGGL(entries[launches[index].kernel], dim3(launches[index].grid[0], launches[index].grid[1], launches[index].grid[2]),
                           dim3(launches[index].block[0], launches[index].block[1], launches[index].block[2]), 0, (hipStream_t)stream,
                           argument, (unsigned char *)arena_device);
        const hipError_t launched = hipGetLastError();
        if (launched != hipSuccess) {
            (void)fprintf(stderr, "anemone: exl3_tc_run_static: launch %u: %s\n", index, hipGetErrorString(launched));
            return STATUS_DEVICE_ERROR;
        }
    }
    return STATUS_OK;
}
