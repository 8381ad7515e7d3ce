/*
 * kernel_selfcheck.hip -- the library's check of its own short cuts in arithmetic. Two helpers of the kernels take a
 * shorter way than the arithmetic they are defined by: det_silu and det_sigmoid (no tests around the exponential) and quantize_codes4
 * (the card's FP8 conversions). This kernel runs both ways over every input there is and counts the disagreements, so
 * that a test on the card proves the two ways equal instead of sampling them. No counterpart in the reference; not on
 * the routed-expert path.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernel_registry.h"
#include "quantize_device.cuh"
#include "router_device.cuh"
#include "linear_device.cuh"

struct arithmetic_selfcheck_arguments {
    uint64_t output_offset; /* written: uint32 [threads of the grid][2]: disagreements, and the first input that disagreed */
    uint32_t check;         /* 0: det_silu over all 2^32 float32; 1: quantize_codes4 over all 2^16 values x 2^8 scale codes; 2: det_sigmoid; 3: linear_silu within its bound of det_silu */
    uint32_t reserved_zero;
};
static_assert(sizeof(struct arithmetic_selfcheck_arguments) == 16, "arithmetic_selfcheck_arguments ABI");

extern "C" __global__ void arithmetic_selfcheck(struct arithmetic_selfcheck_arguments arguments, unsigned char *arena)
{
    const uint64_t threads = (uint64_t)gridDim.x * blockDim.x, thread = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t disagreements = 0, first = 0;
    if (arguments.check == 0u) {
        for (uint64_t pattern = thread; pattern < (1ull << 32); pattern += threads) {
            const float gate = __uint_as_float((uint32_t)pattern);
            const float defined = __fdiv_rn(gate, __fadd_rn(1.0f, det_expf(-gate))), taken = det_silu(gate);
            const bool same = __float_as_uint(defined) == __float_as_uint(taken) || (defined != defined && taken != taken);
            if (!same && disagreements++ == 0u) {
                first = (uint32_t)pattern;
            }
        }
    } else if (arguments.check == 2u) {
        for (uint64_t pattern = thread; pattern < (1ull << 32); pattern += threads) {
            const float score = __uint_as_float((uint32_t)pattern);
            const float defined = __fdiv_rn(1.0f, __fadd_rn(1.0f, det_expf(-score))), taken = det_sigmoid(score);
            const bool same = __float_as_uint(defined) == __float_as_uint(taken) || (defined != defined && taken != taken);
            if (!same && disagreements++ == 0u) {
                first = (uint32_t)pattern;
            }
        }
    } else if (arguments.check == 3u) {
        for (uint64_t pattern = thread; pattern < (1ull << 32); pattern += threads) {
            const float gate = __uint_as_float((uint32_t)pattern);
            const float defined = det_silu(gate), taken = linear_silu(gate);
            const bool same = taken == defined || fabsf(taken - defined) <= __fmaf_rn(LINEAR_SILU_BOUND, fabsf(defined), LINEAR_SILU_FLOOR) ||
                              (defined != defined && taken != taken);
            if (!same && disagreements++ == 0u) {
                first = (uint32_t)pattern;
            }
        }
    } else {
        for (uint64_t pattern = thread; pattern < (1ull << 24); pattern += threads) {
            const uint32_t code_exponent = (uint32_t)(pattern >> 16), value = (uint32_t)pattern & 0xFFFFu;
            /* the value in each of the four places, beside three others */
            const uint32_t bits[4] = {value, (value + 0x1111u) & 0xFFFFu, (value + 0x8421u) & 0xFFFFu, value ^ 0x8000u};
            uint32_t codes, carried[4];
            quantize_codes4(bits, code_exponent, codes, carried);
            const uint32_t pairs[2] = {quantize_operand_pair(carried[0], carried[1], code_exponent),
                                       quantize_operand_pair(carried[2], carried[3], code_exponent)};
            bool same = true;
#pragma unroll
            for (uint32_t i = 0; i < 4u; i++) {
                uint32_t code, operand;
                quantize_code_defined(bits[i], code_exponent, code, operand);
                same = same && code == ((codes >> (8u * i)) & 0xFFu) && operand == ((pairs[i / 2u] >> (16u * (i % 2u))) & 0xFFFFu);
            }
            uint32_t code, operand, one_code, one_operand;
            quantize_code_defined(value, code_exponent, code, operand);
            quantize_code(value, code_exponent, one_code, one_operand);
            same = same && code == one_code && operand == one_operand;
            if (!same && disagreements++ == 0u) {
                first = (uint32_t)pattern;
            }
        }
    }
    uint32_t *output = (uint32_t *)(arena + arguments.output_offset) + 2u * thread;
    output[0] = disagreements;
    output[1] = first;
}
ANEMONE_KERNEL("kernel_selfcheck", arithmetic_selfcheck, arithmetic_selfcheck_arguments);
