/*
 * linear_device.cuh -- what the kernels of the FP4 / FP8 linears share: memory-to-LDS loads written as assembly, the
 * wait on them, the sizes of a tile's K step.
 */
#ifndef LINEAR_DEVICE_CUH
#define LINEAR_DEVICE_CUH

#include "exl3_device.cuh" /* det_expf, bf16 helpers, vector types */

typedef int int8_vector __attribute__((ext_vector_type(8)));

#define NIBBLE_STEP_BYTES 1024u /* a tile's K step of 128 inputs: 16 outputs x 128 inputs x 4 bits */
#define BYTE_STEP_BYTES 2048u   /* the same of one-byte weights */
#define NIBBLE_MASK 0x0F0F0F0Fu

typedef __attribute__((address_space(3))) void *lds_pointer;

/* Memory straight into LDS, 16 or 4 bytes a lane: lane L's bytes land at lds_base + 16 L (4 L); the address is a
 * base common to the wavefront plus the lane's own byte offset. Written as assembly so that the compiler keeps no
 * book on these loads: it would guard every LDS read that might alias one with a wait for all of them. The waits
 * are this file's own (wait_loads). A fence for the compiler as well, so the loads keep their order, which the waits
 * count on. */
__device__ static __forceinline__ void load_to_lds_16(const unsigned char *base, uint32_t lane_offset, uint32_t lds_base)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(lane_offset), "s"(base), "s"(lds_base)
                 : "memory", "m0");
}

__device__ static __forceinline__ void load_to_lds_4(const unsigned char *base, uint32_t lane_offset, uint32_t lds_base)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                 :
                 : "v"(lane_offset), "s"(base), "s"(lds_base)
                 : "memory", "m0");
}

/* gate / (1 + e^(-gate)) of the FP4 / FP8 experts' hidden step, by the card's own exponential and reciprocal (v_exp_f32,
 * v_rcp_f32: five instructions where the fixed float32 sequence with an IEEE division is twenty-eight). The reference
 * takes "the card's expf" here as well (source/kernel_linear_common.cuh:195-202 there): the hidden values are held to a
 * bound, not to bits, on either side. Within 2^-17 of det_silu's value, relatively (the rounding of gate log2(e) moves
 * the exponential by |gate| 2^-24 ln 2: 2^-20 down to a gate of -16, 2^-17.6 at -87), plus 2^-119 (below a gate of -87.3
 * the reciprocal is subnormal and the card gives 0 for a value of at most 1.03e-36), for every float32 gate (the library's
 * arithmetic_selfcheck kernel runs all 2^32); a not-a-number for a not-a-number, and for -infinity as there. */
#define LINEAR_SILU_BOUND 7.62939453125e-06f /* 2^-17 */
#define LINEAR_SILU_FLOOR 1.50463276905252801e-36f /* 2^-119 */
__device__ static __forceinline__ float linear_silu(float gate)
{
    const float e = __builtin_amdgcn_exp2f(__fmul_rn(gate, -1.44269502162933349609375f));
    return __fmul_rn(gate, __builtin_amdgcn_rcpf(__fadd_rn(1.0f, e)));
}

/* wait until at most `count` of the wavefront's memory loads are outstanding (they retire in order); also a fence
 * for the compiler: LDS reads of a stage stay behind the wait for the loads that fill it */
template <uint32_t count>
__device__ static __forceinline__ void wait_loads()
{
    static_assert(count < 64u, "vmcnt has six bits");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(count) : "memory");
}

#endif
