// Shared device/host helpers for the MI355X (gfx950, wave64) MoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/picomoe.h"

#define PICOMOE_CHECK_ARG(cond)                 \
    do {                                        \
        if (!(cond)) return PICOMOE_ERR_ARG;    \
    } while (0)

// Launch errors are reported as PICOMOE_ERR_HIP_BASE + hipError_t.
static inline int picomoe_launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? PICOMOE_OK : PICOMOE_ERR_HIP_BASE + (int)e;
}

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

constexpr int kWave = 64;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// round-to-nearest-even fp32 -> bf16 bit pattern (NaN stays NaN)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    __bf16 h = (__bf16)f;  // v_cvt_pk_bf16_f32 on gfx950
    return (uint32_t)__builtin_bit_cast(uint16_t, h);
}

// two fp32 -> two bf16 in one register (one v_cvt_pk_bf16_f32; round-to-nearest-even like f32_to_bf16_bits)
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

template <typename T>
__device__ __forceinline__ T wave_max(T v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        T o = __shfl_xor(v, off, kWave);
        v = o > v ? o : v;
    }
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
