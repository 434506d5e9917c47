// Shared host/device helpers of libsegq (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include "segq.h"

namespace segq {

// Records a message for segq_last_error() and returns the status, so callers
// can write `return fail(SEGQ_ERR_ARG, "...")`.
int fail(int status, const char* fmt, ...);

// Checks the launch that was just enqueued.
int check_launch(const char* what);

// Compute units of the current device (read once per device).
int device_cus();

// hipFuncAttributeMaxDynamicSharedMemorySize for `kern`, set once per kernel and
// device: `done` is the kernel's own flag word, one bit per device ordinal.
int reserve_lds(const void* kern, int bytes, unsigned long long* done);

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);  // round to nearest even
    return u >> 16;
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return __half2float(__ushort_as_half((unsigned short)h));
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
    return (uint32_t)__half_as_ushort(__float2half_rn(f));
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// Two fp32 values rounded to nearest even and packed, a in the low half
// (v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32 on gfx950).
__device__ __forceinline__ float load_bias(const void* bias, int dtype, int64_t n) {
    if (dtype == SEGQ_F32) return static_cast<const float*>(bias)[n];
    const uint32_t h = static_cast<const uint16_t*>(bias)[n];
    return dtype == SEGQ_BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
}

__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{a, b}, bf16x2_t));
}
__device__ __forceinline__ uint32_t pack2_f16(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{a, b}, f16x2_t));
}

}  // namespace segq
