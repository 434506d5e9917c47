// Activation functions and code packing shared by the quantise kernels and by the GEMM epilogue
// that writes codes: both must turn a value into the same code bit for bit.
#pragma once
#include "segq_common.h"

namespace segq {

// ---- the producer's activation function, fused -----------------------------
// What the layer in front of the linear would have written to memory in the
// tensor's own dtype: op(x), or x * op(gate), each result rounded to that dtype
// (torch evaluates these in fp32 and rounds once per operator).  The formulas
// are torch's: gelu(tanh) = 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))),
// gelu = 0.5 x (1 + erf(x / sqrt 2)), silu = x / (1 + exp(-x)).
// The transcendental parts run on the hardware's exp2 and reciprocal (an ulp
// each) instead of the math library's tanhf / erff / expf, which cost ~50
// instruction slots per element and made the fused kernel slower than the
// separate activation kernel it replaces:
//   0.5 (1 + tanh(u)) = 1 / (1 + e^(-2u))   (torch's 1 + tanhf(u) cancels for u < 0 and
//   carries an absolute error of an ulp of 1 there; this form keeps the relative accuracy)
//   1 + erf(z) = q or 2 - q for z < 0 or not, q = erfc(|z|) by Abramowitz and
//   Stegun 7.1.26 (absolute error below 1.5e-7; no cancellation for z < 0)
// Both are far inside a quantisation step of the codes they feed.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }

// (fp contraction is switched off inside: the quantise kernels and the GEMM epilogue that writes
// codes must evaluate the same operations, not whatever fused forms each call site invites)
__device__ __forceinline__ float act_value(int op, float x) {
#pragma clang fp contract(off)
    if (op == SEGQ_PRE_GELU_TANH) {
        // 0.5 x (1 + tanh u) = x / (1 + e^(-2u)), u = sqrt(2/pi) (x + 0.044715 x^3): nothing cancels
        const float w = x * __builtin_fmaf(0.044715f, x * x, 1.0f);
        return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(w * -2.3022081986f));  // 2 sqrt(2/pi) log2(e)
    }
    if (op == SEGQ_PRE_GELU) {
        const float z = fabsf(x) * 0.7071067811865476f;
        const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f, z, 1.0f));
        const float poly = t * __builtin_fmaf(t, __builtin_fmaf(t, __builtin_fmaf(t, __builtin_fmaf(t, 1.061405429f, -1.453152027f), 1.421413741f),
                                                                -0.284496736f), 0.254829592f);
        const float q = poly * fast_exp(-z * z);
        return x * 0.5f * (x < 0.0f ? q : 2.0f - q);
    }
    return x * __builtin_amdgcn_rcpf(1.0f + fast_exp(-x));  // SEGQ_PRE_SILU
}

// clamp first, then round half to even; a NaN operand is dropped by fmaxf and
// becomes the lower bound (segquant/src/real_quant/quantizer.cuh:31-35).
__device__ __forceinline__ int q_i8(float v) { return (int)rintf(fminf(fmaxf(v, -128.0f), 127.0f)); }
__device__ __forceinline__ int q_i4(float v) { return (int)rintf(fminf(fmaxf(v, -8.0f), 7.0f)); }

// e4m3 with saturation to +-448 (fminf/fmaxf drop a NaN operand, so NaN is
// patched afterwards: it encodes as 0x7F whatever its sign).
__device__ __forceinline__ float sat_e4m3(float v) { return fminf(fmaxf(v, -448.0f), 448.0f); }

__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d) {
    int r = __builtin_amdgcn_cvt_pk_fp8_f32(sat_e4m3(a), sat_e4m3(b), 0, false);
    r = __builtin_amdgcn_cvt_pk_fp8_f32(sat_e4m3(c), sat_e4m3(d), r, true);
    const uint32_t nan = (a != a ? 0xFFu : 0u) | (b != b ? 0xFF00u : 0u) | (c != c ? 0xFF0000u : 0u) |
                         (d != d ? 0xFF000000u : 0u);
    return ((uint32_t)r & ~nan) | (0x7F7F7F7Fu & nan);
}

// Four int8 codes in one dword.  Adding 1.5 * 2^23 to the clamped value rounds it to
// an integer (ties to even, as rintf) and leaves that integer, in two's complement,
// in the low mantissa bits: the low byte of the sum's bit pattern is the code.  One
// add instead of round + convert + mask, and three byte permutes per dword.
__device__ __forceinline__ uint32_t pack4_i8(float a, float b, float c, float d) {
    const float magic = 12582912.0f;
    const uint32_t ua = __float_as_uint(fminf(fmaxf(a, -128.0f), 127.0f) + magic);
    const uint32_t ub = __float_as_uint(fminf(fmaxf(b, -128.0f), 127.0f) + magic);
    const uint32_t uc = __float_as_uint(fminf(fmaxf(c, -128.0f), 127.0f) + magic);
    const uint32_t ud = __float_as_uint(fminf(fmaxf(d, -128.0f), 127.0f) + magic);
    const uint32_t lo = __builtin_amdgcn_perm(ub, ua, 0x0c0c0400u);  // ua.b0 | ub.b0 << 8
    const uint32_t hi = __builtin_amdgcn_perm(ud, uc, 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);             // lo.b0 lo.b1 hi.b0 hi.b1
}

// Rounds to the 16-bit dtype dt (SEGQ_BF16 / SEGQ_F16; anything else: unchanged) and back: what a
// tensor of that dtype would have held.
__device__ __forceinline__ float round_to(int dt, float v) {
    if (dt == SEGQ_BF16) return __uint_as_float(pack2_bf16(v, 0.0f) << 16);
    if (dt == SEGQ_F16) return f16_bits_to_f32(pack2_f16(v, 0.0f) & 0xffffu);
    return v;
}

}  // namespace segq
