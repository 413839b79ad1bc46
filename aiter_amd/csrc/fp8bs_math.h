// Scalar arithmetic shared by the quantisation kernels.  Plain C++ with no HIP dependency in
// the function bodies, so the same source can be compiled for the host by the CPU tests that
// check the fast division path exhaustively against IEEE division.
//
// Semantics being reproduced (aiter/ops/quant.py:64-94, torch CPU):
//     scale = amax / 448            one fp32 IEEE division; exact zero replaced by 1
//     code  = e4m3fn_rne(x / scale) one fp32 IEEE division, then round-to-nearest-even to
//                                   OCP e4m3fn with |q| > 464 (and inf/NaN) -> NaN code
#pragma once

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define FP8BS_HD __host__ __device__ __forceinline__
#else
#define FP8BS_HD static inline
#include <math.h>
#endif

namespace fp8bs {

FP8BS_HD uint32_t f32_bits(float f)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __float_as_uint(f);
#else
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
#endif
}

FP8BS_HD float bits_f32(uint32_t u)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __uint_as_float(u);
#else
    float f;
    memcpy(&f, &u, 4);
    return f;
#endif
}

FP8BS_HD float fma32(float a, float b, float c)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_fmaf(a, b, c);
#else
    return fmaf(a, b, c);
#endif
}

// The fast path is used only when the group's amax (a finite, normal fp32 taken from a 16-bit
// float) lies in [kFastAmaxMin, kFastAmaxMax]: then scale = amax/448, its reciprocal, every
// quotient (|q| <= 448.0001) and every residual below stay far from the subnormal and
// overflow ranges, which is what the exactness argument needs.
//   2^-80 <= amax <= 2^100
// The lower bound also keeps the residual exact for every x whose quotient can reach the fp8
// grid: |q| >= 2^-11 needs |x| >= amax * 2^-20 >= 2^-100, and the residual q0*s - x has its last
// bit at 2^-47 |x| >= 2^-149.  Smaller x give |q| < 2^-11, which encodes as (signed) zero even if
// the low bits of q are off.
constexpr uint32_t kFastAmaxMinBits = (127u - 80u) << 23;
constexpr uint32_t kFastAmaxMaxBits = (127u + 100u) << 23;

FP8BS_HD bool amax_allows_fast_path(uint32_t amax_bits)
{
    return amax_bits >= kFastAmaxMinBits && amax_bits <= kFastAmaxMaxBits;
}

// amax / 448 as IEEE division rounds it, without the division: the same three-operation sequence
// as div_by_scale below with the constant RN(1/448).  Holds for every amax that is a 16-bit float
// (bf16 or fp16, widened) inside the fast range; the CPU tests compare it with the division for
// every such value.
FP8BS_HD float amax_over_448(float m)
{
    const float c  = bits_f32(0x3b124925u); // RN(1 / 448)
    const float q0 = m * c;
    const float t  = fma32(q0, 448.0f, -m);
    return fma32(-t, c, q0);
}

// RN(1 / s) for 2^-100 <= |s| <= 2^100 without the division sequence (13 instructions with its scaling
// and fix-up): the hardware's reciprocal approximation and one Newton step.  Equal to the IEEE
// division for every float in that range (all 1.68e9 of them are compared on the GPU by
// tests/gpu_math); outside the range callers divide.  The host form is the division itself.
constexpr uint32_t kRecipMinBits = (127u - 100u) << 23;
constexpr uint32_t kRecipMaxBits = (127u + 100u) << 23;
FP8BS_HD float recip_in_range(float s)
{
#if defined(__HIP_DEVICE_COMPILE__)
    const float r0 = __builtin_amdgcn_rcpf(s);
    return fma32(fma32(-s, r0, 1.0f), r0, r0);
#else
    return 1.0f / s;
#endif
}

// RN(a / n) in fp64 from inv = RN(1 / n): q0 = RN(a * inv), the exact residual a - q0 * n by one FMA,
// one correction (the quotient is then the correctly rounded one provided inv is and n's significand
// is not all ones: n is a row length here).  An infinite a stays infinite (its residual is NaN).
FP8BS_HD double div_by_count(double a, double n, double inv)
{
    const double q0 = a * inv;
    const double r  = __builtin_fma(-q0, n, a);
    const double q  = __builtin_fma(r, inv, q0);
    return r == r ? q : q0;
}

// Correctly rounded x / s from the correctly rounded reciprocal r = RN(1 / s):
//     q0 = RN(x * r);  t = q0 * s - x (exact, one FMA);  q = RN(q0 - t * r)
// With r = RN(1/s) this sequence returns RN(x / s) for binary32 operands whenever no
// intermediate under/overflows (Markstein's theorem); the CPU tests additionally compare it
// with IEEE division for every 16-bit-float x against every reachable scale.
// The residual is formed as q0*s - x and subtracted (rather than x - q0*s and added) so that
// x = -0 yields -0, as IEEE division does: t = (-0)*s + (+0) = +0, q = (-0)*r + (-0) = -0.
FP8BS_HD float div_by_scale(float x, float s, float r)
{
    float q0 = x * r;
    float t  = fma32(q0, s, -x);
#if !defined(__HIP_DEVICE_COMPILE__) && defined(__x86_64__)
    // host builds only: keep the compiler from folding the negation of t into a fused
    // negate-multiply-subtract, whose zero result has the other sign
    __asm__ volatile("" : "+x"(t));
#endif
    return fma32(-t, r, q0);
}

// Software e4m3fn conversion (round to nearest even on the real value), used on the rare slow
// path and by host-side checks.  The fast path uses the hardware conversion instead; both
// agree on every finite |q| <= 464.
FP8BS_HD uint8_t f32_to_e4m3fn_sw(float f)
{
    uint32_t u    = f32_bits(f);
    uint32_t sign = (u >> 24) & 0x80u;
    uint32_t a    = u & 0x7fffffffu;
    if(a >= 0x43f00000u) // >= 480, inf, NaN
        return (uint8_t)(sign | 0x7fu);
    uint32_t code;
    if(a < 0x3c800000u) // below 2^-6: subnormal grid with quantum 2^-9
    {
        // adding 2^14 (ulp = 2^-9) makes the fp32 adder do the round-to-nearest-even
        float t = bits_f32(a) + 16384.0f;
        code    = f32_bits(t) - 0x46800000u;
    }
    else
    {
        uint32_t lsb = (a >> 20) & 1u;
        uint32_t rnd = a + 0x7ffffu + lsb;     // RNE on the 20 dropped mantissa bits
        code         = (rnd >> 20) - (120u << 3); // rebias 127 -> 7
    }
    if(code > 0x7fu)
        code = 0x7fu;
    return (uint8_t)(sign | code);
}

} // namespace fp8bs
