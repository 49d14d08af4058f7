// Scalar low-precision helpers shared by the HIP kernels (gfx950).
//
// Software casts are used on slow paths (tiles holding NaN/inf, extreme scale
// exponents) and by the on-device self tests that compare the hardware
// conversion instructions against them over every input.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lowp {

__device__ __forceinline__ uint32_t f2u(float f) { return __float_as_uint(f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __uint_as_float(u); }

constexpr float kE4M3Max = 448.0f;

// fp32 -> OCP e4m3fn, round-to-nearest-even, no saturation (magnitudes that
// round past 448 give the NaN code 0x7F), sign kept for NaN.
__device__ __forceinline__ uint8_t sw_f32_to_e4m3fn(float f)
{
    uint32_t u = f2u(f);
    uint32_t sign = (u >> 24) & 0x80u;
    uint32_t a = u & 0x7FFFFFFFu;
    uint32_t code;
    if (a >= 0x43F00000u) {                 // >= 480, inf, NaN
        code = 0x7Fu;
    } else if (a < 0x3C800000u) {           // < 2^-6: subnormal target, quantum 2^-9
        // adding 2^14 aligns the quantum with the fp32 ulp, so the add rounds RNE
        float t = u2f(a) + 16384.0f;
        code = f2u(t) - 0x46800000u;
    } else {
        uint32_t odd = (a >> 20) & 1u;
        a += 0x7FFFFu + odd;                // RNE on the 20 dropped bits
        code = (a >> 20) - ((127u - 7u) << 3);
        if (code > 0x7Eu) code = 0x7Fu;     // rounded past 448
    }
    return (uint8_t)(sign | code);
}

__device__ __forceinline__ float sw_e4m3fn_to_f32(uint8_t c)
{
    uint32_t sign = ((uint32_t)c & 0x80u) << 24;
    uint32_t e = (c >> 3) & 0xFu, m = c & 7u;
    uint32_t bits;
    if (e == 15u && m == 7u) bits = 0x7FC00000u;
    else if (e == 0u) return u2f(sign | f2u((float)m * 0.001953125f));
    else bits = ((e + 120u) << 23) | (m << 20);
    return u2f(sign | bits);
}

// fp32 -> bf16 bits, RNE, NaN -> 0x7FC0.
__device__ __forceinline__ uint16_t sw_f32_to_bf16(float f)
{
    uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0u;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return u2f(h << 16); }

// e8m0 byte -> fp32: 2^(b-127); 0xFF -> NaN; 0x00 -> 2^-127 (fp32 subnormal).
__device__ __forceinline__ float e8m0_to_f32(uint32_t b)
{
    if (b == 0xFFu) return u2f(0x7FC00000u);
    if (b == 0u) return u2f(0x00400000u);
    return u2f(b << 23);
}

// fp32 -> e8m0: sign dropped, nearest power of two with the hidden bit acting
// as the LSB for ties (normal values round half up, subnormals half down);
// inf/NaN -> 0xFF.
__device__ __forceinline__ uint8_t f32_to_e8m0(float f)
{
    uint32_t u = f2u(f);
    uint32_t e = (u >> 23) & 0xFFu;
    if (e == 0xFFu) return 0xFFu;
    uint32_t g = (u >> 22) & 1u, rest = u & 0x3FFFFFu;
    if (g && (rest || e > 0u)) e += 1u;
    return (uint8_t)e;
}

// exact ceil(log2(r)) for finite r > 0, from the bit pattern.
__device__ __forceinline__ int ceil_log2_exact(float r)
{
    uint32_t u = f2u(r);
    int e = (int)((u >> 23) & 0xFFu);
    uint32_t m = u & 0x7FFFFFu;
    if (e == 0) {
        int top = 31 - __clz((int)m);
        return (top - 149) + ((m & (m - 1u)) ? 1 : 0);
    }
    return (e - 127) + (m ? 1 : 0);
}

// e2m1 code point (4 bits) -> fp32; code 8 is -0 when neg_zero, else +0.
__device__ __forceinline__ float sw_e2m1_to_f32(uint32_t code, bool neg_zero)
{
    uint32_t mag = code & 7u;
    uint32_t bits;
    if (mag == 0u) bits = 0u;
    else if (mag == 1u) bits = 0x3F000000u;                        // 0.5
    else bits = (((mag >> 1) + 126u) << 23) | ((mag & 1u) << 22);   // (1 + m/2) * 2^(e-1)
    if ((code & 8u) && (mag != 0u || neg_zero)) bits |= 0x80000000u;
    return u2f(bits);
}

// e2m1 code of y with ties to the smaller magnitude; the sign bit of y (also of -0) is bit 3
__device__ __forceinline__ uint32_t sw_f32_to_e2m1_half_down(float y)
{
    const float a = __builtin_fabsf(y);
    uint32_t code = (a > 0.25f) + (a > 0.75f) + (a > 1.25f) + (a > 1.75f) + (a > 2.5f) + (a > 3.5f) + (a > 5.0f);
    if (a != a) code = 7u;                      // NaN: above every boundary
    return code | ((f2u(y) >> 28) & 8u);
}

// Correctly rounded v / s from a correctly rounded reciprocal y = RN(1/s):
// two residual corrections.  After the first, q1 is a faithful rounding of
// v/s; the second then lands on RN(v/s) (Markstein).  Requires that neither
// y nor the residuals leave the normal range: callers use it only for
// 2^-60 <= s <= 2^60 and fall back to a true division otherwise.  Quotients
// whose magnitude is far below 2^-10 may be off by an ulp when v itself is
// near the subnormal range; they round to zero in e4m3fn either way.
__device__ __forceinline__ float div_by_recip(float v, float s, float y)
{
    float q0 = v * y;
    float r0 = __builtin_fmaf(-s, q0, v);
    float q1 = __builtin_fmaf(r0, y, q0);
    float r1 = __builtin_fmaf(-s, q1, v);
    float q2 = __builtin_fmaf(r1, y, q1);
    // s > 0, so the quotient carries the sign of v; the corrections above turn
    // -0 into +0 (x + -x and +0 + -0 are +0), so the sign is put back
    return u2f((f2u(v) & 0x80000000u) | f2u(q2));
}

__device__ __forceinline__ bool recip_div_safe(float s) { return s >= 0x1p-60f && s <= 0x1p60f; }

}  // namespace lowp
