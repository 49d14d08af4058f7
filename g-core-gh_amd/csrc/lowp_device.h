// Device-side building blocks shared by the gfx950 quantise / convert kernels.
#pragma once
#include "lowp_common.h"
#include "lowp_math.h"

namespace lowp {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

struct BlockScale {
    float stored;   // the value written to scale_out (before the dtype cast)
    float div;      // DIV: divisor s;  MUL: multiplier f;  POW2: unused
    float recip;    // DIV fast path: RN(1/s)
    int exp2;       // POW2: e with s = 2^e
    bool fast;      // DIV: reciprocal path is safe
};

// scale modes that divide by a general divisor / by a power of two
constexpr bool div_like(int mode) { return mode == LP_SCALE_DIV || mode == LP_SCALE_RCP; }
constexpr bool pow2_like(int mode) { return mode == LP_SCALE_POW2 || mode == LP_SCALE_RCP_POW2; }
constexpr float kInv448 = 0.002232142857142857f;      // fl32(1 / 448)

template <int MODE>
__device__ __forceinline__ BlockScale derive_scale(float amax, float amax_floor, int zero_rule)
{
    BlockScale b;
    b.stored = 1.0f; b.div = 1.0f; b.recip = 1.0f; b.exp2 = 0; b.fast = true;
    if (MODE == LP_SCALE_POW2) {
        // amax_floor = 0: the all-zero rule of the eager quantiser; a positive floor (the round_sf branch of the
        // 1 x 128 / 128 x 128 test quantisers) replaces it, a floored block is never "all zero"
        const float a = amax < amax_floor ? amax_floor : amax;
        float safe = a < 1.17549435e-38f ? 1.17549435e-38f : a;
        float r = safe / kE4M3Max;
        int e = ceil_log2_exact(r);
        if (!(a > 0.0f)) e = 0;
        b.exp2 = e;
        b.stored = ldexpf(1.0f, e);
    } else if (MODE == LP_SCALE_RCP_POW2) {
        // bit-defined: exponent field - 127, + 1 when any mantissa bit is set; 2^e rebuilt from bits
        const float a = amax < amax_floor ? amax_floor : amax;
        const uint32_t rb = f2u(a * kInv448);
        const int e = (int)((rb >> 23) & 0xFFu) - 127 + ((rb & 0x7FFFFFu) ? 1 : 0);
        b.exp2 = e;
        b.stored = u2f((uint32_t)(e + 127) << 23);
    } else if (div_like(MODE)) {
        float a = amax < amax_floor ? amax_floor : amax;
        float s = MODE == LP_SCALE_RCP ? a * kInv448 : a / kE4M3Max;
        if (zero_rule == LP_ZERO_SCALE_TO_ONE && s == 0.0f) s = 1.0f;
        if (zero_rule == LP_ZERO_AMAX_TO_ONE && amax == 0.0f) s = 1.0f;
        b.div = s;
        b.stored = s;
        b.fast = recip_div_safe(s);
        b.recip = 1.0f / s;
    } else if (MODE == LP_SCALE_MUL_FLOOR) {
        const float a = amax < amax_floor ? amax_floor : amax;
        b.div = (1.0f / a) * kE4M3Max;
        b.stored = a / kE4M3Max;
    } else {
        // `448 / tensor` in torch is reciprocal(tensor) * 448: two roundings
        float f = amax > 0.0f ? (1.0f / amax) * kE4M3Max : 1.0f;
        b.div = f;
        b.stored = 1.0f / f;
    }
    return b;
}

// scaled value of one element on the fast path (finite block, sane scale)
template <int MODE>
__device__ __forceinline__ float scale_fast(float v, const BlockScale &b)
{
    if (pow2_like(MODE)) return ldexpf(v, -b.exp2);
    if (div_like(MODE)) return div_by_recip(v, b.div, b.recip);
    return v * b.div;
}

// literal arithmetic, used for blocks with NaN/inf or extreme scales
template <int MODE>
__device__ __forceinline__ uint8_t quant_slow(float v, const BlockScale &b)
{
    float y;
    if (pow2_like(MODE)) y = v / b.stored;
    else if (div_like(MODE)) y = v / b.div;
    else y = v * b.div;
    if (y > kE4M3Max) y = kE4M3Max;
    if (y < -kE4M3Max) y = -kE4M3Max;
    return sw_f32_to_e4m3fn(y);
}

// Slow-path worker, deliberately out of line and not unrolled so that it adds
// neither instructions nor registers to the hot kernels: quantises `n`
// consecutive elements starting at element `off` of x into q with the literal
// arithmetic.  `mul` is the factor of the MUL mode, `div` the divisor otherwise.
template <int MODE>
__device__ __noinline__ void quant_slow_span(const void *x, int is_bf16, int64_t off, int n, float div_or_mul,
                                             uint8_t *q)
{
    BlockScale b;
    b.stored = div_or_mul; b.div = div_or_mul; b.recip = 0.0f; b.exp2 = 0; b.fast = false;
#pragma unroll 1
    for (int j = 0; j < n; ++j) {
        float v = is_bf16 ? u2f((uint32_t)((const uint16_t *)x)[off + j] << 16) : ((const float *)x)[off + j];
        q[off + j] = quant_slow<MODE>(v, b);
    }
}

__device__ __forceinline__ float clamp448(float y) { return __builtin_amdgcn_fmed3f(y, -kE4M3Max, kE4M3Max); }

// four floats -> four e4m3fn bytes (element 0 in the low byte)
__device__ __forceinline__ uint32_t cvt4(float a, float b, float c, float d)
{
    // the first conversion keeps the other half of its destination and the second one overwrites that half:
    // starting from an undefined register (an asm output) saves the move that a zero would cost
    int w;
    asm volatile("" : "=v"(w));
    w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
    return (uint32_t)w;
}

__device__ __forceinline__ void store_scale(void *scale_out, int scale_dtype, int64_t idx, float s)
{
    if (scale_dtype == LP_F32) ((float *)scale_out)[idx] = s;
    else if (scale_dtype == LP_BF16) ((uint16_t *)scale_out)[idx] = sw_f32_to_bf16(s);
    else ((uint8_t *)scale_out)[idx] = f32_to_e8m0(s);
}

__device__ __forceinline__ float load_scale(const void *scale, int scale_dtype, int64_t idx)
{
    if (scale_dtype == LP_F32) return ((const float *)scale)[idx];
    if (scale_dtype == LP_BF16) return bf16_bits_to_f32(((const uint16_t *)scale)[idx]);
    return e8m0_to_f32(((const uint8_t *)scale)[idx]);
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t m)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        uint32_t o = (uint32_t)__shfl_xor((int)m, off, 64);
        m = o > m ? o : m;
    }
    return m;
}

// max over the 16 lanes of a DPP row, result in every lane
__device__ __forceinline__ uint32_t row16_max_u32(uint32_t m)
{
    uint32_t o;
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x128, 0xF, 0xF, false); m = o > m ? o : m;  // row_ror:8
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x124, 0xF, 0xF, false); m = o > m ? o : m;  // row_ror:4
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x122, 0xF, 0xF, false); m = o > m ? o : m;  // row_ror:2
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x121, 0xF, 0xF, false); m = o > m ? o : m;  // row_ror:1
    return m;
}

__device__ __forceinline__ uint32_t pack_bf16(float a, float b)
{
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// clear the sign bit of every e2m1 nibble whose magnitude bits are zero
__device__ __forceinline__ uint32_t fp4_pos_zero(uint32_t w)
{
    uint32_t m = w & 0x77777777u;
    uint32_t nz = (m + 0x77777777u) & 0x88888888u;   // bit 3 of a nibble set iff its magnitude != 0
    return w & (0x77777777u | nz);
}

// 4 packed bytes -> the 8 e2m1 table values (element 0 = low nibble of byte 0)
__device__ __forceinline__ void fp4_decode8(uint32_t x, float v[8])
{
    f32x2 t;
    t = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(x, 1.0f, 0); v[0] = t.x; v[1] = t.y;
    t = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(x, 1.0f, 1); v[2] = t.x; v[3] = t.y;
    t = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(x, 1.0f, 2); v[4] = t.x; v[5] = t.y;
    t = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(x, 1.0f, 3); v[6] = t.x; v[7] = t.y;
}

}  // namespace lowp
