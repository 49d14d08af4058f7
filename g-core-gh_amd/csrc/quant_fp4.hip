// Block quantisation to packed FP4 (e2m1) with power-of-two (e8m0) block scales for gfx950.
//
//   quant_fp4_row32 : 1 x 32 blocks (the MoE expert layout).  A lane owns 8 consecutive values (one 16-byte
//                     load of bf16), four lanes own a block; the block amax is an integer max over sign-cleared
//                     bits, finished with two DPP quad swaps.  The scale exponent follows from the amax bits
//                     alone: 2^e is the smallest power of two with 6 * 2^e >= amax, i.e. e = E - 2 + (m > 1.5)
//                     for amax = m * 2^E -- which equals ceil(log2(fl(amax / 6))) for every fp32 amax (the
//                     rounding of the division never crosses a power of two).  The codes come from
//                     v_cvt_scalef32_pk_fp4_f32 (divides by the scale, rounds to nearest even, saturates at 6,
//                     packs two nibbles); the reference sends ties to the smaller magnitude, which differs from
//                     nearest-even exactly at |x| / 2^e in {0.75, 1.75, 3.5}: those inputs are moved one ulp
//                     towards zero first.  8 nibbles = one 4-byte store per lane.
//   quant_fp4_generic : any (bm, bn) with even bn, extreme exponents, inf: one workgroup per block, software
//                     rounding.
#include "lowp_device.h"

using namespace lowp;

namespace {

// scale exponent from the sign-cleared amax bits (finite): see the file comment
__device__ __forceinline__ int fp4_scale_exp(uint32_t mbits)
{
    if (mbits == 0u) return 0;                              // all-zero block: scale 1
    if (mbits < 0x00800000u) mbits = 0x00800000u;           // clamp(min = FLT_MIN)
    return (int)(mbits >> 23) - 127 - 2 + ((mbits & 0x7FFFFFu) > 0x400000u ? 1 : 0);
}

// e8m0 byte of 2^e as the cast of the fp32 value gives it (2^-128, a subnormal, lands on byte 0)
__device__ __forceinline__ uint8_t fp4_scale_byte(int e) { return (uint8_t)(e < -127 ? 0 : e + 127); }

__device__ __forceinline__ uint32_t quad_max_u32(uint32_t v)
{
    uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);     // quad_perm [1,0,3,2]
    v = v > o ? v : o;
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);              // quad_perm [2,3,0,1]
    return v > o ? v : o;
}

// literal arithmetic for one lane's 8 values, out of line (arguments in registers): y = x / s, software rounding
__device__ __noinline__ uint32_t fp4_slow8(float v0, float v1, float v2, float v3, float v4, float v5, float v6, float v7,
                                           float s)
{
    return sw_f32_to_e2m1_half_down(v0 / s) | sw_f32_to_e2m1_half_down(v1 / s) << 4 |
           sw_f32_to_e2m1_half_down(v2 / s) << 8 | sw_f32_to_e2m1_half_down(v3 / s) << 12 |
           sw_f32_to_e2m1_half_down(v4 / s) << 16 | sw_f32_to_e2m1_half_down(v5 / s) << 20 |
           sw_f32_to_e2m1_half_down(v6 / s) << 24 | sw_f32_to_e2m1_half_down(v7 / s) << 28;
}

template <bool IS_BF16, int PASSES>
__global__ __launch_bounds__(256) void quant_fp4_row32(const void *__restrict__ xin, int64_t chunks,
                                                       uint32_t *__restrict__ packed, uint8_t *__restrict__ scale_out,
                                                       int32_t *nan_count)
{
    const int t = threadIdx.x;
    // all loads of the workgroup first: the branches below would otherwise keep them one pass apart
    u32x4 w0[PASSES], w1[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const int64_t c = ((int64_t)blockIdx.x * PASSES + p) * 256 + t;
        const int64_t cc = c < chunks ? c : chunks - 1;
        if (IS_BF16) {
            w0[p] = __builtin_nontemporal_load((const u32x4 *)xin + cc);
        } else {
            w0[p] = __builtin_nontemporal_load((const u32x4 *)xin + 2 * cc);
            w1[p] = __builtin_nontemporal_load((const u32x4 *)xin + 2 * cc + 1);
        }
    }
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const int64_t c = ((int64_t)blockIdx.x * PASSES + p) * 256 + t;       // chunk of 8 values
        const bool live = c < chunks;
        float v[8];
        if (IS_BF16) {
#pragma unroll
            for (int j = 0; j < 4; ++j) { v[2 * j] = u2f(w0[p][j] << 16); v[2 * j + 1] = u2f(w0[p][j] & 0xFFFF0000u); }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) { v[j] = u2f(w0[p][j]); v[4 + j] = u2f(w1[p][j]); }
        }
        uint32_t m = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) { const uint32_t a = f2u(v[j]) & 0x7FFFFFFFu; m = a > m ? a : m; }
        m = quad_max_u32(m);
        uint32_t out;
        uint8_t sbyte;
        if (m >= 0x7F800000u) {
            // inf or NaN in the block (the reference asserts there is no NaN; inf is not pinned): literal arithmetic
            if (nan_count && live) {
                int n = 0;
#pragma unroll
                for (int j = 0; j < 8; ++j) n += v[j] != v[j];
                if (n) atomicAdd(nan_count, n);
            }
            sbyte = 0xFFu;
            out = fp4_slow8(v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], m > 0x7F800000u ? u2f(0x7FC00000u) : u2f(0x7F800000u));
        } else {
            const int e = fp4_scale_exp(m);
            sbyte = fp4_scale_byte(e);
            if (e < -120) {
                out = fp4_slow8(v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], ldexpf(1.0f, e));
            } else {
                const uint32_t eb = (uint32_t)e << 23;
                const uint32_t t0 = 0x3F400000u + eb, t1 = 0x3FE00000u + eb, t2 = 0x40600000u + eb;   // 0.75, 1.75, 3.5 times 2^e
                const float s = u2f((uint32_t)(e + 127) << 23);
                out = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    uint32_t b0 = f2u(v[2 * j]), b1 = f2u(v[2 * j + 1]);
                    const uint32_t a0 = b0 & 0x7FFFFFFFu, a1 = b1 & 0x7FFFFFFFu;
                    b0 -= (a0 == t0) | (a0 == t1) | (a0 == t2);
                    b1 -= (a1 == t0) | (a1 == t1) | (a1 == t2);
                    if (j == 0) out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, u2f(b0), u2f(b1), s, 0);
                    if (j == 1) out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, u2f(b0), u2f(b1), s, 1);
                    if (j == 2) out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, u2f(b0), u2f(b1), s, 2);
                    if (j == 3) out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, u2f(b0), u2f(b1), s, 3);
                }
            }
        }
        if (live) {
            packed[c] = out;
            if ((t & 3) == 0) scale_out[c >> 2] = sbyte;
        }
    }
}

// One workgroup per block; bn even so that both nibbles of a byte belong to one block.
__global__ __launch_bounds__(256) void quant_fp4_generic(const void *__restrict__ xin, int is_bf16, int64_t cols, int bm,
                                                         int bn, int64_t blocks_c, uint8_t *__restrict__ packed,
                                                         uint8_t *__restrict__ scale_out, int32_t *nan_count)
{
    __shared__ uint32_t wave_amax[4];
    const int64_t blk = blockIdx.x;
    const int64_t br = blk / blocks_c, bc = blk - br * blocks_c;
    const int t = threadIdx.x;
    const int n = bm * bn;
    auto load = [&](int idx) -> float {
        const int i = idx / bn, j = idx - i * bn;
        const int64_t off = (br * bm + i) * cols + bc * bn + j;
        return is_bf16 ? u2f((uint32_t)((const uint16_t *)xin)[off] << 16) : ((const float *)xin)[off];
    };
    uint32_t mbits = 0;
    int nans = 0;
    for (int idx = t; idx < n; idx += 256) {
        const float v = load(idx);
        nans += v != v;
        const uint32_t a = f2u(v) & 0x7FFFFFFFu;
        mbits = a > mbits ? a : mbits;
    }
    if (nans && nan_count) atomicAdd(nan_count, nans);
    mbits = wave_max_u32(mbits);
    if ((t & 63) == 0) wave_amax[t >> 6] = mbits;
    __syncthreads();
    {
        uint32_t a = wave_amax[0], b = wave_amax[1], c = wave_amax[2], d = wave_amax[3];
        a = a > b ? a : b; c = c > d ? c : d; mbits = a > c ? a : c;
    }
    float s;
    uint8_t sbyte;
    if (mbits >= 0x7F800000u) {
        s = u2f(mbits > 0x7F800000u ? 0x7FC00000u : 0x7F800000u);
        sbyte = 0xFFu;
    } else {
        const int e = fp4_scale_exp(mbits);
        s = ldexpf(1.0f, e);
        sbyte = fp4_scale_byte(e);
    }
    if (t == 0) scale_out[blk] = sbyte;
    for (int pr = t; pr < n / 2; pr += 256) {
        const int idx = 2 * pr, i = idx / bn, j = idx - i * bn;
        const uint32_t lo = sw_f32_to_e2m1_half_down(load(idx) / s), hi = sw_f32_to_e2m1_half_down(load(idx + 1) / s);
        packed[((br * bm + i) * cols + bc * bn + j) >> 1] = (uint8_t)(lo | (hi << 4));
    }
}

}  // namespace

extern "C" int lp_quant_fp4_block(const void *x, int x_dtype, int64_t rows, int64_t cols, int bm, int bn, void *packed_out,
                                  void *scale_out, int32_t *nan_count, lp_stream_t stream)
{
    LP_REQUIRE(x_dtype == LP_F32 || x_dtype == LP_BF16, "lp_quant_fp4_block: x_dtype must be LP_F32 or LP_BF16");
    LP_REQUIRE(rows >= 0 && cols >= 0 && bm > 0 && bn > 0, "lp_quant_fp4_block: bad shape");
    LP_REQUIRE(rows % bm == 0 && cols % bn == 0, "lp_quant_fp4_block: shape (%lld, %lld) not divisible by block (%d, %d)",
               (long long)rows, (long long)cols, bm, bn);
    LP_REQUIRE(cols % 2 == 0, "lp_quant_fp4_block: FP4 packing requires an even number of columns (got %lld)", (long long)cols);
    if (rows == 0 || cols == 0) return LP_OK;
    LP_REQUIRE(x && packed_out && scale_out, "lp_quant_fp4_block: null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (bm == 1 && bn == 32 && (uintptr_t)x % 16 == 0 && (uintptr_t)packed_out % 4 == 0) {
        constexpr int PASSES = 4;
        const int64_t chunks = rows * cols / 8;
        const int64_t wgs = (chunks + 256 * PASSES - 1) / (256 * PASSES);
        LP_REQUIRE(wgs <= 0x7FFFFFFF, "lp_quant_fp4_block: tensor too large");
        if (x_dtype == LP_BF16)
            hipLaunchKernelGGL((quant_fp4_row32<true, PASSES>), dim3((unsigned)wgs), dim3(256), 0, st, x, chunks,
                               (uint32_t *)packed_out, (uint8_t *)scale_out, nan_count);
        else
            hipLaunchKernelGGL((quant_fp4_row32<false, PASSES>), dim3((unsigned)wgs), dim3(256), 0, st, x, chunks,
                               (uint32_t *)packed_out, (uint8_t *)scale_out, nan_count);
        return check_launch("lp_quant_fp4_block");
    }
    LP_REQUIRE(bn % 2 == 0, "lp_quant_fp4_block: block width must be even (got %d)", bn);
    const int64_t blocks = (rows / bm) * (cols / bn);
    LP_REQUIRE(blocks <= 0x7FFFFFFF, "lp_quant_fp4_block: too many blocks");
    hipLaunchKernelGGL(quant_fp4_generic, dim3((unsigned)blocks), dim3(256), 0, st, x, x_dtype == LP_BF16 ? 1 : 0, cols, bm, bn,
                       cols / bn, (uint8_t *)packed_out, (uint8_t *)scale_out, nan_count);
    return check_launch("lp_quant_fp4_block");
}
