// Block quantiser to OCP e4m3fn for gfx950.
//
// Three kernels:
//   quant_tile128  : 128 x 128 blocks, one 256-thread workgroup per block.  The
//                    block is read from HBM once (128-bit loads) and stays in
//                    registers between the amax reduction and the cast.
//   quant_group128 : 1 x 128 groups (activations); 16 lanes own a group, the
//                    amax reduction stays inside a DPP row.
//   quant_generic  : any other (bm, bn); one workgroup per block, two passes.
//
// The division x / s is formed with a correctly rounded reciprocal and two
// residual corrections (lowp::div_by_recip), which yields the correctly rounded
// quotient at a fraction of the cost of the full IEEE division sequence; blocks
// whose scale lies outside 2^+-60 or that hold NaN/inf take a slow, literal path.
#include "lowp_device.h"

using namespace lowp;

namespace {

// ---------------------------------------------------------------- 128 x 128

// amax bits are compared as integers: for non-NaN values the ordering of |x|
// equals the ordering of the sign-cleared bit patterns, and any NaN sorts
// above +inf, so one integer max finds both amax and NaN/inf presence.
template <bool IS_BF16, int MODE>
__global__ __launch_bounds__(256) void quant_tile128(const void *__restrict__ xin, int64_t cols, int64_t tiles_c,
                                                     uint8_t *__restrict__ q, void *__restrict__ scale_out,
                                                     int scale_dtype, float amax_floor, int zero_rule,
                                                     int32_t *nan_count)
{
    __shared__ uint32_t wave_amax[4];
    const int64_t tile = blockIdx.x;
    const int64_t tr = tile / tiles_c, tc = tile - tr * tiles_c;
    const int t = threadIdx.x;

    constexpr int NV = IS_BF16 ? 8 : 16;        // 128-bit vectors per thread
    u32x4 w[NV];
    int64_t row0, col0;
    int row_step;
    if (IS_BF16) { row0 = tr * 128 + (t >> 4); col0 = tc * 128 + (t & 15) * 8; row_step = 16; }
    else         { row0 = tr * 128 + (t >> 5); col0 = tc * 128 + (t & 31) * 4; row_step = 8; }

    const char *xb = (const char *)xin;
    const int esz = IS_BF16 ? 2 : 4;
#pragma unroll
    for (int i = 0; i < NV; ++i)
        w[i] = __builtin_nontemporal_load((const u32x4 *)(xb + ((row0 + (int64_t)i * row_step) * cols + col0) * esz));

    uint32_t mbits;
    if (IS_BF16) {
        u16x2 m = {0, 0};
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t a = w[i][j] & 0x7FFF7FFFu;
                m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2, a));
            }
        uint32_t hi = m.x > m.y ? m.x : m.y;
        mbits = hi << 16;
    } else {
        uint32_t m = 0;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t a = w[i][j] & 0x7FFFFFFFu;
                m = a > m ? a : m;
            }
        mbits = m;
    }
    mbits = wave_max_u32(mbits);
    if ((t & 63) == 0) wave_amax[t >> 6] = mbits;
    __syncthreads();
    {
        uint32_t a = wave_amax[0], b = wave_amax[1], c = wave_amax[2], d = wave_amax[3];
        a = a > b ? a : b; c = c > d ? c : d; mbits = a > c ? a : c;
    }
    const bool special = mbits >= 0x7F800000u;       // inf or NaN somewhere in the block
    const bool has_nan = mbits > 0x7F800000u;
    const float amax = u2f(has_nan ? 0x7FC00000u : mbits);

    BlockScale bs = derive_scale<MODE>(amax, amax_floor, zero_rule);
    if (has_nan && div_like(MODE)) { bs.div = amax; bs.stored = amax; }
    if (t == 0) {
        store_scale(scale_out, scale_dtype, tile, bs.stored);
        if (has_nan && nan_count) atomicAdd(nan_count, 1);
    }

    const bool slow = special || (div_like(MODE) && !bs.fast);
    if (slow) {
        // rare: NaN/inf in the block or a scale outside 2^+-60; literal arithmetic, inputs re-read
        const float d = pow2_like(MODE) ? bs.stored : bs.div;
#pragma unroll 1
        for (int i = 0; i < NV; ++i)
            quant_slow_span<MODE>(xin, IS_BF16, (row0 + (int64_t)i * row_step) * cols + col0, IS_BF16 ? 8 : 4, d, q);
        return;
    }
    if (IS_BF16) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) { v[2 * j] = u2f(w[i][j] << 16); v[2 * j + 1] = u2f(w[i][j] & 0xFFFF0000u); }
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = clamp448(scale_fast<MODE>(v[j], bs));
            u32x2 out = {cvt4(v[0], v[1], v[2], v[3]), cvt4(v[4], v[5], v[6], v[7])};
            __builtin_nontemporal_store(out, (u32x2 *)(q + (row0 + (int64_t)i * row_step) * cols + col0));
        }
    } else {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = clamp448(scale_fast<MODE>(u2f(w[i][j]), bs));
            __builtin_nontemporal_store(cvt4(v[0], v[1], v[2], v[3]),
                                        (uint32_t *)(q + (row0 + (int64_t)i * row_step) * cols + col0));
        }
    }
}

// ------------------------------------------------------------------ 1 x 128

// One group = 128 consecutive elements of a row = 16 lanes x 8 elements.
// A 256-thread workgroup owns 16 groups per pass and PASSES passes.
// CHECKED = false: every group of the workgroup exists (no bounds tests).
template <bool IS_BF16, int MODE, int PASSES, bool CHECKED>
__global__ __launch_bounds__(256) void quant_group128(const void *__restrict__ xin, int64_t group0, int64_t n_groups,
                                                      uint8_t *__restrict__ q, void *__restrict__ scale_out,
                                                      int scale_dtype, float amax_floor, int zero_rule,
                                                      int32_t *nan_count)
{
    const int t = threadIdx.x;
    const int64_t g0 = group0 + (int64_t)blockIdx.x * (16 * PASSES) + (t >> 4);
    const int lane16 = t & 15;

    u32x4 w[PASSES][IS_BF16 ? 1 : 2];
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        int64_t g = g0 + p * 16;
        if (!CHECKED || g < n_groups) {
            if (IS_BF16) {
                w[p][0] = __builtin_nontemporal_load((const u32x4 *)((const char *)xin + (g * 128 + lane16 * 8) * 2));
            } else {
                const u32x4 *src = (const u32x4 *)((const char *)xin + (g * 128 + lane16 * 8) * 4);
                w[p][0] = __builtin_nontemporal_load(src);
                w[p][1] = __builtin_nontemporal_load(src + 1);
            }
        } else {
            w[p][0] = u32x4{0, 0, 0, 0};
            if (!IS_BF16) w[p][1] = u32x4{0, 0, 0, 0};
        }
    }

#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        int64_t g = g0 + p * 16;
        float v[8];
        uint32_t mbits = 0;
        if (IS_BF16) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t lo = w[p][0][j] << 16, hi = w[p][0][j] & 0xFFFF0000u;
                v[2 * j] = u2f(lo); v[2 * j + 1] = u2f(hi);
                uint32_t a = lo & 0x7FFFFFFFu, b = hi & 0x7FFFFFFFu;
                mbits = a > mbits ? a : mbits; mbits = b > mbits ? b : mbits;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                uint32_t u = w[p][IS_BF16 ? 0 : (j >> 2)][j & 3];
                v[j] = u2f(u);
                uint32_t a = u & 0x7FFFFFFFu;
                mbits = a > mbits ? a : mbits;
            }
        }
        mbits = row16_max_u32(mbits);
        const bool special = mbits >= 0x7F800000u;
        const bool has_nan = mbits > 0x7F800000u;
        const float amax = u2f(has_nan ? 0x7FC00000u : mbits);
        BlockScale bs = derive_scale<MODE>(amax, amax_floor, zero_rule);
        if (has_nan && div_like(MODE)) { bs.div = amax; bs.stored = amax; }
        const bool slow = special || (div_like(MODE) && !bs.fast);
        if (slow) {
            if (!CHECKED || g < n_groups)
                quant_slow_span<MODE>(xin, IS_BF16, g * 128 + lane16 * 8, 8, pow2_like(MODE) ? bs.stored : bs.div, q);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = clamp448(scale_fast<MODE>(v[j], bs));
            u32x2 out = {cvt4(v[0], v[1], v[2], v[3]), cvt4(v[4], v[5], v[6], v[7])};
            if (!CHECKED || g < n_groups) __builtin_nontemporal_store(out, (u32x2 *)(q + g * 128 + lane16 * 8));
        }
        if (!CHECKED || g < n_groups) {
            if (lane16 == 0) {
                store_scale(scale_out, scale_dtype, g, bs.stored);
                if (has_nan && nan_count) atomicAdd(nan_count, 1);
            }
        }
    }
}

// ------------------------------------------------------------------ generic

template <int MODE>
__global__ __launch_bounds__(256) void quant_generic(const void *__restrict__ xin, int is_bf16, int64_t cols,
                                                     int bm, int bn, int64_t blocks_c,
                                                     uint8_t *__restrict__ q, void *__restrict__ scale_out,
                                                     int scale_dtype, float amax_floor, int zero_rule,
                                                     int32_t *nan_count)
{
    __shared__ uint32_t wave_amax[4];
    const int64_t blk = blockIdx.x;
    const int64_t br = blk / blocks_c, bc = blk - br * blocks_c;
    const int t = threadIdx.x;
    const int n = bm * bn;
    auto load = [&](int idx) -> float {
        int i = idx / bn, j = idx - i * bn;
        int64_t off = (br * bm + i) * cols + bc * bn + j;
        return is_bf16 ? u2f((uint32_t)((const uint16_t *)xin)[off] << 16) : ((const float *)xin)[off];
    };
    uint32_t mbits = 0;
    for (int idx = t; idx < n; idx += 256) {
        uint32_t a = f2u(load(idx)) & 0x7FFFFFFFu;
        mbits = a > mbits ? a : mbits;
    }
    mbits = wave_max_u32(mbits);
    if ((t & 63) == 0) wave_amax[t >> 6] = mbits;
    __syncthreads();
    {
        uint32_t a = wave_amax[0], b = wave_amax[1], c = wave_amax[2], d = wave_amax[3];
        a = a > b ? a : b; c = c > d ? c : d; mbits = a > c ? a : c;
    }
    const bool has_nan = mbits > 0x7F800000u;
    const float amax = u2f(has_nan ? 0x7FC00000u : mbits);
    BlockScale bs = derive_scale<MODE>(amax, amax_floor, zero_rule);
    if (has_nan && div_like(MODE)) { bs.div = amax; bs.stored = amax; }
    if (t == 0) {
        store_scale(scale_out, scale_dtype, blk, bs.stored);
        if (has_nan && nan_count) atomicAdd(nan_count, 1);
    }
    for (int idx = t; idx < n; idx += 256) {
        int i = idx / bn, j = idx - i * bn;
        q[(br * bm + i) * cols + bc * bn + j] = quant_slow<MODE>(load(idx), bs);
    }
}

template <int MODE>
int launch_mode(const void *x, bool is_bf16, int64_t rows, int64_t cols, int bm, int bn, float amax_floor,
                int zero_rule, uint8_t *q, void *scale_out, int scale_dtype, int32_t *nan_count, hipStream_t st)
{
    const bool aligned16 = ((uintptr_t)x % 16 == 0) && ((uintptr_t)q % 8 == 0) &&
                           ((cols * (is_bf16 ? 2 : 4)) % 16 == 0);
    if (bm == 128 && bn == 128 && aligned16) {
        int64_t tiles_c = cols / 128, tiles = (rows / 128) * tiles_c;
        if (tiles > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_quant_fp8_block: too many tiles");
        if (is_bf16)
            hipLaunchKernelGGL((quant_tile128<true, MODE>), dim3((unsigned)tiles), dim3(256), 0, st, x, cols, tiles_c,
                               q, scale_out, scale_dtype, amax_floor, zero_rule, nan_count);
        else
            hipLaunchKernelGGL((quant_tile128<false, MODE>), dim3((unsigned)tiles), dim3(256), 0, st, x, cols, tiles_c,
                               q, scale_out, scale_dtype, amax_floor, zero_rule, nan_count);
    } else if (bm == 1 && bn == 128 && aligned16) {
        constexpr int PASSES = 4;
        const int64_t groups = rows * (cols / 128), per_wg = 16 * PASSES;
        const int64_t full = groups / per_wg, tail0 = full * per_wg;
        if (full > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_quant_fp8_block: too many groups");
        // full workgroups run without bounds tests; the ragged end is a one-workgroup launch
        if (full > 0) {
            if (is_bf16)
                hipLaunchKernelGGL((quant_group128<true, MODE, PASSES, false>), dim3((unsigned)full), dim3(256), 0, st, x,
                                   (int64_t)0, groups, q, scale_out, scale_dtype, amax_floor, zero_rule, nan_count);
            else
                hipLaunchKernelGGL((quant_group128<false, MODE, PASSES, false>), dim3((unsigned)full), dim3(256), 0, st, x,
                                   (int64_t)0, groups, q, scale_out, scale_dtype, amax_floor, zero_rule, nan_count);
        }
        if (tail0 < groups) {
            if (is_bf16)
                hipLaunchKernelGGL((quant_group128<true, MODE, PASSES, true>), dim3(1), dim3(256), 0, st, x, tail0, groups, q,
                                   scale_out, scale_dtype, amax_floor, zero_rule, nan_count);
            else
                hipLaunchKernelGGL((quant_group128<false, MODE, PASSES, true>), dim3(1), dim3(256), 0, st, x, tail0, groups, q,
                                   scale_out, scale_dtype, amax_floor, zero_rule, nan_count);
        }
    } else {
        int64_t blocks_c = cols / bn, blocks = (rows / bm) * blocks_c;
        if (blocks > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_quant_fp8_block: too many blocks");
        if ((int64_t)bm * bn > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_quant_fp8_block: block too large");
        hipLaunchKernelGGL((quant_generic<MODE>), dim3((unsigned)blocks), dim3(256), 0, st, x, (int)is_bf16, cols, bm, bn,
                           blocks_c, q, scale_out, scale_dtype, amax_floor, zero_rule, nan_count);
    }
    return check_launch("lp_quant_fp8_block");
}

}  // namespace

extern "C" int lp_quant_fp8_block(const void *x, int x_dtype, int64_t rows, int64_t cols, int bm, int bn,
                                  int scale_mode, float amax_floor, int zero_rule, void *q_out, void *scale_out,
                                  int scale_dtype, int32_t *nan_count, lp_stream_t stream)
{
    LP_REQUIRE(x_dtype == LP_BF16 || x_dtype == LP_F32, "lp_quant_fp8_block: x_dtype must be LP_BF16 or LP_F32");
    LP_REQUIRE(is_scale_dtype(scale_dtype), "lp_quant_fp8_block: bad scale_dtype %d", scale_dtype);
    LP_REQUIRE(rows >= 0 && cols >= 0 && bm > 0 && bn > 0, "lp_quant_fp8_block: bad shape");
    LP_REQUIRE(rows % bm == 0 && cols % bn == 0,
               "lp_quant_fp8_block: shape (%lld, %lld) not divisible by block (%d, %d)", (long long)rows,
               (long long)cols, bm, bn);
    LP_REQUIRE(scale_mode >= LP_SCALE_POW2 && scale_mode <= LP_SCALE_MUL_FLOOR, "lp_quant_fp8_block: bad scale_mode");
    LP_REQUIRE(zero_rule >= LP_ZERO_NONE && zero_rule <= LP_ZERO_SCALE_TO_ONE, "lp_quant_fp8_block: bad zero_rule");
    LP_REQUIRE(amax_floor >= 0.0f, "lp_quant_fp8_block: amax_floor must be >= 0");
    if (rows == 0 || cols == 0) return LP_OK;
    LP_REQUIRE(x && q_out && scale_out, "lp_quant_fp8_block: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const bool bf = x_dtype == LP_BF16;
    switch (scale_mode) {
    case LP_SCALE_POW2:
        return launch_mode<LP_SCALE_POW2>(x, bf, rows, cols, bm, bn, amax_floor, zero_rule, (uint8_t *)q_out, scale_out,
                                          scale_dtype, nan_count, st);
    case LP_SCALE_DIV:
        return launch_mode<LP_SCALE_DIV>(x, bf, rows, cols, bm, bn, amax_floor, zero_rule, (uint8_t *)q_out, scale_out,
                                         scale_dtype, nan_count, st);
    case LP_SCALE_RCP:
        return launch_mode<LP_SCALE_RCP>(x, bf, rows, cols, bm, bn, amax_floor, zero_rule, (uint8_t *)q_out, scale_out,
                                         scale_dtype, nan_count, st);
    case LP_SCALE_RCP_POW2:
        return launch_mode<LP_SCALE_RCP_POW2>(x, bf, rows, cols, bm, bn, amax_floor, zero_rule, (uint8_t *)q_out, scale_out,
                                              scale_dtype, nan_count, st);
    case LP_SCALE_MUL_FLOOR:
        return launch_mode<LP_SCALE_MUL_FLOOR>(x, bf, rows, cols, bm, bn, amax_floor, zero_rule, (uint8_t *)q_out, scale_out,
                                               scale_dtype, nan_count, st);
    default:
        return launch_mode<LP_SCALE_MUL>(x, bf, rows, cols, bm, bn, amax_floor, zero_rule, (uint8_t *)q_out, scale_out,
                                         scale_dtype, nan_count, st);
    }
}
