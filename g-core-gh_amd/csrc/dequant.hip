// Block dequantisers for gfx950: e4m3fn codes or packed e2m1 codes times a
// per-block scale -> bf16 / fp32.  Pure streaming kernels: 8 outputs per lane
// per pass so that loads (8 or 4 bytes per lane) and stores (16 bytes per
// lane) are contiguous across the wave.
//
// Arithmetic: out = cast(fl32(fl32(code) * fl32(scale))) -- the fp32 product is
// formed and rounded first, then narrowed to bf16 with RNE (two roundings).
#include "lowp_device.h"

using namespace lowp;

namespace {

// NaN products must come out as the canonical bf16 NaN 0x7FC0 regardless of
// payload, which is what the software cast does.
__device__ __forceinline__ uint32_t pack_bf16_checked(float a, float b, bool any_nan)
{
    if (!any_nan) return pack_bf16(a, b);
    return (uint32_t)sw_f32_to_bf16(a) | ((uint32_t)sw_f32_to_bf16(b) << 16);
}

template <bool OUT_BF16>
__device__ __forceinline__ void store8(void *out, int64_t elem0, const float v[8])
{
    if (OUT_BF16) {
        bool any_nan = false;
#pragma unroll
        for (int j = 0; j < 8; ++j) any_nan |= (v[j] != v[j]);
        u32x4 o;
        o.x = pack_bf16_checked(v[0], v[1], any_nan);
        o.y = pack_bf16_checked(v[2], v[3], any_nan);
        o.z = pack_bf16_checked(v[4], v[5], any_nan);
        o.w = pack_bf16_checked(v[6], v[7], any_nan);
        __builtin_nontemporal_store(o, (u32x4 *)((uint16_t *)out + elem0));
    } else {
        u32x4 a = {f2u(v[0]), f2u(v[1]), f2u(v[2]), f2u(v[3])};
        u32x4 b = {f2u(v[4]), f2u(v[5]), f2u(v[6]), f2u(v[7])};
        __builtin_nontemporal_store(a, (u32x4 *)((float *)out + elem0));
        __builtin_nontemporal_store(b, (u32x4 *)((float *)out + elem0 + 4));
    }
}

// e4m3fn NaN codes decode through the software path (the hardware result for
// 0x7F / 0xFF is not relied upon).
__device__ __forceinline__ void decode_fp8x4(uint32_t w, float v[4])
{
    f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
    f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    v[0] = lo.x; v[1] = lo.y; v[2] = hi.x; v[3] = hi.y;
    // a byte is a NaN code iff its low 7 bits are all ones
    uint32_t t = (w & 0x7F7F7F7Fu) + 0x01010101u;
    if (t & 0x80808080u) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = sw_e4m3fn_to_f32((uint8_t)(w >> (8 * j)));
    }
}

// Chunks (8 elements) per lane: a workgroup converts 256 * PASSES consecutive chunks.  Few passes = many small
// workgroups, which the memory system likes better on large tensors (measured on [18432, 7168] FP8 -> bf16:
// 5.9 / 6.1 / 6.4 TB/s with 8 / 4 / 2 passes; packed FP4 is best at 4); small tensors are launch-bound and
// keep 8 (a quarter of the workgroups).
constexpr int kMaxPasses = 8;

// Scale index of chunk c (8 consecutive elements of one row).  With one-row blocks (bm == 1) and
// cols % bn == 0 the scale grid is just the element index divided by bn: no row / column split.
template <bool ROWSCALE>
__device__ __forceinline__ int64_t scale_index(uint32_t c, uint32_t chunks_per_row, int bm_shift, int bn_shift,
                                               uint32_t scale_cols)
{
    if (ROWSCALE) return (int64_t)(((uint64_t)c * 8u) >> bn_shift);
    const uint32_t row = c / chunks_per_row, cc = c - row * chunks_per_row;
    return (int64_t)(row >> bm_shift) * scale_cols + ((cc * 8u) >> bn_shift);
}

// FP8: each lane owns 8 consecutive codes of one row per pass.
// chunks_per_row = cols / 8; bm, bn powers of two given as shifts; bn >= 8.
// CHECKED = false: every chunk of the workgroup exists (no bounds tests at all).
template <bool OUT_BF16, bool CHECKED, bool ROWSCALE, int kPasses>
__global__ __launch_bounds__(256) void dequant_fp8_fast(const uint8_t *__restrict__ q, const void *__restrict__ scale,
                                                        int scale_dtype, uint32_t chunk0, uint32_t n_chunks,
                                                        uint32_t chunks_per_row, int bm_shift, int bn_shift,
                                                        uint32_t scale_cols, void *__restrict__ out)
{
    const uint32_t base = chunk0 + blockIdx.x * (256u * kPasses) + threadIdx.x;
    u32x2 w[kPasses];
    float s[kPasses];
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
        const uint32_t c = base + p * 256u;
        if (!CHECKED || c < n_chunks) {
            w[p] = __builtin_nontemporal_load((const u32x2 *)(q + (int64_t)c * 8));
            s[p] = load_scale(scale, scale_dtype, scale_index<ROWSCALE>(c, chunks_per_row, bm_shift, bn_shift, scale_cols));
        } else {
            w[p] = u32x2{0, 0};
            s[p] = 0.0f;
        }
    }
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
        const uint32_t c = base + p * 256u;
        float v[8];
        decode_fp8x4(w[p].x, v);
        decode_fp8x4(w[p].y, v + 4);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = v[j] * s[p];
        if (!CHECKED || c < n_chunks) store8<OUT_BF16>(out, (int64_t)c * 8, v);
    }
}

// FP4: each lane owns 4 packed bytes = 8 consecutive elements of one row.
// chunks_per_row = cols / 8 (logical columns); bn >= 8.
template <bool OUT_BF16, bool CHECKED, bool ROWSCALE, int kPasses>
__global__ __launch_bounds__(256) void dequant_fp4_fast(const uint8_t *__restrict__ packed, const void *__restrict__ scale,
                                                        int scale_dtype, uint32_t chunk0, uint32_t n_chunks,
                                                        uint32_t chunks_per_row, int bm_shift, int bn_shift,
                                                        uint32_t scale_cols, int neg_zero, void *__restrict__ out)
{
    const uint32_t base = chunk0 + blockIdx.x * (256u * kPasses) + threadIdx.x;
    uint32_t w[kPasses];
    float s[kPasses];
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
        const uint32_t c = base + p * 256u;
        if (!CHECKED || c < n_chunks) {
            w[p] = __builtin_nontemporal_load((const uint32_t *)(packed + (int64_t)c * 4));
            s[p] = load_scale(scale, scale_dtype, scale_index<ROWSCALE>(c, chunks_per_row, bm_shift, bn_shift, scale_cols));
        } else {
            w[p] = 0;
            s[p] = 0.0f;
        }
    }
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
        const uint32_t c = base + p * 256u;
        const uint32_t x = neg_zero ? w[p] : fp4_pos_zero(w[p]);
        float v[8];
        fp4_decode8(x, v);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = v[j] * s[p];
        if (!CHECKED || c < n_chunks) store8<OUT_BF16>(out, (int64_t)c * 8, v);
    }
}

// any block shape, one element per thread per step
__global__ __launch_bounds__(256) void dequant_generic(const uint8_t *__restrict__ codes, int is_fp4, int neg_zero,
                                                       const void *__restrict__ scale, int scale_dtype, int64_t rows,
                                                       int64_t cols, int bm, int bn, void *__restrict__ out, int out_bf16)
{
    const int64_t n = rows * cols;
    const int64_t scale_cols = cols / bn;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        int64_t r = i / cols, c = i - r * cols;
        float v;
        if (is_fp4) {
            uint8_t b = codes[r * (cols / 2) + c / 2];
            v = sw_e2m1_to_f32((c & 1) ? (b >> 4) : (b & 0xF), neg_zero != 0);
        } else {
            v = sw_e4m3fn_to_f32(codes[i]);
        }
        float p = v * load_scale(scale, scale_dtype, (r / bm) * scale_cols + c / bn);
        if (out_bf16) ((uint16_t *)out)[i] = sw_f32_to_bf16(p);
        else ((float *)out)[i] = p;
    }
}

inline int log2_if_pow2(int v)
{
    if (v <= 0 || (v & (v - 1))) return -1;
    int s = 0;
    while ((1 << s) < v) ++s;
    return s;
}

int dequant_common(const char *name, bool is_fp4, const void *codes, const void *scale, int scale_dtype, int64_t rows,
                   int64_t cols, int bm, int bn, int neg_zero, void *out, int out_dtype, hipStream_t st)
{
    LP_REQUIRE(is_scale_dtype(scale_dtype), "%s: bad scale_dtype %d", name, scale_dtype);
    LP_REQUIRE(out_dtype == LP_BF16 || out_dtype == LP_F32, "%s: out_dtype must be LP_BF16 or LP_F32", name);
    LP_REQUIRE(rows >= 0 && cols >= 0 && bm > 0 && bn > 0, "%s: bad shape", name);
    LP_REQUIRE(rows % bm == 0 && cols % bn == 0, "%s: shape (%lld, %lld) not divisible by scale block (%d, %d)", name,
               (long long)rows, (long long)cols, bm, bn);
    LP_REQUIRE(!is_fp4 || cols % 2 == 0, "%s: packed FP4 needs an even column count", name);
    if (rows == 0 || cols == 0) return LP_OK;
    LP_REQUIRE(codes && scale && out, "%s: null pointer", name);

    const int bm_shift = log2_if_pow2(bm), bn_shift = log2_if_pow2(bn);
    const int64_t n_chunks = rows * cols / 8;
    const bool fast = bm_shift >= 0 && bn_shift >= 3 && cols % 8 == 0 && n_chunks < 0xFFFFFFFFll - 256 * kMaxPasses &&
                      (uintptr_t)codes % 8 == 0 && (uintptr_t)out % 16 == 0;
    const bool bf = out_dtype == LP_BF16;
    if (fast) {
        // full workgroups run without bounds tests; the ragged end (< one workgroup of chunks) is a second launch
        const bool large = n_chunks >= (1ll << 23);
        const int passes = !large ? 8 : (is_fp4 ? 4 : 2);
        const uint32_t per_wg = 256 * passes;
        const uint32_t full_wgs = (uint32_t)(n_chunks / per_wg), tail0 = full_wgs * per_wg;
        const uint32_t cpr = (uint32_t)(cols / 8), sc = (uint32_t)(cols / bn);
        const bool rowscale = bm == 1;
#define LP_DQ(KERNEL, BF, CHK, RS, P, GRID, C0, ...)                                                                     \
    hipLaunchKernelGGL((KERNEL<BF, CHK, RS, P>), dim3(GRID), dim3(256), 0, st, (const uint8_t *)codes, scale, scale_dtype, \
                       (uint32_t)(C0), (uint32_t)n_chunks, cpr, bm_shift, bn_shift, sc, ##__VA_ARGS__, out)
#define LP_DQ_P(KERNEL, BF, CHK, RS, GRID, C0, ...)                                                                   \
    do {                                                                                                              \
        if (passes == 8) LP_DQ(KERNEL, BF, CHK, RS, 8, GRID, C0, ##__VA_ARGS__);                                      \
        else if (passes == 4) LP_DQ(KERNEL, BF, CHK, RS, 4, GRID, C0, ##__VA_ARGS__);                                 \
        else LP_DQ(KERNEL, BF, CHK, RS, 2, GRID, C0, ##__VA_ARGS__);                                                  \
    } while (0)
#define LP_DQ_ALL(KERNEL, ...)                                                                                        \
    do {                                                                                                              \
        for (int part = 0; part < 2; ++part) {                                                                        \
            const bool chk = part == 1;                                                                               \
            const uint32_t grid = chk ? (tail0 < n_chunks ? 1u : 0u) : full_wgs, c0 = chk ? tail0 : 0u;               \
            if (!grid) continue;                                                                                      \
            if (bf && !chk && rowscale) LP_DQ_P(KERNEL, true, false, true, grid, c0, ##__VA_ARGS__);                  \
            else if (bf && !chk) LP_DQ_P(KERNEL, true, false, false, grid, c0, ##__VA_ARGS__);                        \
            else if (bf && rowscale) LP_DQ_P(KERNEL, true, true, true, grid, c0, ##__VA_ARGS__);                      \
            else if (bf) LP_DQ_P(KERNEL, true, true, false, grid, c0, ##__VA_ARGS__);                                 \
            else if (!chk && rowscale) LP_DQ_P(KERNEL, false, false, true, grid, c0, ##__VA_ARGS__);                  \
            else if (!chk) LP_DQ_P(KERNEL, false, false, false, grid, c0, ##__VA_ARGS__);                             \
            else if (rowscale) LP_DQ_P(KERNEL, false, true, true, grid, c0, ##__VA_ARGS__);                           \
            else LP_DQ_P(KERNEL, false, true, false, grid, c0, ##__VA_ARGS__);                                        \
        }                                                                                                             \
    } while (0)
        if (is_fp4) LP_DQ_ALL(dequant_fp4_fast, neg_zero);
        else LP_DQ_ALL(dequant_fp8_fast);
#undef LP_DQ_ALL
#undef LP_DQ_P
#undef LP_DQ
    } else {
        int64_t n = rows * cols;
        unsigned wgs = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
        hipLaunchKernelGGL(dequant_generic, dim3(wgs), dim3(256), 0, st, (const uint8_t *)codes, (int)is_fp4, neg_zero, scale,
                           scale_dtype, rows, cols, bm, bn, out, (int)bf);
    }
    return check_launch(name);
}

}  // namespace

extern "C" int lp_dequant_fp8_block(const void *q, const void *scale, int scale_dtype, int64_t rows, int64_t cols,
                                    int bm, int bn, void *out, int out_dtype, lp_stream_t stream)
{
    return dequant_common("lp_dequant_fp8_block", false, q, scale, scale_dtype, rows, cols, bm, bn, 0, out, out_dtype,
                          (hipStream_t)stream);
}

extern "C" int lp_dequant_fp4_block(const void *packed, const void *scale, int scale_dtype, int64_t rows, int64_t cols,
                                    int bm, int bn, int fp4_zero, void *out, int out_dtype, lp_stream_t stream)
{
    LP_REQUIRE(fp4_zero == LP_FP4_POS_ZERO || fp4_zero == LP_FP4_NEG_ZERO, "lp_dequant_fp4_block: bad fp4_zero");
    return dequant_common("lp_dequant_fp4_block", true, packed, scale, scale_dtype, rows, cols, bm, bn,
                          fp4_zero == LP_FP4_NEG_ZERO, out, out_dtype, (hipStream_t)stream);
}
