// Fused quantise-dequantise kernels of the QAT / weight-export path for gfx950.
//
//   qdq_tile128   : bf16 [M, N] -> e4m3 with one power-of-two scale per 128 x 128 tile -> bf16, in one pass
//                   (the tile is read once and stays in registers between the amax reduction and the store).
//   fp4_qat_fp8   : fp32 [M, N] -> e2m1 with a 1 x 32 power-of-two scale -> rebased to e4m3 with one e8m0 scale per
//                   128 x 128 tile.  The e2m1 codes stay in registers as packed nibbles (8 per lane and pass);
//                   the hardware encodes (v_cvt_scalef32_pk_fp4_f32, ties fixed up as in quant_fp4.hip) and
//                   decodes them straight into the rebased scale (v_cvt_scalef32_pk_f32_fp4 with scale
//                   2^(e_group - e_tile)), so the rebase costs one conversion per two values.
//   fp4_qdq_row32 : bf16 -> e2m1 with a 1 x 32 power-of-two scale -> bf16 (the FP4 fake-quantiser of training), flat over
//                   the tensor: a group is 32 consecutive values = 4 lanes.
//   act_qdq_group : bf16 -> e4m3 with a 1 x g scale -> bf16 (the activation / KV fake-quantiser), same flat layout,
//                   g / 8 lanes per group; a second flavour reproduces the in-place branch of the activation
//                   quantiser, which rounds the quotient to bf16 instead of e4m3.
// Scales are defined on bits in the reference (exponent field - 127, + 1 when a mantissa bit is set; 2^e rebuilt
// from bits) and are computed the same way here.
#include "lowp_device.h"

using namespace lowp;

namespace {

__device__ __forceinline__ int log2_ceil_bits(float x)
{
    const uint32_t b = f2u(x);
    return (int)((b >> 23) & 0xFFu) - 127 + ((b & 0x7FFFFFu) ? 1 : 0);
}

__device__ __forceinline__ float pow2_bits(int e) { return u2f((uint32_t)(e + 127) << 23); }

__device__ __forceinline__ uint32_t quad_max_u32(uint32_t v)
{
    uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);     // quad_perm [1,0,3,2]
    v = v > o ? v : o;
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);              // quad_perm [2,3,0,1]
    return v > o ? v : o;
}

// ------------------------------------------------------------------ bf16 -> e4m3 (128 x 128, 2^e) -> bf16
__global__ __launch_bounds__(256) void qdq_tile128(const uint16_t *__restrict__ x, int64_t cols, int64_t tiles_c,
                                                   uint16_t *__restrict__ out)
{
    __shared__ uint32_t wave_amax[4];
    const int64_t tile = blockIdx.x;
    const int64_t tr = tile / tiles_c, tc = tile - tr * tiles_c;
    const int t = threadIdx.x;
    const int64_t row0 = tr * 128 + (t >> 4), col0 = tc * 128 + (t & 15) * 8;
    u32x4 w[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = __builtin_nontemporal_load((const u32x4 *)(x + (row0 + i * 16) * cols + col0));
    u16x2 m2 = {0, 0};
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) m2 = __builtin_elementwise_max(m2, __builtin_bit_cast(u16x2, w[i][j] & 0x7FFF7FFFu));
    uint32_t mbits = (uint32_t)(m2.x > m2.y ? m2.x : m2.y) << 16;
    mbits = wave_max_u32(mbits);
    if ((t & 63) == 0) wave_amax[t >> 6] = mbits;
    __syncthreads();
    {
        uint32_t a = wave_amax[0], b = wave_amax[1], c = wave_amax[2], d = wave_amax[3];
        a = a > b ? a : b; c = c > d ? c : d; mbits = a > c ? a : c;
    }
    if (mbits >= 0x7F800000u) {
        // inf or NaN in the tile: the scale is inf or NaN and every output is NaN
#pragma unroll
        for (int i = 0; i < 8; ++i)
            *(u32x4 *)(out + (row0 + i * 16) * cols + col0) = u32x4{0x7FC07FC0u, 0x7FC07FC0u, 0x7FC07FC0u, 0x7FC07FC0u};
        return;
    }
    const float amax = u2f(mbits);
    int e = 0;
    if (amax > 0.0f) e = log2_ceil_bits((amax < 1.0e-30f ? 1.0e-30f : amax) / kE4M3Max);
    const float s = pow2_bits(e);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) { v[2 * j] = u2f(w[i][j] << 16); v[2 * j + 1] = u2f(w[i][j] & 0xFFFF0000u); }
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = clamp448(ldexpf(v[j], -e));
        const uint32_t c0 = cvt4(v[0], v[1], v[2], v[3]), c1 = cvt4(v[4], v[5], v[6], v[7]);
        const f32x2 a0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)c0, false), a1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)c0, true);
        const f32x2 b0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)c1, false), b1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)c1, true);
        u32x4 o = {pack_bf16(a0.x * s, a0.y * s), pack_bf16(a1.x * s, a1.y * s), pack_bf16(b0.x * s, b0.y * s),
                   pack_bf16(b1.x * s, b1.y * s)};
        __builtin_nontemporal_store(o, (u32x4 *)(out + (row0 + i * 16) * cols + col0));
    }
}

// ------------------------------------------------------------------ fp32 -> e2m1 (1 x 32) -> e4m3 (128 x 128)
// 256 threads own one 128 x 128 tile: lane = 8 consecutive values, 16 lanes = one row, 16 rows per pass, 8 passes.
__global__ __launch_bounds__(256) void fp4_qat_fp8(const float *__restrict__ x, int64_t cols, int64_t tiles_c,
                                                   uint8_t *__restrict__ q, uint8_t *__restrict__ scale_out)
{
    __shared__ int wave_emax[4];
    const int64_t tile = blockIdx.x;
    const int64_t tr = tile / tiles_c, tc = tile - tr * tiles_c;
    const int t = threadIdx.x;
    const int64_t row0 = tr * 128 + (t >> 4), col0 = tc * 128 + (t & 15) * 8;
    u32x4 w0[8], w1[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const u32x4 *src = (const u32x4 *)(x + (row0 + i * 16) * cols + col0);
        w0[i] = __builtin_nontemporal_load(src);
        w1[i] = __builtin_nontemporal_load(src + 1);
    }
    uint32_t codes[8];
    int eg[8];
    int emax = -1000;
    bool special = false;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        uint32_t m = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t a = w0[i][j] & 0x7FFFFFFFu, b = w1[i][j] & 0x7FFFFFFFu;
            m = a > m ? a : m; m = b > m ? b : m;
        }
        m = quad_max_u32(m);                                  // 4 lanes = one group of 32
        special |= m >= 0x7F800000u;
        // group scale 2^e: amax > 0 ? max(2^ceil(log2(amax / 6)), 2^-126) : 1
        int e = 0;
        if (m != 0u) {
            e = log2_ceil_bits(u2f(m) / 6.0f);
            e = e < -126 ? -126 : e;
        }
        eg[i] = e;
        emax = e > emax ? e : emax;
        const uint32_t eb = (uint32_t)e << 23;
        const uint32_t t0 = 0x3F400000u + eb, t1 = 0x3FE00000u + eb, t2 = 0x40600000u + eb;   // 0.75, 1.75, 3.5 times 2^e
        const float s = pow2_bits(e);
        uint32_t out = 0;
        if (e < -120) {
            // the tie constants above would be subnormal: software rounding for these (never seen in practice)
#pragma unroll
            for (int j = 0; j < 8; ++j)
                out |= sw_f32_to_e2m1_half_down(u2f(j < 4 ? w0[i][j & 3] : w1[i][j & 3]) / s) << (4 * j);
        } else
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t b0 = j < 2 ? w0[i][2 * j] : w1[i][2 * j - 4], b1 = j < 2 ? w0[i][2 * j + 1] : w1[i][2 * j - 3];
            const uint32_t a0 = b0 & 0x7FFFFFFFu, a1 = b1 & 0x7FFFFFFFu;
            b0 -= (a0 == t0) | (a0 == t1) | (a0 == t2);
            b1 -= (a1 == t0) | (a1 == t1) | (a1 == t2);
            if (j == 0) out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, u2f(b0), u2f(b1), s, 0);
            if (j == 1) out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, u2f(b0), u2f(b1), s, 1);
            if (j == 2) out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, u2f(b0), u2f(b1), s, 2);
            if (j == 3) out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, u2f(b0), u2f(b1), s, 3);
        }
        codes[i] = out;
    }
    // tile scale: max(largest group scale / 64, 2^-126)
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const int o = __shfl_xor(emax, off, 64);
        emax = o > emax ? o : emax;
    }
    const bool any_special = __syncthreads_or(special ? 1 : 0) != 0;
    if ((t & 63) == 0) wave_emax[t >> 6] = emax;
    __syncthreads();
    {
        int a = wave_emax[0], b = wave_emax[1], c = wave_emax[2], d = wave_emax[3];
        a = a > b ? a : b; c = c > d ? c : d; emax = a > c ? a : c;
    }
    int eo = emax - 6;
    eo = eo < -126 ? -126 : eo;
    if (t == 0) scale_out[tile] = any_special ? 0xFFu : (uint8_t)(eo + 127);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        uint32_t lo, hi;
        if (any_special) {
            lo = hi = 0x7F7F7F7Fu;                            // inf / NaN in the tile: not pinned by anything
        } else {
            // 2^(e_group - e_tile) <= 2^6; below 2^-126 every product rounds to (signed) zero in e4m3 either way
            const float rs = pow2_bits(eg[i] - eo < -126 ? -126 : eg[i] - eo);
            float v[8];
            const uint32_t c = codes[i];
            f32x2 p;
            p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 0); v[0] = p.x * rs; v[1] = p.y * rs;
            p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 1); v[2] = p.x * rs; v[3] = p.y * rs;
            p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 2); v[4] = p.x * rs; v[5] = p.y * rs;
            p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, 1.0f, 3); v[6] = p.x * rs; v[7] = p.y * rs;
            lo = cvt4(v[0], v[1], v[2], v[3]);
            hi = cvt4(v[4], v[5], v[6], v[7]);
        }
        __builtin_nontemporal_store(u32x2{lo, hi}, (u32x2 *)(q + (row0 + i * 16) * cols + col0));
    }
}

// ------------------------------------------------------------------ bf16 -> e2m1 (1 x 32, 2^e) -> bf16
// Flat over the tensor: chunk = 8 consecutive values = one lane, 4 lanes = one group.  Each lane owns 4 chunks, one
// per pass, and loads all of them before any arithmetic.
constexpr float kInv6 = 0.16666667163372040f;                   // fl32(1 / 6)
constexpr int kQdqPasses = 4;

__device__ __forceinline__ uint32_t bf16x8_absmax_bits(const u32x4 &w)
{
    u16x2 m2 = {0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) m2 = __builtin_elementwise_max(m2, __builtin_bit_cast(u16x2, w[j] & 0x7FFF7FFFu));
    return (uint32_t)(m2.x > m2.y ? m2.x : m2.y) << 16;
}

__global__ __launch_bounds__(256) void fp4_qdq_row32(const uint16_t *__restrict__ x, int64_t nchunks, uint16_t *__restrict__ out,
                                                     uint8_t *__restrict__ scale_out)
{
    const int t = threadIdx.x;
    u32x4 w[kQdqPasses];
    int64_t chunk[kQdqPasses];
#pragma unroll
    for (int p = 0; p < kQdqPasses; ++p) {
        chunk[p] = ((int64_t)blockIdx.x * kQdqPasses + p) * 256 + t;
        // lanes past the end read the last chunk again (a whole group is either inside or outside); nothing is stored for them
        const int64_t ld = chunk[p] < nchunks ? chunk[p] : nchunks - 1;
        w[p] = __builtin_nontemporal_load((const u32x4 *)(x + ld * 8));
    }
#pragma unroll
    for (int p = 0; p < kQdqPasses; ++p) {
        const uint32_t m = quad_max_u32(bf16x8_absmax_bits(w[p]));
        u32x4 o;
        int e = 0;
        if (m >= 0x7F800000u) {
            // inf or NaN in the group: the scale is inf or NaN and so is every output (not pinned by anything)
            o = u32x4{0x7FC07FC0u, 0x7FC07FC0u, 0x7FC07FC0u, 0x7FC07FC0u};
            e = 128;
        } else {
            const float a = fmaxf(u2f(m), 0x1.8p-124f);           // 6 * 2^-126
            e = log2_ceil_bits(a * kInv6);
            const float s = pow2_bits(e);
            float v[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) { v[2 * j] = u2f(w[p][j] << 16); v[2 * j + 1] = u2f(w[p][j] & 0xFFFF0000u); }
            if (e < -120) {
                // the tie constants below would be subnormal: software rounding (never seen in practice)
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = sw_e2m1_to_f32(sw_f32_to_e2m1_half_down(v[j] / s), true) * s;
            } else {
                const uint32_t eb = (uint32_t)e << 23;
                const uint32_t t0 = 0x3F400000u + eb, t1 = 0x3FE00000u + eb, t2 = 0x40600000u + eb;   // 0.75, 1.75, 3.5 times 2^e
                uint32_t c = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    uint32_t b0 = f2u(v[2 * j]), b1 = f2u(v[2 * j + 1]);
                    const uint32_t a0 = b0 & 0x7FFFFFFFu, a1 = b1 & 0x7FFFFFFFu;
                    b0 -= (a0 == t0) | (a0 == t1) | (a0 == t2);
                    b1 -= (a1 == t0) | (a1 == t1) | (a1 == t2);
                    if (j == 0) c = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(c, u2f(b0), u2f(b1), s, 0);
                    if (j == 1) c = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(c, u2f(b0), u2f(b1), s, 1);
                    if (j == 2) c = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(c, u2f(b0), u2f(b1), s, 2);
                    if (j == 3) c = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(c, u2f(b0), u2f(b1), s, 3);
                }
                f32x2 q;
                q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, s, 0); v[0] = q.x; v[1] = q.y;
                q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, s, 1); v[2] = q.x; v[3] = q.y;
                q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, s, 2); v[4] = q.x; v[5] = q.y;
                q = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c, s, 3); v[6] = q.x; v[7] = q.y;
            }
            o = u32x4{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
        }
        if (chunk[p] < nchunks) {
            __builtin_nontemporal_store(o, (u32x4 *)(out + chunk[p] * 8));
            if (scale_out && (t & 3) == 0) scale_out[chunk[p] >> 2] = (uint8_t)(e + 127);
        }
    }
}

// ------------------------------------------------------------------ bf16 -> e4m3 (1 x g) -> bf16
// s = max(amax, 1e-4) * fl32(1/448), rounded up to a power of two on its bits when POW2.  KIND 0 is the fake-quantiser
// (quotient to e4m3, back through fp32, times s); KIND 1 is the in-place branch of the reference's activation
// quantiser, whose quotient is rounded to bf16 (its output type) and never reaches e4m3.
template <int KIND, bool POW2>
__global__ __launch_bounds__(256) void act_qdq_group(const uint16_t *__restrict__ x, int64_t nchunks, int lanes,
                                                     uint16_t *__restrict__ out, float *__restrict__ scale_out)
{
    const int t = threadIdx.x;
    u32x4 w[kQdqPasses];
    int64_t chunk[kQdqPasses];
#pragma unroll
    for (int p = 0; p < kQdqPasses; ++p) {
        chunk[p] = ((int64_t)blockIdx.x * kQdqPasses + p) * 256 + t;
        const int64_t ld = chunk[p] < nchunks ? chunk[p] : nchunks - 1;
        w[p] = __builtin_nontemporal_load((const u32x4 *)(x + ld * 8));
    }
#pragma unroll
    for (int p = 0; p < kQdqPasses; ++p) {
        uint32_t m = bf16x8_absmax_bits(w[p]);
        for (int off = lanes >> 1; off; off >>= 1) {
            const uint32_t o = (uint32_t)__shfl_xor((int)m, off, 64);
            m = o > m ? o : m;
        }
        const float a = fmaxf(u2f(m), 1.0e-4f);
        float s = a * kInv448;
        int e = 0;
        if (POW2) {
            e = log2_ceil_bits(s);
            s = pow2_bits(e);
        }
        float v[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) { v[2 * j] = u2f(w[p][j] << 16); v[2 * j + 1] = u2f(w[p][j] & 0xFFFF0000u); }
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = clamp448(POW2 ? v[j] * pow2_bits(-e) : v[j] / s);
        if (KIND == 0) {
            const uint32_t c0 = cvt4(v[0], v[1], v[2], v[3]), c1 = cvt4(v[4], v[5], v[6], v[7]);
            const f32x2 a0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)c0, false), a1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)c0, true);
            const f32x2 b0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)c1, false), b1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)c1, true);
            v[0] = a0.x; v[1] = a0.y; v[2] = a1.x; v[3] = a1.y; v[4] = b0.x; v[5] = b0.y; v[6] = b1.x; v[7] = b1.y;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t h = pack_bf16(v[2 * j], v[2 * j + 1]);
                v[2 * j] = u2f(h << 16);
                v[2 * j + 1] = u2f(h & 0xFFFF0000u);
            }
        }
        const u32x4 o = {pack_bf16(v[0] * s, v[1] * s), pack_bf16(v[2] * s, v[3] * s), pack_bf16(v[4] * s, v[5] * s),
                         pack_bf16(v[6] * s, v[7] * s)};
        if (chunk[p] < nchunks) {
            __builtin_nontemporal_store(o, (u32x4 *)(out + chunk[p] * 8));
            if (scale_out && (t & (lanes - 1)) == 0) scale_out[chunk[p] / lanes] = s;
        }
    }
}

}  // namespace

extern "C" int lp_qdq_fp8_tile128(const void *x, int64_t rows, int64_t cols, void *out, lp_stream_t stream)
{
    LP_REQUIRE(rows >= 0 && cols >= 0 && rows % 128 == 0 && cols % 128 == 0,
               "lp_qdq_fp8_tile128: shape (%lld, %lld) must be 128 x 128-aligned", (long long)rows, (long long)cols);
    if (rows == 0 || cols == 0) return LP_OK;
    LP_REQUIRE(x && out, "lp_qdq_fp8_tile128: null pointer");
    LP_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)out % 16 == 0, "lp_qdq_fp8_tile128: pointers must be 16-byte aligned");
    const int64_t tiles_c = cols / 128, tiles = (rows / 128) * tiles_c;
    LP_REQUIRE(tiles <= 0x7FFFFFFF, "lp_qdq_fp8_tile128: too many tiles");
    hipLaunchKernelGGL(qdq_tile128, dim3((unsigned)tiles), dim3(256), 0, (hipStream_t)stream, (const uint16_t *)x, cols, tiles_c,
                       (uint16_t *)out);
    return check_launch("lp_qdq_fp8_tile128");
}

extern "C" int lp_fp4_qat_to_fp8(const void *x, int64_t rows, int64_t cols, void *q_out, void *scale_out, lp_stream_t stream)
{
    LP_REQUIRE(rows >= 0 && cols >= 0 && rows % 128 == 0 && cols % 128 == 0,
               "lp_fp4_qat_to_fp8: shape (%lld, %lld) must be 128 x 128-aligned", (long long)rows, (long long)cols);
    if (rows == 0 || cols == 0) return LP_OK;
    LP_REQUIRE(x && q_out && scale_out, "lp_fp4_qat_to_fp8: null pointer");
    LP_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)q_out % 8 == 0, "lp_fp4_qat_to_fp8: pointers must be 16 / 8-byte aligned");
    const int64_t tiles_c = cols / 128, tiles = (rows / 128) * tiles_c;
    LP_REQUIRE(tiles <= 0x7FFFFFFF, "lp_fp4_qat_to_fp8: too many tiles");
    hipLaunchKernelGGL(fp4_qat_fp8, dim3((unsigned)tiles), dim3(256), 0, (hipStream_t)stream, (const float *)x, cols, tiles_c,
                       (uint8_t *)q_out, (uint8_t *)scale_out);
    return check_launch("lp_fp4_qat_to_fp8");
}

extern "C" int lp_fp4_qdq_row32(const void *x, int64_t n, void *out, void *scale_out, lp_stream_t stream)
{
    LP_REQUIRE(n >= 0 && n % 32 == 0, "lp_fp4_qdq_row32: element count %lld must be a multiple of 32", (long long)n);
    if (n == 0) return LP_OK;
    LP_REQUIRE(x && out, "lp_fp4_qdq_row32: null pointer");
    LP_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)out % 16 == 0, "lp_fp4_qdq_row32: pointers must be 16-byte aligned");
    const int64_t nchunks = n / 8, blocks = (nchunks + 256 * kQdqPasses - 1) / (256 * kQdqPasses);
    LP_REQUIRE(blocks <= 0x7FFFFFFF, "lp_fp4_qdq_row32: tensor too large");
    hipLaunchKernelGGL(fp4_qdq_row32, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const uint16_t *)x, nchunks,
                       (uint16_t *)out, (uint8_t *)scale_out);
    return check_launch("lp_fp4_qdq_row32");
}

extern "C" int lp_act_qdq_group(const void *x, int64_t n, int group, int pow2_scale, int through_bf16, void *out,
                                void *scale_out, lp_stream_t stream)
{
    LP_REQUIRE(group >= 8 && group <= 512 && (group & (group - 1)) == 0,
               "lp_act_qdq_group: group size %d must be a power of two in 8..512", group);
    LP_REQUIRE(n >= 0 && n % group == 0, "lp_act_qdq_group: element count %lld must be a multiple of the group size %d",
               (long long)n, group);
    LP_REQUIRE(through_bf16 || pow2_scale, "lp_act_qdq_group: the e4m3 flavour is built for power-of-two scales only");
    if (n == 0) return LP_OK;
    LP_REQUIRE(x && out, "lp_act_qdq_group: null pointer");
    LP_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)out % 16 == 0, "lp_act_qdq_group: pointers must be 16-byte aligned");
    const int64_t nchunks = n / 8, blocks = (nchunks + 256 * kQdqPasses - 1) / (256 * kQdqPasses);
    LP_REQUIRE(blocks <= 0x7FFFFFFF, "lp_act_qdq_group: tensor too large");
    const int lanes = group / 8;
    auto k = !through_bf16 ? act_qdq_group<0, true> : pow2_scale ? act_qdq_group<1, true> : act_qdq_group<1, false>;
    hipLaunchKernelGGL(k, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const uint16_t *)x, nchunks, lanes,
                       (uint16_t *)out, (float *)scale_out);
    return check_launch("lp_act_qdq_group");
}
