/*
 * CPU oracle for the low-precision weight / GEMM path.  TEST INFRASTRUCTURE ONLY.
 *
 * Plain scalar C restatement of the reference's arithmetic.  Only tests, the
 * smoke check and the cpu-baseline leg of the benchmark may load this file's
 * library; the product (HIP kernels + Python wrappers) never does.
 *
 * Every function cites the reference file:line it follows.  All loops are
 * deliberately naive: one element at a time, IEEE fp32 arithmetic written out
 * with explicit intermediates (compile with -ffp-contract=off, no fast-math).
 *
 * Pinning status (what checks each function independently of its own formula):
 *   orc_f32_to_e4m3fn / orc_e4m3fn_to_f32 : torch CPU cast (library) over every
 *       fp32 bit pattern (sampled in the default suite, exhaustive on demand).
 *   orc_f32_to_bf16                      : torch CPU cast, same coverage.
 *   orc_f32_to_e8m0 / orc_e8m0_to_f32    : torch CPU cast + the reference's
 *       known-answer list tools/dsv4_quant_and_dequant/test_cuda_parity.py:70-81.
 *   orc_e2m1_value                       : 16-entry tables at
 *       tools/convert_deepseek_v4_fp4_to_bf16.py:15-18 and
 *       gpatch_v4/kernel/quantize/eager_quant_kernels.py:56-58.
 *   block quant / dequant / FP4 converts : hand-derived vectors from the
 *       reference's CPU tests, grid round-trip invariants, and equality with an
 *       independent eager-torch restatement (oracle/torch_ref.py).
 *   orc_quant_fp4_block                  : the reference's known answers
 *       (tests/test_gfused/test_eager_quantize_kernels.py:54-150), hand-made tie vectors at
 *       three scales, the closed form "smallest 2^e with 6 * 2^e >= amax", equality
 *       with the eager-torch restatement; blocks holding NaN / inf: parity unpinned.
 *   orc_pow2_exponent (libm flavour)     : equals the exact flavour for every
 *       bf16-grid amax (exhaustive test); for raw fp32 amax within a few ulp
 *       above a power of two the reference itself depends on the log2
 *       implementation of its device -- parity unpinned on that set.
 *   scale modes RCP / RCP_POW2 (act_quant)  : bit-defined in the reference (qat.py:98-113); equality with the
 *       eager-torch restatement, which the compositions the reference's tests equate it with pin
 *       (tests/test_oracle_qat.py).  The non-power-of-two quotient x / s is an fp32 division whose flavour the
 *       reference leaves to its kernel compiler: parity unpinned for scale_fmt=None beyond IEEE division.
 *   scale mode MUL_FLOOR (per_block_cast_to_fp8 of SGLang / DeepGEMM, called at
 *       sglang_weight_update_dsv4.py:205-223,309-310): the library is not in the reference tree and the repo
 *       pins no version; restated from the published function, equality with the eager-torch restatement
 *       only -- parity unpinned.
 * Restated in oracle/torch_ref.py only (eager torch, no C twin): fp4_simulate (pinned by the reference's
 * known-answer vector tests/test_gfused/test_deepseek_v4_fp4_qat.py:37-62 and its forward == export property),
 * fp8_simulate, act_quant_inplace, fp_qat_128x128 / fp4_qat_then_to_fp8 (pinned by the eager compositions the
 * reference's tests equate them with), quant_colwise_t (TransformerEngine's column-wise Float8BlockScaling
 * quantiser, restated from the recipe's definition through the pinned 1 x 128 quantiser: TE is not in the tree,
 * parity with TE unpinned).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <stdlib.h>
#include <float.h>

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ------------------------------------------------------------------ casts */

/* fp32 -> OCP e4m3fn, round-to-nearest-even, no saturation: magnitudes that
 * round past 448 become NaN (0x7F), as torch's CPU cast does.  The reference
 * always clamps to +-448 first (eager_quant_kernels.py:177) except in the
 * FP4->FP8 rebase (tools/dsv4_quant_and_dequant/kernels.py:126). */
uint8_t orc_f32_to_e4m3fn(float f)
{
    uint32_t u = f2u(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint8_t)(sign | 0x7Fu);      /* NaN */
    if (a == 0x7F800000u) return (uint8_t)(sign | 0x7Fu);     /* inf -> NaN (no inf in fn) */
    double x = (double)u2f(a);                                /* exact */
    if (x == 0.0) return sign;
    /* quantum of the target grid at this magnitude */
    int e;
    (void)frexp(x, &e);              /* x = m * 2^e, m in [0.5,1) -> exponent of x is e-1 */
    int ex = e - 1;
    if (ex < -6) ex = -6;            /* subnormal range shares the 2^-6 binade's quantum */
    double quantum = ldexp(1.0, ex - 3);
    double q = x / quantum;          /* exact: power-of-two scaling of a double */
    double fl = floor(q);
    double rem = q - fl;
    double r;
    if (rem > 0.5) r = fl + 1.0;
    else if (rem < 0.5) r = fl;
    else r = (fmod(fl, 2.0) == 0.0) ? fl : fl + 1.0;
    double y = r * quantum;          /* rounded magnitude */
    if (y > 448.0) return (uint8_t)(sign | 0x7Fu);
    if (y == 0.0) return sign;
    /* encode y */
    int ey;
    double my = frexp(y, &ey);       /* y = my * 2^ey, my in [0.5,1) */
    int e_unb = ey - 1;
    if (e_unb < -6) {
        /* subnormal: y = k * 2^-9, k in 1..7 */
        int k = (int)(y * 512.0);
        return (uint8_t)(sign | (uint8_t)k);
    }
    int mant = (int)((my * 2.0 - 1.0) * 8.0);
    return (uint8_t)(sign | (uint8_t)(((e_unb + 7) << 3) | mant));
}

float orc_e4m3fn_to_f32(uint8_t c)
{
    int sign = c & 0x80;
    int e = (c >> 3) & 0xF;
    int m = c & 7;
    float v;
    if (e == 15 && m == 7) v = NAN;
    else if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return sign ? -v : v;
}

/* fp32 -> bf16 RNE (torch: NaN -> 0x7FC0). */
uint16_t orc_f32_to_bf16(float f)
{
    uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0u;
    uint32_t lower = u & 0xFFFFu;
    uint32_t upper = u >> 16;
    if (lower > 0x8000u || (lower == 0x8000u && (upper & 1u))) upper += 1u;
    return (uint16_t)upper;
}

float orc_bf16_to_f32(uint16_t h) { return u2f(((uint32_t)h) << 16); }

/* e8m0 byte -> fp32: 2^(b-127); 0xFF is NaN; 0x00 is 2^-127 (an fp32 subnormal). */
float orc_e8m0_to_f32(uint8_t b)
{
    if (b == 0xFF) return NAN;
    if (b == 0) return u2f(0x00400000u);
    return u2f(((uint32_t)b) << 23);
}

/* fp32 -> e8m0 as torch's CPU cast does it: sign dropped, mantissa rounded to
 * nearest on its top bit with ties going up only when something below the
 * guard bit is set or the value is normal (round-half-even with the hidden bit
 * as LSB); inf/NaN -> 0xFF.  Known answers:
 * tools/dsv4_quant_and_dequant/test_cuda_parity.py:70-81. */
uint8_t orc_f32_to_e8m0(float f)
{
    uint32_t u = f2u(f);
    uint32_t e = (u >> 23) & 0xFFu;
    if (e == 0xFFu) return 0xFFu;
    uint32_t g = (u >> 22) & 1u;
    uint32_t rest = u & 0x3FFFFFu;
    uint32_t lsb = e > 0 ? 1u : 0u;
    if (g && (rest || lsb)) e += 1u;
    return (uint8_t)e;
}

/* FP4 e2m1 code point -> value.  neg_zero != 0 keeps code 8 as -0.0
 * (eager_quant_kernels.py:56-58); neg_zero == 0 maps it to +0.0
 * (tools/convert_deepseek_v4_fp4_to_bf16.py:15-18,
 *  tools/dsv4_quant_and_dequant/kernels.py:46-66). */
float orc_e2m1_value(int code, int neg_zero)
{
    static const float mag[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    float v = mag[code & 7];
    if (code & 8) {
        if ((code & 7) == 0) return neg_zero ? -0.0f : 0.0f;
        return -v;
    }
    return v;
}

/* bulk wrappers so Python can compare whole ranges against torch's casts */
void orc_bulk_f32_to_e4m3fn(const float *x, uint8_t *y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = orc_f32_to_e4m3fn(x[i]); }
void orc_bulk_e4m3fn_to_f32(const uint8_t *x, float *y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = orc_e4m3fn_to_f32(x[i]); }
void orc_bulk_f32_to_bf16(const float *x, uint16_t *y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = orc_f32_to_bf16(x[i]); }
void orc_bulk_f32_to_e8m0(const float *x, uint8_t *y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = orc_f32_to_e8m0(x[i]); }
void orc_bulk_e8m0_to_f32(const uint8_t *x, float *y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = orc_e8m0_to_f32(x[i]); }

/* ------------------------------------------------------- scale derivation */

/* ceil(log2(r)) two ways.  kind 0: libm log2f then ceilf, the literal reading
 * of eager_quant_kernels.py:169.  kind 1: exact, from the bit pattern, as the
 * reference's own fused kernel does (fused_quant_kernels.py:32-43). */
int orc_pow2_exponent(float r, int kind)
{
    if (kind == 0) return (int)ceilf(log2f(r));
    uint32_t u = f2u(r);
    int e = (int)((u >> 23) & 0xFF);
    uint32_t m = u & 0x7FFFFFu;
    if (e == 0) {                       /* subnormal: value = m * 2^-149 */
        int top = 31 - __builtin_clz(m);
        int exact = (m & (m - 1)) == 0;
        return (top - 149) + (exact ? 0 : 1);
    }
    return (e - 127) + (m ? 1 : 0);
}

enum { ORC_SCALE_POW2 = 0, ORC_SCALE_DIV = 1, ORC_SCALE_MUL = 2, ORC_SCALE_RCP = 3, ORC_SCALE_RCP_POW2 = 4, ORC_SCALE_MUL_FLOOR = 5 };
enum { ORC_ZERO_NONE = 0, ORC_ZERO_AMAX_TO_ONE = 1, ORC_ZERO_SCALE_TO_ONE = 2 };

/*
 * Block quantiser to e4m3fn.  x is fp32 [rows, cols] row-major (a bf16 input
 * is widened by the caller, which is exact).  One scale per bm x bn block.
 *
 * mode POW2 (eager_quant_kernels.py:132-181): r = max(amax, FLT_MIN)/448,
 *     s = 2^ceil(log2 r), all-zero block -> s = 1, q = cast(clamp(x / s)).
 *     scale_out holds s as fp32; *scale_e8m0 (optional) its e8m0 byte.
 * mode DIV  (tests/test_gfused/test_te_gemm_fp8.py:82-101,
 *     tests/test_gfused/test_deepseek_tilekernels_quant.py:22-58 with
 *     amax_floor = 1e-12; tests/test_gpatch_v4/test_deep_gemm_grouped_gemm_fp8.py:29-72
 *     with zero rule SCALE_TO_ONE): s = amax/448, q = cast(clamp(x / s)).
 * mode RCP / RCP_POW2 (gpatch_v4/kernel/quantize/qat.py:116-223, act_quant with amax_floor = 1e-4):
 *     s = max(amax, floor) * fl32(1/448), optionally rounded up to a power of two on its bits,
 *     q = cast(clamp(x / s)).
 * mode MUL  (tools/convert_fp8/qwen3_5/qwen3_mtp_fp8_postprocess.py:138-149):
 *     f = fl(fl(1/amax) * 448) (1 for a zero block), q = cast(clamp(x * f)),
 *     scale_out = fl(1/f).
 * Returns the number of NaN inputs seen (the POW2 reference asserts none).
 */
int64_t orc_quant_fp8_block(const float *x, int64_t rows, int64_t cols, int bm, int bn,
                            int mode, float amax_floor, int zero_rule, int log2_kind,
                            uint8_t *q, float *scale_out, uint8_t *scale_e8m0)
{
    int64_t nbr = rows / bm, nbc = cols / bn, nan_count = 0;
    for (int64_t br = 0; br < nbr; ++br) {
        for (int64_t bc = 0; bc < nbc; ++bc) {
            float amax = 0.0f;
            int saw_nan = 0;
            for (int i = 0; i < bm; ++i)
                for (int j = 0; j < bn; ++j) {
                    float v = x[(br * bm + i) * cols + bc * bn + j];
                    if (v != v) { saw_nan = 1; ++nan_count; }
                    float a = fabsf(v);
                    if (a > amax) amax = a;
                }
            if (saw_nan) amax = NAN;
            float s = 1.0f, f = 1.0f;
            if (mode == ORC_SCALE_POW2) {
                /* amax_floor > 0: the round_sf branch of tests/test_gfused/test_deepseek_tilekernels_quant.py:22-58
                 * (amax.clamp(min=1e-12) first, no all-zero rule); amax_floor = 0: eager_quant_kernels.py:168-171 */
                float a = amax < amax_floor ? amax_floor : amax;
                float safe = a < FLT_MIN ? FLT_MIN : a;             /* clamp(min=tiny) */
                float r = safe / 448.0f;
                s = ldexpf(1.0f, orc_pow2_exponent(r, log2_kind));
                if (!(a > 0.0f)) s = 1.0f;                           /* where(max_abs > 0, s, 1) */
            } else if (mode == ORC_SCALE_RCP || mode == ORC_SCALE_RCP_POW2) {
                /* gpatch_v4/kernel/quantize/qat.py:155-161: amax = max(amax, floor); s = amax * fl32(1/448),
                 * or 2^ceil(log2 s) built on the bits of s (qat.py:98-113) when the scale is rounded */
                float a = amax;
                if (a < amax_floor) a = amax_floor;
                s = a * (float)(1.0 / 448.0);
                if (mode == ORC_SCALE_RCP_POW2) {
                    uint32_t b = f2u(s);
                    int e = (int)((b >> 23) & 0xFFu) - 127 + ((b & 0x7FFFFFu) ? 1 : 0);
                    s = u2f((uint32_t)(e + 127) << 23);
                }
            } else if (mode == ORC_SCALE_DIV) {
                float a = amax;
                if (a < amax_floor) a = amax_floor;                  /* clamp(min=floor); floor 0 = off */
                s = a / 448.0f;
                if (zero_rule == ORC_ZERO_SCALE_TO_ONE && s == 0.0f) s = 1.0f;
                if (zero_rule == ORC_ZERO_AMAX_TO_ONE && !(amax > 0.0f) && amax == amax) s = 1.0f;
            } else if (mode == ORC_SCALE_MUL_FLOOR) {
                /* per_block_cast_to_fp8 as published by SGLang / DeepGEMM (the library itself is not in the
                 * reference tree): amax.clamp(1e-4); x * (448.0 / amax) -> e4m3; scale amax / 448.0 */
                float a = amax;
                if (a < amax_floor) a = amax_floor;
                float rinv = 1.0f / a;
                f = rinv * 448.0f;
                s = a / 448.0f;
            } else {
                float safe = amax > 0.0f ? amax : 1.0f;              /* NaN amax also lands on 1 */
                /* the reference writes `448 / tensor`, which torch evaluates as
                 * reciprocal(tensor) * 448 (torch/_tensor.py __rdiv__): two roundings */
                float rinv = 1.0f / safe;
                f = rinv * 448.0f;
                if (!(amax > 0.0f)) f = 1.0f;
                s = 1.0f / f;
            }
            scale_out[br * nbc + bc] = s;
            if (scale_e8m0) scale_e8m0[br * nbc + bc] = orc_f32_to_e8m0(s);
            for (int i = 0; i < bm; ++i)
                for (int j = 0; j < bn; ++j) {
                    int64_t idx = (br * bm + i) * cols + bc * bn + j;
                    float v = x[idx];
                    float y = (mode == ORC_SCALE_MUL || mode == ORC_SCALE_MUL_FLOOR) ? v * f : v / s;
                    if (y > 448.0f) y = 448.0f;                      /* clamp keeps NaN */
                    if (y < -448.0f) y = -448.0f;
                    q[idx] = orc_f32_to_e4m3fn(y);
                }
        }
    }
    return nan_count;
}

/*
 * Block quantiser to packed FP4 e2m1 + e8m0 scales (eager_quant_kernels.py:63-129).
 * x is fp32 [rows, cols]; packed is [rows, cols/2] (low nibble = even column); scale_e8m0 is
 * [rows/bm, cols/bn].  Per block: r = max(amax, FLT_MIN) / 6 (an fp32 division, :105-106),
 * s = 2^ceil(log2 r) (:106-107), all-zero block -> s = 1 (:108); y = x / s (:111); the code is
 * the number of midpoints {0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0} strictly below |y| -- ties go
 * to the smaller magnitude, what torch.bucketize(right=False) does (:116-121) -- plus 8 when the
 * sign bit of y is set (-0.0 keeps its sign, :112,121).  The stored scale is the e8m0 cast of s
 * (:128); the division uses s itself.  Returns the number of NaN inputs (the reference asserts
 * there are none, :97); what a block holding NaN or inf yields is not pinned by anything.
 * Pinned by: the reference's known answers (tests/test_gfused/test_eager_quantize_kernels.py:
 * 54-150: grid round trip with +6 planted per block, zero block, signed extremes, first byte 0xE6),
 * hand-made tie vectors, and equality with the eager-torch restatement.
 */
int64_t orc_quant_fp4_block(const float *x, int64_t rows, int64_t cols, int bm, int bn, int log2_kind,
                            uint8_t *packed, uint8_t *scale_e8m0)
{
    static const float mid[7] = {0.25f, 0.75f, 1.25f, 1.75f, 2.5f, 3.5f, 5.0f};
    int64_t nbr = rows / bm, nbc = cols / bn, nan_count = 0;
    for (int64_t i = 0; i < rows * (cols / 2); ++i) packed[i] = 0;
    for (int64_t br = 0; br < nbr; ++br) {
        for (int64_t bc = 0; bc < nbc; ++bc) {
            float amax = 0.0f;
            for (int i = 0; i < bm; ++i)
                for (int j = 0; j < bn; ++j) {
                    float v = x[(br * bm + i) * cols + bc * bn + j];
                    if (v != v) ++nan_count;
                    float a = fabsf(v);
                    if (a > amax) amax = a;
                }
            float safe = amax < FLT_MIN ? FLT_MIN : amax;
            float r = safe / 6.0f;
            float s = ldexpf(1.0f, orc_pow2_exponent(r, log2_kind));
            if (!(amax > 0.0f)) s = 1.0f;
            scale_e8m0[br * nbc + bc] = orc_f32_to_e8m0(s);
            for (int i = 0; i < bm; ++i)
                for (int j = 0; j < bn; ++j) {
                    int64_t row = br * bm + i, col = bc * bn + j;
                    float y = x[row * cols + col] / s;
                    float a = fabsf(y);
                    int code = 0;
                    for (int k = 0; k < 7; ++k)
                        if (a > mid[k]) ++code;
                    if (f2u(y) >> 31) code += 8;
                    packed[row * (cols / 2) + col / 2] |= (uint8_t)(code << (4 * (col & 1)));
                }
        }
    }
    return nan_count;
}

/*
 * Block dequant (eager_quant_kernels.py:200-233; tools/convert_deepseek_v4_fp4_to_bf16.py:51-63):
 * out = fl32(fl32(code) * scale), scale already widened to fp32 by the caller
 * (from e8m0 / bf16 / fp32, all exact).  codes are e4m3fn bytes [rows, cols];
 * scale is [rows/bm, cols/bn].  out_bf16 (optional) receives the RNE bf16 of
 * the fp32 product -- two roundings, as the reference performs them.
 */
void orc_dequant_fp8_block(const uint8_t *codes, const float *scale, int64_t rows, int64_t cols,
                           int bm, int bn, float *out_f32, uint16_t *out_bf16)
{
    int64_t nbc = cols / bn;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            float p = orc_e4m3fn_to_f32(codes[r * cols + c]) * scale[(r / bm) * nbc + c / bn];
            if (out_f32) out_f32[r * cols + c] = p;
            if (out_bf16) out_bf16[r * cols + c] = orc_f32_to_bf16(p);
        }
}

/*
 * Packed FP4 (two e2m1 codes per byte, low nibble = even column) with one
 * e8m0 scale per bm x bn block of logical elements -> fp32 product and its
 * bf16 rounding.  neg_zero selects the table flavour (see orc_e2m1_value):
 *   0 -> tools/convert_deepseek_v4_fp4_to_bf16.py:24-46 (1 x 32 blocks),
 *   1 -> eager_quant_kernels.py:190-233 (any block).
 * packed is [rows, cols/2]; scale_bytes is [rows/bm, cols/bn].
 */
void orc_fp4_dequant(const uint8_t *packed, const uint8_t *scale_bytes, int64_t rows, int64_t cols,
                     int bm, int bn, int neg_zero, float *out_f32, uint16_t *out_bf16)
{
    int64_t nbc = cols / bn;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            uint8_t byte = packed[r * (cols / 2) + c / 2];
            int code = (c & 1) ? (byte >> 4) & 0xF : byte & 0xF;
            float s = orc_e8m0_to_f32(scale_bytes[(r / bm) * nbc + c / bn]);
            float p = orc_e2m1_value(code, neg_zero) * s;
            if (out_f32) out_f32[r * cols + c] = p;
            if (out_bf16) out_bf16[r * cols + c] = orc_f32_to_bf16(p);
        }
}

/*
 * Lossless FP4 -> e4m3fn rebase with a 128 x 128 outer scale
 * (tools/dsv4_quant_and_dequant/kernels.py:91-126).  Per tile: S = max of the
 * 128 x 4 per-32 scales, outer = S / 64, element = table(code) * (s / outer),
 * cast to e4m3fn WITHOUT a clamp.  outer_f32 gets the e8m0-rounded outer scale
 * widened to fp32 (official_expert_to_sgl, kernels.py:129-133); outer_e8m0 the byte.
 */
void orc_fp4_to_e4m3_rebase(const uint8_t *packed, const uint8_t *scale_bytes, int64_t rows, int64_t cols,
                            uint8_t *q, float *outer_f32, uint8_t *outer_e8m0)
{
    int64_t nbr = rows / 128, nbc = cols / 128, nsc = cols / 32;
    for (int64_t br = 0; br < nbr; ++br)
        for (int64_t bc = 0; bc < nbc; ++bc) {
            float smax = -INFINITY;
            int nan = 0;
            for (int i = 0; i < 128; ++i)
                for (int g = 0; g < 4; ++g) {
                    float s = orc_e8m0_to_f32(scale_bytes[(br * 128 + i) * nsc + bc * 4 + g]);
                    if (s != s) nan = 1;
                    if (s > smax) smax = s;
                }
            if (nan) smax = NAN;
            float outer = smax / 64.0f;
            uint8_t ob = orc_f32_to_e8m0(outer);
            if (outer_e8m0) outer_e8m0[br * nbc + bc] = ob;
            if (outer_f32) outer_f32[br * nbc + bc] = orc_e8m0_to_f32(ob);
            for (int i = 0; i < 128; ++i)
                for (int j = 0; j < 128; ++j) {
                    int64_t r = br * 128 + i, c = bc * 128 + j;
                    uint8_t byte = packed[r * (cols / 2) + c / 2];
                    int code = (c & 1) ? (byte >> 4) & 0xF : byte & 0xF;
                    float s = orc_e8m0_to_f32(scale_bytes[r * nsc + c / 32]);
                    float offset = s / outer;
                    q[r * cols + c] = orc_f32_to_e4m3fn(orc_e2m1_value(code, 0) * offset);
                }
        }
}

/*
 * Block-scaled FP8 GEMM reference (gfused/mygemm_fp8.py:44-97 and the numeric
 * references tests/test_gfused/test_my_gemm_fp8.py:176-186,
 * tests/test_gpatch_v4/test_deep_gemm_grouped_gemm_fp8.py:75-89): dequantise
 * both operands, contract in double, return fp32.  Aq [M,K], As [M,K/128],
 * Bq [N,K], Bs [N/128,K/128] (fp32 scales).  Small shapes only.
 */
void orc_gemm_fp8_block(const uint8_t *Aq, const float *As, const uint8_t *Bq, const float *Bs,
                        int64_t M, int64_t N, int64_t K, float *C)
{
    int64_t kb = K / 128;
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k) {
                double a = (double)orc_e4m3fn_to_f32(Aq[i * K + k]) * (double)As[i * kb + k / 128];
                double b = (double)orc_e4m3fn_to_f32(Bq[j * K + k]) * (double)Bs[(j / 128) * kb + k / 128];
                acc += a * b;
            }
            C[i * N + j] = (float)acc;
        }
}
