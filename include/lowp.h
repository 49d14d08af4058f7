/*
 * lowp -- C ABI of the MI355X (gfx950) low-precision weight / GEMM path.
 *
 * One shared library, plain pointers and sizes.  Every pointer marked "device"
 * must be device memory on the GPU that is current on the calling thread; all
 * work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the
 * default stream) and the call returns without waiting.  The caller owns and
 * allocates every buffer.  Return value: 0 on success, a negative lp_status
 * otherwise, with a message available from lp_last_error() (thread local).
 * Arguments are validated on the host before anything is launched.
 *
 * File:line citations name the reference (Tencent/G-Core-GH) interface that an
 * entry point stands in for.
 */
#ifndef LOWP_H
#define LOWP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *lp_stream_t;

enum lp_status {
    LP_OK = 0,
    LP_ERR_INVALID = -1,      /* bad shape / dtype / null pointer            */
    LP_ERR_UNSUPPORTED = -2,  /* valid request this build has no kernel for */
    LP_ERR_HIP = -3           /* the HIP runtime reported an error           */
};

enum lp_dtype {
    LP_F32 = 0,
    LP_BF16 = 1,
    LP_E8M0 = 2,   /* float8_e8m0fnu: one byte, value 2^(b-127)            */
    LP_E4M3 = 3    /* float8_e4m3fn (OCP)                                   */
};

/* How the per-block scale is derived from the block's amax. */
enum lp_scale_mode {
    /* s = 2^ceil(log2(max(amax, amax_floor, FLT_MIN)/448)), q = cast(clamp(x / s)); with amax_floor = 0 an
     * all-zero block gets s = 1: gpatch_v4/kernel/quantize/eager_quant_kernels.py:132-181; with a positive
     * floor (1e-12) it is the round_sf branch of tests/test_gfused/test_deepseek_tilekernels_quant.py:22-58 */
    LP_SCALE_POW2 = 0,
    /* s = max(amax, amax_floor)/448, q = cast(clamp(x / s));
     * tests/test_gfused/test_te_gemm_fp8.py:82-101,
     * tests/test_gpatch_v4/test_deep_gemm_grouped_gemm_fp8.py:29-72 */
    LP_SCALE_DIV = 1,
    /* f = fl(fl(1/amax) * 448), q = cast(clamp(x * f)), stored scale = fl(1/f);
     * tools/convert_fp8/qwen3_5/qwen3_mtp_fp8_postprocess.py:138-149 */
    LP_SCALE_MUL = 2,
    /* s = max(amax, amax_floor) * fl32(1/448), q = cast(clamp(x / s));
     * gpatch_v4/kernel/quantize/qat.py:116-223 (act_quant, amax_floor = 1e-4) */
    LP_SCALE_RCP = 3,
    /* as LP_SCALE_RCP with s rounded up to a power of two from its bits
     * (exponent field - 127, + 1 when a mantissa bit is set); act_quant with
     * scale_fmt set: qat.py:98-113 */
    LP_SCALE_RCP_POW2 = 4,
    /* a = max(amax, amax_floor), f = fl(fl(1/a) * 448), q = cast(clamp(x * f)), stored scale = a / 448:
     * the published per_block_cast_to_fp8 of SGLang / DeepGEMM (x * (448.0 / amax) with amax clamped at
     * 1e-4; scale amax / 448), which the weight-update path calls
     * (gpatch_v4/generation_backend/sglang_model_specific/sglang_weight_update_dsv4.py:205-223,309-310) */
    LP_SCALE_MUL_FLOOR = 5
};

enum lp_zero_rule {
    LP_ZERO_NONE = 0,          /* no special case                              */
    LP_ZERO_AMAX_TO_ONE = 1,   /* amax == 0      -> scale 1                    */
    LP_ZERO_SCALE_TO_ONE = 2   /* computed s == 0 -> scale 1                   */
};

/* Table flavour for FP4 code 8: */
enum lp_fp4_zero {
    LP_FP4_POS_ZERO = 0,  /* +0.0: tools/convert_deepseek_v4_fp4_to_bf16.py:15-18,
                             tools/dsv4_quant_and_dequant/kernels.py:46-66      */
    LP_FP4_NEG_ZERO = 1   /* -0.0: gpatch_v4/kernel/quantize/eager_quant_kernels.py:56-58 */
};

/* pad_rows of lp_quant_fp8_colwise_t: besides 128, 256 and 512 */
enum lp_pad_rows {
    LP_PAD_MIXED = 0      /* experts of at most 256 rows to multiples of 128, the others to multiples of 512 */
};

int lp_version(void);
const char *lp_last_error(void);

/*
 * Block quantiser to e4m3fn.  x: device, [rows, cols] row-major, LP_BF16 or
 * LP_F32 (leading dims of the reference's [..., M, N] are folded into rows).
 * One scale per bm x bn block; rows % bm == 0, cols % bn == 0.
 * q_out: device u8 [rows, cols].  scale_out: device [rows/bm, cols/bn] of
 * scale_dtype (LP_F32, LP_BF16 or LP_E8M0).  nan_count: optional device
 * int32 that is incremented once per block that holds a NaN (caller zeroes it).
 * Replaces quant_fp8_e4m3_scale_e8m0 (eager_quant_kernels.py:132-181),
 * quantize_fp8_blockwise (qwen3_mtp_fp8_postprocess.py:102-151) and the
 * 1 x 128 / 128 x 128 fp32-scale quantisers used around the GEMM
 * (test_te_gemm_fp8.py:82-101, test_deep_gemm_grouped_gemm_fp8.py:29-72).
 */
int lp_quant_fp8_block(const void *x, int x_dtype, int64_t rows, int64_t cols, int bm, int bn,
                       int scale_mode, float amax_floor, int zero_rule,
                       void *q_out, void *scale_out, int scale_dtype,
                       int32_t *nan_count, lp_stream_t stream);

/*
 * Block dequantiser: out = cast(fl32(fl32(code) * fl32(scale))).
 * q: device [rows, cols] e4m3fn bytes (q_dtype LP_E4M3).  scale: device
 * [rows/bm, cols/bn] of scale_dtype.  out: device [rows, cols], LP_BF16 or LP_F32.
 * Replaces the FP8 branch of dequant_fp4_e2m1_fp8_scale_e8m0_packed
 * (eager_quant_kernels.py:200-233) and cast_e4m3fn_to_bf16
 * (tools/convert_deepseek_v4_fp4_to_bf16.py:51-63).
 */
int lp_dequant_fp8_block(const void *q, const void *scale, int scale_dtype,
                         int64_t rows, int64_t cols, int bm, int bn,
                         void *out, int out_dtype, lp_stream_t stream);

/*
 * Packed FP4 (e2m1, two codes per byte, low nibble = even column) with one
 * scale per bm x bn block of logical elements -> bf16 / fp32.
 * packed: device u8 [rows, cols/2]; scale: device [rows/bm, cols/bn] of
 * scale_dtype; out: device [rows, cols].
 * Replaces cast_e2m1fn_to_bf16 (tools/convert_deepseek_v4_fp4_to_bf16.py:24-46;
 * bm=1, bn=32, LP_E8M0, LP_FP4_POS_ZERO) and the FP4 branch of
 * dequant_fp4_e2m1_fp8_scale_e8m0_packed (eager_quant_kernels.py:190-233;
 * LP_FP4_NEG_ZERO).
 */
int lp_dequant_fp4_block(const void *packed, const void *scale, int scale_dtype,
                         int64_t rows, int64_t cols, int bm, int bn, int fp4_zero,
                         void *out, int out_dtype, lp_stream_t stream);

/*
 * Lossless FP4 (1 x 32 e8m0 scales) -> e4m3fn with one 128 x 128 outer scale
 * = (max e8m0 scale of the tile) / 64; no clamp.
 * packed: device u8 [rows, cols/2]; scale: device u8 (e8m0) [rows, cols/32];
 * q_out: device u8 [rows, cols]; scale_out: device [rows/128, cols/128] of
 * scale_dtype (LP_E8M0 or LP_F32).
 * Replaces cast_e2m1fn_to_e4m3fn / official_expert_to_sgl
 * (tools/dsv4_quant_and_dequant/kernels.py:91-133).
 */
int lp_fp4_to_fp8_rebase(const void *packed, const void *scale, int64_t rows, int64_t cols,
                         void *q_out, void *scale_out, int scale_dtype, lp_stream_t stream);

/*
 * Fused FP4 (1 x 32 e8m0) -> bf16 -> e4m3fn with a 128 x 128 fp32 scale: the
 * result is byte-identical to lp_dequant_fp4_block (bf16, LP_FP4_POS_ZERO)
 * followed by lp_quant_fp8_block on 128 x 128 blocks with the given scale
 * mode, without the bf16 tensor touching HBM unless bf16_out is non-NULL.
 * Stands in for running tools/convert_deepseek_v4_fp4_to_bf16.py:24-46 and then
 * the tools/convert_fp8 quantiser.
 */
int lp_fp4_to_fp8_amax(const void *packed, const void *scale, int64_t rows, int64_t cols,
                       int scale_mode, float amax_floor, int zero_rule,
                       void *q_out, void *scale_out, int scale_dtype, void *bf16_out,
                       lp_stream_t stream);

/*
 * Block quantisation to packed FP4 (e2m1) with e8m0 block scales.
 * x: device [rows, cols] of x_dtype (LP_F32 or LP_BF16); packed_out: device
 * [rows, cols/2] bytes, low nibble = even column; scale_out: device
 * [rows/bm, cols/bn] e8m0 bytes.  scale = 2^ceil(log2(amax/6)) (1 for an all-zero
 * block), code = nearest e2m1 value of x/scale with ties to the smaller
 * magnitude, sign bit kept (also for -0).  cols even; the fast path is
 * bm = 1, bn = 32, other shapes need an even bn.  nan_count: optional device
 * int32 that is incremented by the number of NaN inputs (caller zeroes it; the
 * reference asserts the input holds none).
 * Replaces quant_fp4_e2m1_scale_e8m0_packed
 * (gpatch_v4/kernel/quantize/eager_quant_kernels.py:63-129); with
 * lp_dequant_fp8_block in front it is sgl_expert_to_official
 * (tools/dsv4_quant_and_dequant/kernels.py:136-140).
 */
int lp_quant_fp4_block(const void *x, int x_dtype, int64_t rows, int64_t cols, int bm, int bn,
                       void *packed_out, void *scale_out, int32_t *nan_count, lp_stream_t stream);

/*
 * bf16 [rows, cols] -> e4m3fn with one power-of-two scale per 128 x 128 tile -> bf16, fused:
 * s = 2^ceil(log2(max(amax, 1e-30) / 448)) from the bits of the quotient (1 for an
 * all-zero tile), out = bf16(fp32(e4m3(clamp(x / s))) * s).  rows, cols multiples of 128.
 * Replaces fp_qat_128x128 (gpatch_v4/kernel/quantize/fused_quant_kernels.py:277-403).
 */
int lp_qdq_fp8_tile128(const void *x, int64_t rows, int64_t cols, void *out, lp_stream_t stream);

/*
 * fp32 [rows, cols] -> e2m1 with one scale max(2^ceil(log2(amax / 6)), 2^-126) per 1 x 32 group
 * (1 for an all-zero group; ties to the smaller magnitude, -0.0 kept) -> rebased to e4m3fn with
 * one e8m0 scale max(largest group scale / 64, 2^-126) per 128 x 128 tile.  q_out: [rows, cols]
 * bytes; scale_out: [rows/128, cols/128] e8m0 bytes.  rows, cols multiples of 128.
 * Replaces fp4_qat_then_to_fp8 (gpatch_v4/kernel/quantize/fused_quant_kernels.py:102-274).
 */
int lp_fp4_qat_to_fp8(const void *x, int64_t rows, int64_t cols, void *q_out, void *scale_out, lp_stream_t stream);

/*
 * bf16 -> e2m1 with one power-of-two scale per 32 consecutive values -> bf16, fused.  n values
 * (n % 32 == 0; a [.., N] tensor with N % 32 == 0 is passed flat):
 * s = 2^e, e = ceil(log2(max(amax, 6 * 2^-126) * fl32(1/6))) taken from the bits of the product;
 * out = bf16(e2m1(clamp(x / s, +-6)) * s), ties of the e2m1 rounding to the smaller magnitude,
 * -0.0 kept.  scale_out (optional, may be NULL): n / 32 e8m0 bytes (e + 127).
 * Replaces _fp4_quant_kernel / _fp4_simulate (gpatch_v4/kernel/quantize/qat.py:226-279, 350-366).
 */
int lp_fp4_qdq_row32(const void *x, int64_t n, void *out, void *scale_out, lp_stream_t stream);

/*
 * bf16 -> 8-bit grid with one scale per `group` consecutive values -> bf16, fused.  n values
 * (n % group == 0, group a power of two in 8..512):
 * s = max(amax, 1e-4) * fl32(1/448), rounded up to a power of two on its bits when pow2_scale.
 *   through_bf16 == 0: out = bf16(fp32(e4m3(clamp(x / s, +-448))) * s)    (pow2_scale must be 1)
 *     = act_quant(x, group, "ue8m0") followed by per_token_cast_back, i.e. _fp8_simulate
 *     (gpatch_v4/kernel/quantize/qat.py:286-301).
 *   through_bf16 == 1: out = bf16(fp32(bf16(clamp(x / s, +-448))) * s), what act_quant(inplace=True)
 *     computes (qat.py:131,163-175: the branch casts the quotient to its output type, bf16).
 * scale_out (optional, may be NULL): n / group fp32 scales.
 */
int lp_act_qdq_group(const void *x, int64_t n, int group, int pow2_scale, int through_bf16, void *out,
                     void *scale_out, lp_stream_t stream);

/*
 * Block-scaled FP8 GEMM: C[i,j] = cast(sum_kb (sum_{k in kb} Aq[i,k] Bq[j,k]) * As[i,kb] * Bs[j/128,kb]).
 * Aq: device e4m3fn [M,K]; As: device [M,K/128]; Bq: device e4m3fn [N,K];
 * Bs: device [N/128,K/128]; scales of scale_dtype (LP_F32 or LP_E8M0);
 * C: device [M,N] LP_BF16 or LP_F32.  K % 128 == 0, N % 128 == 0, any M.
 * workspace: optional device scratch of at least lp_gemm_workspace_bytes(M,N,K)
 * bytes (256-byte aligned); with it, problems with few output tiles split K
 * across workgroups (fixed summation order) and LP_E8M0 scales are expanded to
 * fp32 for the fastest kernels.  NULL / too small = slower paths, same results.
 * Replaces gemm_fp8_block_scaling_impl (gfused/mygemm_fp8.py:44-97).
 */
int lp_gemm_fp8_block(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype,
                      int64_t M, int64_t N, int64_t K, void *C, int out_dtype,
                      void *workspace, int64_t workspace_bytes, lp_stream_t stream);

/* Scratch bytes lp_gemm_fp8_block can use for this shape (0 = none needed). */
int64_t lp_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

/*
 * lp_gemm_fp8_block without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc): the K-split partial sums go to a buffer of
 * lp_gemm_static_scratch_bytes() = 32 MiB that is part of the library's device image (every GPU the process uses
 * holds one copy until the process ends).  Same kernels, same summation order and therefore the same bits as
 * lp_gemm_fp8_block with a workspace of lp_gemm_workspace_bytes(M, N, K).  The call allocates and frees nothing.
 * A shape whose K split needed more than the buffer would be rejected with LP_ERR_INVALID and a message naming both
 * sizes; the K split is taken for at most 32 tiles of 128 x 128 in at most 16 K ranges, which is 32 MiB, so no shape
 * is turned away today (shapes that need no scratch always pass).  All calls on one GPU share that GPU's buffer: calls that can
 * overlap on one GPU (different streams, or threads) race on it -- serialise them or use lp_gemm_fp8_block.
 * Nothing has to be cleared between calls: every partial tile is written before it is read.
 * No counterpart in the reference (its GEMM is a JIT kernel without scratch, gfused/mygemm_fp8.py:44-97).
 */
int lp_gemm_fp8_block_static(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype,
                             int64_t M, int64_t N, int64_t K, void *C, int out_dtype, lp_stream_t stream);
int64_t lp_gemm_static_scratch_bytes(void);

/*
 * Unscaled C = A B^T with fp32 accumulation.  A [M,K], B [N,K], both of
 * in_dtype (LP_E4M3 or LP_BF16); C [M,N] of out_dtype (LP_E4M3, LP_BF16, LP_F32).
 * K must be a multiple of 128 (LP_E4M3) or 64 (LP_BF16), N a multiple of 16; M is free.
 * An LP_E4M3 result saturates at +-448 (NaN stays NaN), like the fp8 conversion
 * of the tile compiler the reference uses.
 * Replaces gemm_impl (gfused/mygemm_fp8.py:12-41).
 */
int lp_gemm_nt(const void *A, const void *B, int in_dtype, int64_t M, int64_t N, int64_t K,
               void *C, int out_dtype, lp_stream_t stream);

/*
 * Grouped block-scaled FP8 GEMM for MoE experts.  Rows of Aq are sorted by
 * expert; expert e owns rows m_offsets[e] .. m_offsets[e+1]-1 (zero rows
 * allowed).  Aq [M_total,K], As [M_total,K/128], Bq [E,N,K], Bs [E,N/128,K/128],
 * C [M_total,N].  m_offsets: device int32 [E+1], non-decreasing, m_offsets[0]=0.
 * Rows at or beyond m_offsets[E] are left untouched.
 * Replaces MyTeGroupedLinearFp8.forward (gpatch_v4/models/deepseek_v4/fp8.py:346-394)
 * and the DeepGEMM-style contiguous grouped GEMM called at
 * tests/test_gpatch_v4/test_deep_gemm_grouped_gemm_fp8.py:106-109.
 */
int lp_gemm_fp8_grouped(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype,
                        const int32_t *m_offsets, int E, int64_t M_total, int64_t N, int64_t K,
                        void *C, int out_dtype, lp_stream_t stream);

/*
 * The same grouped GEMM on weights stored for the other product: C_e = A_e W_e with W [E,K,N] row-major (K = the
 * contraction) and its 128 x 128 scales Ws [E,K/128,N/128], scales e8m0 on both operands.  This is the data gradient
 * of the grouped linear, dX_e = dY_e W_e on the layer's own [out, in] weight (K = out features, N = in features),
 * without a transposed copy of the weights: the matrix cores' operand is turned while it is read out of LDS.
 * Aq [M_total,K], As [M_total,K/128] (dY quantised 1 x 128 along K), C [M_total,N].  Needs N % 512 == 0, K % 512 == 0,
 * Ws 4-byte aligned, E <= 512; LP_ERR_UNSUPPORTED otherwise (transpose and call lp_gemm_fp8_grouped).
 * Replaces the dgrad of _MyTeGroupedLinear.backward, general_grouped_gemm(..., layout="NN")
 * (gpatch_v4/models/deepseek_v4/fp8.py:301-313).
 */
int lp_gemm_fp8_grouped_nn(const void *Aq, const void *As, const void *Wq, const void *Ws, int scale_dtype,
                           const int32_t *m_offsets, int E, int64_t M_total, int64_t N, int64_t K, void *C,
                           int out_dtype, lp_stream_t stream);

/*
 * Block-scaled FP8 GEMM with a scale per row and 128-wide K group on BOTH operands:
 * C[m, n] = sum_kb (Aq[m, kb] . Bq[n, kb]) * As[m, kb] * Bs[n, kb], Bs [N, K/128].
 * Same shapes, dtypes and checks as lp_gemm_fp8_block otherwise.  This is the weight-gradient GEMM of
 * the grouped linear (layout "NT" over column-wise quantised operands,
 * gpatch_v4/models/deepseek_v4/fp8.py:325-341): A = dY_e^T, B = X_e^T from lp_quant_fp8_colwise_t.
 */
int lp_gemm_fp8_rowscale(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype,
                         int64_t M, int64_t N, int64_t K, void *C, int out_dtype, lp_stream_t stream);

/*
 * The same for a list of problems that share M and N and differ in K, in one launch: the weight gradients of all
 * experts of a grouped linear, which the reference issues as one grouped GEMM call
 * (gpatch_v4/models/deepseek_v4/fp8.py:325-341).  `groups` is a device array of G entries of four int32:
 * {output slot, K blocks of 128 of this problem, K blocks of all problems stored before it, unused}.  Problem g
 * reads Aq + M * 128 * before (its [M, K_g] codes), As + M * before scales, Bq / Bs likewise with N, and writes
 * C + slot * M * N elements.  max_k_blocks bounds every entry's K blocks (argument checks); k_blocks_multiple is
 * the caller's promise that every entry's K block count is a multiple of it (4 selects the hand-scheduled loop
 * with e8m0 scales; max_k_blocks = k_blocks_multiple = 1 or 2, i.e. every entry has exactly that many blocks,
 * selects the kernel without a K loop for short experts, whose entries of any other size write nothing).  A caller
 * with problems of several kinds makes one call per kind (gcore_lowp/grouped_gemm_fp8.py: rowscale_launches).
 * M must be a multiple of 128.  Entries with 0 blocks write nothing.  The table lives in device memory, so the
 * host cannot check it: an entry that breaks these promises (more K blocks than max_k_blocks, a count that is not
 * a multiple of 4 on the hand-scheduled kernel, a negative slot or offset) computes and writes nothing -- its C_g
 * keeps what it held.
 */
int lp_gemm_fp8_rowscale_grouped(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype,
                                 const int32_t *groups, int G, int max_k_blocks, int k_blocks_multiple, int64_t M,
                                 int64_t N, void *C, int out_dtype, lp_stream_t stream);

/*
 * Column-wise quantiser with transposed output for expert-grouped rows.  x: device [rows, cols]
 * (LP_BF16 or LP_F32), rows of expert e = m_offsets[e] .. m_offsets[e+1]-1 (device int32 [E+1]),
 * cols % 128 == 0.  Per expert, P_e = ceil(M_e / pad_rows) * pad_rows (pad_rows 128, 256 or 512; with 512
 * lp_gemm_fp8_rowscale runs on its hand-scheduled kernel), or with pad_rows = LP_PAD_MIXED: M_e rounded up to 128 for
 * experts of at most 256 rows and to 512 for the others (lp_gemm_fp8_rowscale_grouped has a kernel for problems of one
 * and two K blocks, which most experts of a routed batch are), and
 *   qT block e: [cols, P_e] e4m3fn at byte offset cols * (P_0 + .. + P_{e-1}), zero codes in the pad,
 *   sT block e: [cols, P_e / 128] scales at element offset cols * (P_0 + .. + P_{e-1}) / 128,
 * scale = 2^ceil(log2(amax / 448)) per (column, 128 rows of the expert), 1 for an all-zero block
 * (LP_SCALE_POW2; blocks of padding only get scale 1 and zero codes).  padded_blocks = sum_e P_e / 128 (the caller knows the row counts: the reference
 * passes m_splits as a host list, fp8.py:193).  Replaces the column-wise half of tex.split_quantize
 * (fp8.py:231,292-294) for Float8BlockScaling with power-of-two scales.
 */
int lp_quant_fp8_colwise_t(const void *x, int x_dtype, int64_t rows, int64_t cols, const int32_t *m_offsets,
                           int E, int64_t padded_blocks, int pad_rows, void *qT, void *sT, int scale_dtype,
                           lp_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LOWP_H */
