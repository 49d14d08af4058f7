/*
 * lowp_probe -- measurement and test aids for the MI355X (gfx950) low-precision path.
 *
 * A second, small shared library (liblowp_probe.so) beside the product library declared in lowp.h:
 * on-device self tests of the gfx950 conversion instructions, bulk casts for tests, and the probes the
 * benchmark times beside the kernels (bare stream, register-only matrix loop, L2 -> CU copy loop).
 * Nothing here stands in for a reference interface and no product code path calls it; the product
 * library does not link against it.  Conventions (device pointers, stream, return codes) are those of
 * lowp.h; the message of a failed call comes from lp_probe_last_error() (thread local).
 */
#ifndef LOWP_PROBE_H
#define LOWP_PROBE_H

#include <stdint.h>

#include "lowp.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Message of the last failed call of this library on the calling thread. */
const char *lp_probe_last_error(void);

/*
 * On-device self tests of the gfx950 conversion instructions against the
 * library's software casts.  Each writes the number of mismatching inputs to
 * *mismatches (device uint64, zeroed by the call).  No reference counterpart.
 *   which = 0: v_cvt_pk_fp8_f32 over every fp32 with |x| <= 464 (and +-0)
 *   which = 1: v_cvt_pk_f32_fp8 over all 256 codes except the two NaNs
 *   which = 2: fp32 -> bf16 conversion over every non-NaN fp32
 *   which = 3: v_cvt_scalef32_pk_f32_fp4 over 256 bytes x the scale exponents used
 *   which = 4: v_cvt_scalef32_pk_fp4_f32 with the tie adjustment of lp_quant_fp4_block
 *              over every finite fp32 at three scales
 */
int lp_selftest(int which, uint64_t *mismatches, lp_stream_t stream);

/*
 * Measurement aid: one launch of `workgroups` x 256 threads that reads read_bytes from src (16-byte non-temporal
 * loads, contiguous share per workgroup) and writes write_bytes to dst (16-byte stores of a value derived from what
 * was read).  Either count may be 0; with both 0 it is an empty launch.  It does no work the library needs: it
 * shows what a launch and a stream of that many bytes cost on the box, next to the kernels of the same size
 * (the benchmark times it beside the skinny GEMM's 29 MB weight stream and the 4096 x 4096 quantiser).
 * No reference counterpart.
 */
int lp_probe_stream(const void *src, int64_t read_bytes, void *dst, int64_t write_bytes, int workgroups, lp_stream_t stream);

/*
 * Measurement aid: one launch of `workgroups` x 512 threads (two waves per SIMD) that issues, `iters` times, eight fp8
 * 16x16x128 matrix instructions each followed by fmas_per_instruction (0, 2, 4, 6, 8) fp32 FMAs, on registers only: no
 * LDS, no memory traffic in the loop.  operands: 4096 bytes of e4m3 codes (64 per lane) for the matrix operands, or NULL
 * for zeros.  Flops = workgroups x 8 waves x iters x 8 x 2 x 16 x 16 x 128.  It shows the rate the matrix cores hold
 * with the arithmetic of an fp32-scaled GEMM loop (four FMAs per instruction) and nothing else: the ceiling the GEMM
 * kernels' fraction of peak is to be read against.  Negative values select the accumulate-in-place forms without FMAs:
 * -1 the hardware-scaled instruction (unit e8m0 scale bytes) and -2 the unscaled one with 512 threads per workgroup,
 * -3 and -4 the same two with 256 threads (one wave per SIMD; flops then count 4 waves).  No reference counterpart.
 */
int lp_probe_mfma(int fmas_per_instruction, int iters, const void *operands, int workgroups, lp_stream_t stream);

/*
 * Measurement aid: what a CU's copy path out of the L2 delivers in the shape the GEMM loops use it.  One launch of
 * `workgroups` x 64 * waves threads (waves = 4: 64 KB of LDS per workgroup, two fit a CU; 8: 128 KB, one per CU); every
 * wave issues, `steps` times, eight requests of 1 KB (8 rows x 128 bytes, rows row_stride bytes apart, 16 bytes per lane)
 * and keeps one step in flight behind a wait and a workgroup barrier, as a two-stage K loop does.  to_lds != 0: straight
 * into LDS (global_load_lds, what the loops use); 0: into registers.  src: 4 regions of 512 rows x row_stride bytes
 * (src_bytes says how much is there), read over and over, so it is served by the L2 after the first pass; sink: 2048
 * bytes that are never written in practice.  Bytes moved = workgroups x waves x steps x 8192.  It shows the ceiling of
 * the operand copies: a 128 x 128 tile asks for 32 KB per 16 matrix instructions of each SIMD, a 256 x 256 tile for 64 KB
 * per 64.  No reference counterpart.
 */
int lp_probe_copy(int to_lds, int waves, int steps, const void *src, int64_t src_bytes, int64_t row_stride, void *sink,
                  int workgroups, lp_stream_t stream);

/* Bulk element-wise casts through the library's device code paths (debug aid
 * for tests): kind 0 = fp32 -> e4m3fn software, 1 = fp32 -> e4m3fn hardware
 * (inputs clamped to +-448 first), 2 = fp32 -> e8m0, 3 = fp32 -> bf16. */
int lp_debug_cast(int kind, const float *x, void *out, int64_t n, lp_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LOWP_PROBE_H */
