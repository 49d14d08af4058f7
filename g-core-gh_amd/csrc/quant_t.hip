// Column-wise ("transposed") block quantiser for the weight-gradient GEMM of a grouped linear on gfx950.
//
// The weight gradient of expert e is dY_e^T [N, M_e] x X_e [M_e, K]: the contraction runs over the expert's rows,
// so both operands are needed with that dimension contiguous and scaled per 128 of it.  This kernel takes a
// row-major [rows, cols] tensor whose rows are grouped by expert (m_offsets) and writes, per expert, the
// transposed codes [cols, P_e] with one power-of-two scale per (column, 128 rows), P_e = M_e rounded up to a
// multiple of pad_rows (128, or 512 so that the row-scaled GEMM can run its K loop in whole groups of four blocks).  Blocks restart at every expert; the rows that pad the last block are zero codes and take no
// part in the block's amax.  Expert e's matrices start at cols * (P_0 + .. + P_{e-1}) in the code buffer and at
// that over 128 in the scale buffer, so each expert's pair is a contiguous operand for lp_gemm_fp8_rowscale.
// One workgroup (256 threads) = 128 rows x 128 columns.  A thread owns 8 consecutive rows x 8 consecutive columns
// (16 lanes cover the 256 bytes of a row, all 8 row loads are issued before anything else); the column amax goes
// thread -> the 4 lanes of a wave that share the columns (two shuffles) -> the 4 waves (1 KB of LDS, one barrier);
// every thread then holds the scales of its 8 columns and quantises; per column its 8 codes (8 consecutive rows = 8
// contiguous bytes of the transposed output) go to a 16 KB LDS tile [column][row], swizzled so that neither side has
// bank conflicts, and leave from there as whole 128-byte lines, 16 bytes per lane (measured 5-13 % faster than letting
// the 16 threads of 4 waves that share a line store 8 bytes each).  A block that is padding only loads nothing.
#include <stdlib.h>

#include "lowp_device.h"

using namespace lowp;

namespace {

// max of two pairs of unsigned 16-bit integers
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b)
{
    uint32_t r;
    asm("v_pk_max_u16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

// 128-row blocks an expert of `rows` rows takes: rows rounded up to pad_rows, or with pad_rows = LP_PAD_MIXED to 128 up to
// 256 rows and to 512 beyond (short experts then run the row-scaled GEMM's one- and two-block kernel, the others its loop)
__device__ __forceinline__ int padded_blocks_of(int rows, int pad_rows)
{
    if (pad_rows == LP_PAD_MIXED) return rows <= 256 ? (rows + 127) >> 7 : ((rows + 511) >> 9) << 2;
    return (rows + pad_rows - 1) / pad_rows * (pad_rows >> 7);
}

template <bool IS_BF16>
__global__ __launch_bounds__(256) void quant_colwise_t(const void *__restrict__ x, int64_t cols, const int32_t *__restrict__ m_offsets,
                                                       int E, int pad_rows, uint8_t *__restrict__ qT, void *__restrict__ sT, int scale_dtype,
                                                       int cols_fastest)
{
    __shared__ u32x4 wave_max[4][16][2];                 // [wave][column chunk][8 columns as fp32-bit maxima, 4 + 4]
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int cc = t & 15, rg = t >> 4;                  // column chunk (8 columns), row group (8 rows)
    const int64_t blk = cols_fastest ? blockIdx.y : blockIdx.x, c0 = (int64_t)(cols_fastest ? blockIdx.x : blockIdx.y) * 128;
    // which expert owns padded block `blk`: every wave finds it for itself, without LDS or barriers (the loads cannot start
    // before it is known).  Lane l counts the blocks of experts 64 k + l; a prefix sum over the wave (shuffles) and a
    // running total over the rounds k locate the expert whose range of blocks holds blk.
    int hit_e = -1, hit_pb = 0, hit_rb = 0, hit_re = 0;
    int64_t pb = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
        const int ee = e0 + lane;
        const int rb = ee < E ? m_offsets[ee] : 0, re = ee < E ? m_offsets[ee + 1] : 0;
        const int cnt = padded_blocks_of(re - rb, pad_rows);
        int incl = cnt;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int y = __shfl_up(incl, off, 64);
            if (lane >= off) incl += y;
        }
        const int64_t end = pb + incl;                    // blocks up to and including this lane's expert
        const unsigned long long found = __ballot(cnt > 0 && blk >= end - cnt && blk < end);
        if (found) {
            const int src = __ffsll((long long)found) - 1;
            hit_e = e0 + src;
            hit_pb = __shfl((int)(end - cnt), src, 64);
            hit_rb = __shfl(rb, src, 64);
            hit_re = __shfl(re, src, 64);
            break;
        }
        pb += __shfl(incl, 63, 64);
        if (blk < pb) break;                              // uniform over the wave
    }
    if (hit_e < 0) return;
    pb = hit_pb;
    const int r_begin = hit_rb, r_end = hit_re;
    const int nblk = padded_blocks_of(r_end - r_begin, pad_rows);
    const int lb = (int)(blk - pb);                      // block inside the expert
    const int64_t r0 = (int64_t)r_begin + (int64_t)lb * 128;
    const int valid = r_end - r0 < 128 ? (r_end - r0 > 0 ? (int)(r_end - r0) : 0) : 128;      // 0: a block of padding only

    // ---- loads: row rg * 8 + i, columns c0 + 8 cc .. + 7; rows past the expert's end repeat its last row and
    // are zeroed afterwards (no branch between the loads)
    // The loaded words stay as they are; bf16 pairs are unpacked where they are used (32 registers instead of 64 live
    // across the barrier); with the other waves' maxima read one wave at a time below, a thread needs 69 registers and
    // seven workgroups share a CU (96 and five with those reads unrolled, 123 and four with floats kept).
    constexpr int W = IS_BF16 ? 4 : 8;
    uint32_t rw[8][W];
    {
        u32x4 raw[8][IS_BF16 ? 1 : 2] = {};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (valid == 0) break;                        // uniform over the workgroup
            const int row = rg * 8 + i;
            const int64_t r = r0 + (row < valid ? row : valid - 1);
            if (IS_BF16) {
                raw[i][0] = __builtin_nontemporal_load((const u32x4 *)((const uint16_t *)x + r * cols + c0 + cc * 8));
            } else {
                const u32x4 *src = (const u32x4 *)((const float *)x + r * cols + c0 + cc * 8);
                raw[i][0] = __builtin_nontemporal_load(src);
                raw[i][1] = __builtin_nontemporal_load(src + 1);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const bool live = rg * 8 + i < valid;
#pragma unroll
            for (int k = 0; k < W; ++k) rw[i][k] = live ? raw[i][k >> 2][k & 3] : 0u;
        }
    }
    auto elem = [&](int i, int j) -> float {
        if (IS_BF16) return u2f((j & 1) ? rw[i][(j >> 1) & 3] & 0xFFFF0000u : rw[i][(j >> 1) & 3] << 16);
        return u2f(rw[i][j & (W - 1)]);
    };
    // ---- column maxima of |x| as integers on the sign-cleared bits (inf / NaN sort above every finite value).
    // The kernel is bound by its arithmetic, not by memory (with loads and stores taken out it ran in three quarters
    // of its time), so bf16 maxima are taken on the packed words, two columns per instruction (16-bit integer max).
    uint32_t m[8];
    if constexpr (IS_BF16) {
        uint32_t pk[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            uint32_t a = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) a = pk_max_u16(a, rw[i][k] & 0x7FFF7FFFu);
            // lanes l, l ^ 16, l ^ 32, l ^ 48 hold the same columns
            a = pk_max_u16(a, (uint32_t)__shfl_xor((int)a, 16, 64));
            pk[k] = pk_max_u16(a, (uint32_t)__shfl_xor((int)a, 32, 64));
        }
        if (lane < 16) wave_max[wave][cc][0] = u32x4{pk[0], pk[1], pk[2], pk[3]};
        __syncthreads();
        // opaque to the compiler: what was unpacked for the maxima is not kept, the codes unpack again from these words
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int k = 0; k < W; ++k) asm volatile("" : "+v"(rw[i][k]));
        }
        uint32_t all[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const u32x4 a = wave_max[w][cc][0];
            all[0] = pk_max_u16(all[0], a.x);
            all[1] = pk_max_u16(all[1], a.y);
            all[2] = pk_max_u16(all[2], a.z);
            all[3] = pk_max_u16(all[3], a.w);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) m[j] = (j & 1) ? all[j >> 1] & 0xFFFF0000u : all[j >> 1] << 16;
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            uint32_t a = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t b = f2u(elem(i, j)) & 0x7FFFFFFFu;
                a = b > a ? b : a;
            }
            // lanes l, l ^ 16, l ^ 32, l ^ 48 hold the same columns
            uint32_t o = (uint32_t)__shfl_xor((int)a, 16, 64);
            a = o > a ? o : a;
            o = (uint32_t)__shfl_xor((int)a, 32, 64);
            m[j] = o > a ? o : a;
        }
        if (lane < 16) {
            wave_max[wave][cc][0] = u32x4{m[0], m[1], m[2], m[3]};
            wave_max[wave][cc][1] = u32x4{m[4], m[5], m[6], m[7]};
        }
        __syncthreads();
#pragma unroll 1                         // one wave's maxima at a time: unrolled, the 32 loaded registers set the kernel's peak
        for (int w = 0; w < 4; ++w) {
            const u32x4 a = wave_max[w][cc][0], b = wave_max[w][cc][1];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                m[j] = a[j] > m[j] ? a[j] : m[j];
                m[4 + j] = b[j] > m[4 + j] ? b[j] : m[4 + j];
            }
        }
    }
    // ---- scales, codes, stores
    const int64_t P = (int64_t)nblk * 128;
    const int64_t base = cols * pb * 128;                // codes of the experts before this one
    __shared__ __attribute__((aligned(16))) u32x2 turned[128 * 16];      // [column][16 groups of 8 rows], groups XOR-swizzled by column chunk
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const bool special = m[j] >= 0x7F800000u;        // inf or NaN in the block: literal arithmetic
        const float amax = u2f(m[j] > 0x7F800000u ? 0x7FC00000u : m[j]);
        BlockScale bs;
        if (IS_BF16 && !special) {
            // s = 2^ceil(log2(amax / 448)) without the division: amax = f * 2^k with 1 <= f < 2 and 448 = 1.75 * 2^8, so the
            // exponent is k - 8, and one more when f > 1.75.  (fl32(amax / 448) is a power of two only for f = 1.75: a bf16 f
            // is no closer than 1 / 224 to it otherwise, far beyond the rounding of the division.)  amax below the
            // smallest normal counts as that, a zero block gets the scale 1.
            const uint32_t ab = m[j] < 0x00800000u ? 0x00800000u : m[j];
            const int e = m[j] == 0u ? 0 : (int)(ab >> 23) - 135 + ((ab & 0x7FFFFFu) > 0x600000u ? 1 : 0);
            bs.stored = e < -126 ? u2f(1u << (e + 149)) : u2f((uint32_t)(e + 127) << 23);
            bs.div = 1.0f; bs.recip = 1.0f; bs.exp2 = e; bs.fast = true;
        } else {
            bs = derive_scale<LP_SCALE_POW2>(amax, 0.0f, LP_ZERO_NONE);
        }
        const int64_t c = c0 + cc * 8 + j;
        if (rg == 0) store_scale(sT, scale_dtype, cols * pb + c * nblk + lb, bs.stored);
        uint32_t lo, hi;
        if (special) {
            lo = hi = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                lo |= (uint32_t)quant_slow<LP_SCALE_POW2>(elem(i, j), bs) << (8 * i);
                hi |= (uint32_t)quant_slow<LP_SCALE_POW2>(elem(4 + i, j), bs) << (8 * i);
            }
        } else {
            // |x| <= amax <= 448 * 2^e and x * 2^-e is exact: no quotient leaves the e4m3 range, nothing to clamp
            float y[8];
            if (bs.exp2 < -126 || bs.exp2 > 126) {                       // 2^-e is not a normal float: rare, and exact either way
#pragma unroll
                for (int i = 0; i < 8; ++i) y[i] = ldexpf(elem(i, j), -bs.exp2);
            } else {
                const float f = u2f((uint32_t)(127 - bs.exp2) << 23);
#pragma unroll
                for (int i = 0; i < 8; ++i) y[i] = elem(i, j) * f;
            }
            lo = cvt4(y[0], y[1], y[2], y[3]);
            hi = cvt4(y[4], y[5], y[6], y[7]);
        }
        turned[(cc * 8 + j) * 16 + (rg ^ cc)] = u32x2{lo, hi};
    }
    // 8 lanes write the 128 bytes of a column's line, 16 bytes each: a store instruction of a wave covers 8 whole lines
    __syncthreads();
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int col = p * 32 + (t >> 3), pair = t & 7, sw = (col >> 3) & 15;
        const u32x4 raw = *(const u32x4 *)&turned[col * 16 + ((pair ^ (sw >> 1)) << 1)];
        const u32x4 out = (sw & 1) ? u32x4{raw[2], raw[3], raw[0], raw[1]} : raw;
        *(u32x4 *)(qT + base + (c0 + col) * P + (int64_t)lb * 128 + pair * 16) = out;
    }
}

}  // namespace

extern "C" int lp_quant_fp8_colwise_t(const void *x, int x_dtype, int64_t rows, int64_t cols, const int32_t *m_offsets, int E,
                                      int64_t padded_blocks, int pad_rows, void *qT, void *sT, int scale_dtype, lp_stream_t stream)
{
    LP_REQUIRE(pad_rows == 128 || pad_rows == 256 || pad_rows == 512 || pad_rows == LP_PAD_MIXED,
               "lp_quant_fp8_colwise_t: pad_rows must be 128, 256, 512 or LP_PAD_MIXED");
    LP_REQUIRE(x_dtype == LP_BF16 || x_dtype == LP_F32, "lp_quant_fp8_colwise_t: x_dtype must be LP_BF16 or LP_F32");
    LP_REQUIRE(scale_dtype == LP_F32 || scale_dtype == LP_E8M0, "lp_quant_fp8_colwise_t: scale_dtype must be LP_F32 or LP_E8M0");
    LP_REQUIRE(rows >= 0 && cols >= 0 && E >= 0 && padded_blocks >= 0, "lp_quant_fp8_colwise_t: bad shape");
    LP_REQUIRE(cols % 128 == 0, "lp_quant_fp8_colwise_t: cols (%lld) must be a multiple of 128", (long long)cols);
    if (cols == 0 || padded_blocks == 0 || E == 0) return LP_OK;
    LP_REQUIRE(x && m_offsets && qT && sT, "lp_quant_fp8_colwise_t: null pointer");
    LP_REQUIRE((uintptr_t)qT % 16 == 0, "lp_quant_fp8_colwise_t: qT must be 16-byte aligned");
    LP_REQUIRE(padded_blocks <= 0x7FFFFFFF && cols / 128 <= 65535, "lp_quant_fp8_colwise_t: problem too large");
    // Workgroups that run together should read whole rows between them: the column blocks of one row block are
    // numbered consecutively (217 -> 187 us on a [65536, 4096] gradient against row blocks first, whose concurrent
    // reads were 256-byte pieces 8 KB apart).  The grid's second dimension holds 65535 at most.
    static const int order_env = getenv("LP_COLWISE_ROWS_FIRST") ? atoi(getenv("LP_COLWISE_ROWS_FIRST")) : 0;
    const int cols_fastest = !order_env && padded_blocks <= 65535 ? 1 : 0;
    const dim3 grid = cols_fastest ? dim3((unsigned)(cols / 128), (unsigned)padded_blocks) : dim3((unsigned)padded_blocks, (unsigned)(cols / 128));
    if (x_dtype == LP_BF16)
        hipLaunchKernelGGL(quant_colwise_t<true>, grid, dim3(256), 0, (hipStream_t)stream, x, cols, m_offsets, E, pad_rows, (uint8_t *)qT, sT,
                           scale_dtype, cols_fastest);
    else
        hipLaunchKernelGGL(quant_colwise_t<false>, grid, dim3(256), 0, (hipStream_t)stream, x, cols, m_offsets, E, pad_rows, (uint8_t *)qT, sT,
                           scale_dtype, cols_fastest);
    return check_launch("lp_quant_fp8_colwise_t");
}
