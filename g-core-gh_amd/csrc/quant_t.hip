// Column-wise ("transposed") block quantiser for the weight-gradient GEMM of a grouped linear on gfx950.
//
// The weight gradient of expert e is dY_e^T [N, M_e] x X_e [M_e, K]: the contraction runs over the expert's rows,
// so both operands are needed with that dimension contiguous and scaled per 128 of it.  This kernel takes a
// row-major [rows, cols] tensor whose rows are grouped by expert (m_offsets) and writes, per expert, the
// transposed codes [cols, P_e] with one power-of-two scale per (column, 128 rows), P_e = M_e rounded up to a
// multiple of 128.  Blocks restart at every expert; the rows that pad the last block are zero codes and take no
// part in the block's amax.  Expert e's matrices start at cols * (P_0 + .. + P_{e-1}) in the code buffer and at
// that over 128 in the scale buffer, so each expert's pair is a contiguous operand for lp_gemm_fp8_rowscale.
// One workgroup = 128 rows x 128 columns: read along the rows (coalesced), turned in LDS, one thread per column
// quantises its 128 values and writes them as one 128-byte line.
#include "lowp_device.h"

using namespace lowp;

namespace {

template <bool IS_BF16>
__global__ __launch_bounds__(128) void quant_colwise_t(const void *__restrict__ x, int64_t cols, const int32_t *__restrict__ m_offsets,
                                                       int E, uint8_t *__restrict__ qT, void *__restrict__ sT, int scale_dtype)
{
    __shared__ float tile[128][128];                     // [row][column]
    const int t = threadIdx.x;
    const int64_t blk = blockIdx.x, c0 = (int64_t)blockIdx.y * 128;
    // which expert owns padded block `blk` (every thread walks the offsets; E is a few hundred at most)
    int64_t pb = 0;
    int e = 0, nblk = 0, r_begin = 0, r_end = 0;
    for (; e < E; ++e) {
        r_begin = m_offsets[e];
        r_end = m_offsets[e + 1];
        nblk = (r_end - r_begin + 127) >> 7;
        if (blk < pb + nblk) break;
        pb += nblk;
    }
    if (e >= E) return;
    const int lb = (int)(blk - pb);                      // block inside the expert
    const int64_t r0 = (int64_t)r_begin + (int64_t)lb * 128;
    const int valid = r_end - r0 < 128 ? (int)(r_end - r0) : 128;
    for (int i = 0; i < 128; ++i) {
        float v = 0.0f;
        if (i < valid) {
            const int64_t idx = (r0 + i) * cols + c0 + t;
            v = IS_BF16 ? u2f((uint32_t)((const uint16_t *)x)[idx] << 16) : ((const float *)x)[idx];
        }
        tile[i][t] = v;
    }
    __syncthreads();
    uint32_t mbits = 0;
    for (int i = 0; i < 128; ++i) {
        const uint32_t a = f2u(tile[i][t]) & 0x7FFFFFFFu;
        mbits = a > mbits ? a : mbits;
    }
    const bool special = mbits >= 0x7F800000u;           // inf or NaN in the block: literal arithmetic
    const float amax = u2f(mbits > 0x7F800000u ? 0x7FC00000u : mbits);
    const BlockScale bs = derive_scale<LP_SCALE_POW2>(amax, 0.0f, LP_ZERO_NONE);
    const int64_t P = (int64_t)nblk * 128;
    const int64_t base = cols * pb * 128;                // codes of the experts before this one
    uint8_t *dst = qT + base + (c0 + t) * P + (int64_t)lb * 128;
    store_scale(sT, scale_dtype, cols * pb + (c0 + t) * nblk + lb, bs.stored);
#pragma unroll 4
    for (int i = 0; i < 128; i += 16) {
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float v0 = tile[i + 4 * j][t], v1 = tile[i + 4 * j + 1][t], v2 = tile[i + 4 * j + 2][t], v3 = tile[i + 4 * j + 3][t];
            if (special)
                w[j] = (uint32_t)quant_slow<LP_SCALE_POW2>(v0, bs) | ((uint32_t)quant_slow<LP_SCALE_POW2>(v1, bs) << 8) |
                       ((uint32_t)quant_slow<LP_SCALE_POW2>(v2, bs) << 16) | ((uint32_t)quant_slow<LP_SCALE_POW2>(v3, bs) << 24);
            else
                w[j] = cvt4(clamp448(scale_fast<LP_SCALE_POW2>(v0, bs)), clamp448(scale_fast<LP_SCALE_POW2>(v1, bs)),
                            clamp448(scale_fast<LP_SCALE_POW2>(v2, bs)), clamp448(scale_fast<LP_SCALE_POW2>(v3, bs)));
        }
        *(u32x4 *)(dst + i) = u32x4{w[0], w[1], w[2], w[3]};
    }
}

}  // namespace

extern "C" int lp_quant_fp8_colwise_t(const void *x, int x_dtype, int64_t rows, int64_t cols, const int32_t *m_offsets, int E,
                                      int64_t padded_blocks, void *qT, void *sT, int scale_dtype, lp_stream_t stream)
{
    LP_REQUIRE(x_dtype == LP_BF16 || x_dtype == LP_F32, "lp_quant_fp8_colwise_t: x_dtype must be LP_BF16 or LP_F32");
    LP_REQUIRE(scale_dtype == LP_F32 || scale_dtype == LP_E8M0, "lp_quant_fp8_colwise_t: scale_dtype must be LP_F32 or LP_E8M0");
    LP_REQUIRE(rows >= 0 && cols >= 0 && E >= 0 && padded_blocks >= 0, "lp_quant_fp8_colwise_t: bad shape");
    LP_REQUIRE(cols % 128 == 0, "lp_quant_fp8_colwise_t: cols (%lld) must be a multiple of 128", (long long)cols);
    if (cols == 0 || padded_blocks == 0 || E == 0) return LP_OK;
    LP_REQUIRE(x && m_offsets && qT && sT, "lp_quant_fp8_colwise_t: null pointer");
    LP_REQUIRE((uintptr_t)qT % 16 == 0, "lp_quant_fp8_colwise_t: qT must be 16-byte aligned");
    LP_REQUIRE(padded_blocks <= 0x7FFFFFFF && cols / 128 <= 65535, "lp_quant_fp8_colwise_t: problem too large");
    const dim3 grid((unsigned)padded_blocks, (unsigned)(cols / 128));
    if (x_dtype == LP_BF16)
        hipLaunchKernelGGL(quant_colwise_t<true>, grid, dim3(128), 0, (hipStream_t)stream, x, cols, m_offsets, E, (uint8_t *)qT, sT,
                           scale_dtype);
    else
        hipLaunchKernelGGL(quant_colwise_t<false>, grid, dim3(128), 0, (hipStream_t)stream, x, cols, m_offsets, E, (uint8_t *)qT, sT,
                           scale_dtype);
    return check_launch("lp_quant_fp8_colwise_t");
}
