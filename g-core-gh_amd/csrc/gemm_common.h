// Pieces shared by the FP8 GEMM translation units.
#pragma once
#include "lowp_device.h"

namespace lowp {
namespace gemm {

template <int SDT>
__device__ __forceinline__ float scale_at(const void *s, int64_t idx)
{
    if (SDT == LP_F32) return ((const float *)s)[idx];
    // e8m0: 2^(b-127); byte 0 is the fp32 subnormal 2^-127 and 0xFF is NaN
    const uint32_t b = ((const uint8_t *)s)[idx];
    return u2f(b == 0u ? 0x00400000u : (b == 0xFFu ? 0x7FC00000u : b << 23));
}

// Tile order: tiles are numbered so that 32 consecutive numbers form a block of
// 8 M-tiles x 4 N-tiles (shared operand panels), and each XCD (workgroup id
// modulo 8) is handed whole blocks, so panels are re-used out of one L2.
constexpr int GROUP_M = 8, GROUP_N = 4, CHUNK = GROUP_M * GROUP_N;

// ends_first: the chunks an XCD works through come alternately from the front and the back of the tile
// list (grid = number of workgroups launched, a multiple of 8 * CHUNK).  Grouped problems list experts in
// caller order; when the heavy experts sit at one end, this keeps compute-bound tiles and tiles that only
// stream weights on the machine at the same time.
__device__ __forceinline__ bool tile_coords(int64_t b, int64_t tiles_m, int64_t tiles_n, int64_t &tm, int64_t &tn,
                                            bool ends_first = false, int64_t grid = 0)
{
    const int64_t xcd = b & 7, s = b >> 3;
    int64_t q = s / CHUNK;
    if (ends_first) {
        const int64_t Q = grid / (8 * CHUNK);
        q = (q & 1) ? Q - 1 - (q >> 1) : (q >> 1);
    }
    const int64_t lin = (q * 8 + xcd) * CHUNK + s % CHUNK;
    if (lin >= tiles_m * tiles_n) return false;
    // groups of GROUP_M m-tiles (the last may be short); inside a group, blocks of
    // GROUP_N n-tiles (the last may be narrow); inside a block m runs fastest
    const int64_t per_group = GROUP_M * tiles_n;
    const int64_t grp = lin / per_group, in_grp = lin - grp * per_group;
    const int64_t left = tiles_m - grp * GROUP_M;
    const int64_t gm = left < GROUP_M ? left : GROUP_M;
    const int64_t per_nblock = gm * GROUP_N;
    const int64_t nblk = in_grp / per_nblock, in_blk = in_grp - nblk * per_nblock;
    tm = grp * GROUP_M + in_blk % gm;
    tn = nblk * GROUP_N + in_blk / gm;
    return true;
}

// Rows of expert e from the caller's offset table, made safe to use: both ends are clamped to [0, M_total] and a
// decreasing pair is an empty expert, so a bad table cannot send a tile outside the operands.
__device__ __forceinline__ int expert_rows(const int32_t *__restrict__ m_offsets, int e, int64_t M_total, int64_t &begin)
{
    int64_t a = m_offsets[e], b = m_offsets[e + 1];
    a = a < 0 ? 0 : (a > M_total ? M_total : a);
    b = b < 0 ? 0 : (b > M_total ? M_total : b);
    begin = a;
    return b > a ? (int)(b - a) : 0;
}

inline int64_t padded_grid(int64_t tiles_m, int64_t tiles_n)
{
    const int64_t chunks = (tiles_m * tiles_n + CHUNK - 1) / CHUNK;
    return ((chunks + 7) / 8) * 8 * CHUNK;
}

// gemm_fp8_big.hip
int choose_big_tn(int64_t M, int64_t N);
int launch_big(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N,
               int64_t K, void *C, int64_t ldc, int out_dtype, int tn, hipStream_t st);

bool rowscale_asm_ok(const void *As, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K);
int launch_rowscale_asm(const void *Aq, const void *As, const void *Bq, const void *Bs, int64_t M, int64_t N, int64_t K, void *C,
                        int out_dtype, hipStream_t st);

// gemm_skinny.hip: at most 64 activation rows
constexpr int kSkinnyBlocks = 7;          // K blocks one workgroup handles
// at most 16 activation rows: one workgroup per 16 weight rows over all of K (gemm_thin.hip)
bool thin_ok(int64_t M, int64_t N, int64_t K);
bool thin_rows_ok(int64_t M, int64_t N, int64_t K);
int launch_thin_rows(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K,
                     void *C, int out_dtype, hipStream_t st);
// per-row e8m0 scales, problems of one or two K blocks, no K loop (gemm_rowscale_small.hip); groups == nullptr: one problem
int launch_rowscale_small(const void *Aq, const void *As, const void *Bq, const void *Bs, const int32_t *groups, int G, int k_blocks,
                          int64_t M, int64_t N, void *C, int out_dtype, hipStream_t st);
int launch_thin(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K,
                void *C, int out_dtype, hipStream_t st);
void skinny_plan(int64_t N, int64_t K, int &splits, int &per);
int64_t skinny_workspace_bytes(int64_t N, int splits);
int launch_skinny(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N,
                  int64_t K, void *C, int out_dtype, float *ws, int splits, int per, hipStream_t st);

int launch_rowscale_grouped_asm(const void *Aq, const void *As, const void *Bq, const void *Bs, const int32_t *groups, int G, int max_k_blocks, int64_t M,
                                int64_t N, void *C, int out_dtype, hipStream_t st);
int launch_nt_unit_scales(const void *A, const void *B, const void *ones, int64_t M, int64_t N, int64_t K, void *C, int out_dtype,
                          hipStream_t st, bool bf16 = false);
bool nt_unit_scales_ok(const void *ones, int64_t M, int64_t N, int64_t K);
bool launch_wide(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K,
                 void *C, int64_t ldc, int out_dtype, hipStream_t st, int *rc);
bool launch_mixed(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K,
                  int64_t n_big, void *C, int64_t ldc, int out_dtype, hipStream_t st, int *rc);
bool mid_asm_ok(const void *As, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K);
int launch_mid_asm(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N,
                   int64_t K, void *C, int64_t ldc, int out_dtype, hipStream_t st);
bool big_grouped_ok(const void *As, const void *Bs, int scale_dtype, int64_t M_total, int64_t N, int64_t K);
bool grouped_nn_ok(const void *As, const void *Bs, int scale_dtype, int E, int64_t M_total, int64_t N, int64_t K);
int launch_grouped_nn(const void *Aq, const void *As, const void *Bq, const void *Bs, const int32_t *m_offsets, int E,
                      int64_t M_total, int64_t N, int64_t K, void *C, int out_dtype, hipStream_t st);
int launch_big_grouped(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype,
                       const int32_t *m_offsets, int E, int64_t M_total, int64_t N, int64_t K, void *C, int out_dtype,
                       hipStream_t st);

}  // namespace gemm
}  // namespace lowp
