// Block-scaled FP8 GEMM for gfx950:  C[m,n] = sum_kb (sum_{k in kb} Aq[m,k] Bq[n,k]) * As[m,kb] * Bs[n/128,kb].
//
// One 256-thread workgroup (4 waves, 2 x 2) owns a 128(M) x 128(N) tile of C and
// walks K in steps of 128 = one scale block.  Per step the two operand tiles
// (128 rows x 128 bytes each) are staged through LDS (double buffered, rows
// padded to 144 bytes so that 128-bit reads and writes are bank-conflict free),
// each wave issues v_mfma_f32_32x32x64_f8f6f4 with FP8 operands on its
// 64 x 64 sub-tile into a zero-initialised partial accumulator, and the partial
// is folded into the fp32 accumulator with one FMA per element by
// As[m,kb] * Bs[n/128,kb].
//
// The weight tile is the MFMA "A" operand and the activation tile the "B"
// operand, so the accumulator of a lane holds one activation row m (lane % 32)
// and 16 weight rows n: the activation scale is then a single value per lane.
//
// The same tile routine serves the dense, split-K (skinny M) and grouped
// (per-expert row ranges) entry points.
#include <pthread.h>
#include <stdlib.h>

#include "gemm_common.h"

using namespace lowp;
using lowp::gemm::scale_at;
using lowp::gemm::tile_coords;
using lowp::gemm::padded_grid;

namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int TM = 128, TN = 128, TK = 128;
constexpr int LDS_ROW = TK + 16;                 // bytes per staged row
constexpr int TILE_BYTES = 128 * LDS_ROW;        // one operand tile in LDS

struct alignas(16) Smem {
    uint8_t a[2][TILE_BYTES];
    uint8_t b[2][TILE_BYTES];
    float as[2][TM];
    float bs[2][TN];     // per-row weight scales (row-scaled variant only)
};

struct TileArgs {
    const uint8_t *Aq;   // [*, K] activation codes
    const void *As;      // [*, K/128] activation scales
    const uint8_t *Bq;   // [N, K] weight codes of this problem (expert)
    const void *Bs;      // [N/128, K/128]
    int scale_dtype;
    int64_t K;
    int64_t kblocks;     // K / 128
    int64_t m0;          // first row of the tile
    int64_t m_end;       // rows >= m_end are not read or written
    int64_t n0;          // first weight row of the tile
    int kb_begin, kb_end;
};

// accumulators of one wave: acc[mb][nb] is a 32(n) x 32(m) block
struct Acc { f32x16 v[2][2]; };

// BROW: the second operand carries one scale per row and K block ([N, K/128]) instead of one per 128 x 128 block
template <int SDT, bool BROW = false>
__device__ __forceinline__ void gemm_tile(const TileArgs &ta, Smem &sm, Acc &acc)
{
    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lhi = lane >> 5;

#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc.v[mb][nb][r] = 0.0f;

    // global -> register staging: 4 chunks of 16 bytes per operand per thread
    u32x4 ga[4], gb[4];
    float gas = 0.0f;
    auto gload = [&](int kb) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = t + 256 * i;
            const int row = c >> 3, col = (c & 7) * 16;
            const int64_t m = ta.m0 + row;
            if (m < ta.m_end) ga[i] = *(const u32x4 *)(ta.Aq + m * ta.K + (int64_t)kb * TK + col);
            else ga[i] = u32x4{0, 0, 0, 0};
            gb[i] = *(const u32x4 *)(ta.Bq + (ta.n0 + row) * ta.K + (int64_t)kb * TK + col);
        }
        if (t < TM) {
            const int64_t m = ta.m0 + t;
            gas = m < ta.m_end ? scale_at<SDT>(ta.As, m * ta.kblocks + kb) : 0.0f;
        } else if (BROW) {
            gas = scale_at<SDT>(ta.Bs, (ta.n0 + t - TM) * ta.kblocks + kb);
        }
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = t + 256 * i;
            const int row = c >> 3, col = (c & 7) * 16;
            *(u32x4 *)(sm.a[buf] + row * LDS_ROW + col) = ga[i];
            *(u32x4 *)(sm.b[buf] + row * LDS_ROW + col) = gb[i];
        }
        if (t < TM) sm.as[buf][t] = gas;
        else if (BROW) sm.bs[buf][t - TM] = gas;
    };

    gload(ta.kb_begin);
    sstore(0);
    __syncthreads();

    for (int kb = ta.kb_begin; kb < ta.kb_end; ++kb) {
        const int buf = (kb - ta.kb_begin) & 1;
        const bool more = kb + 1 < ta.kb_end;
        if (more) gload(kb + 1);

        const float bscale = BROW ? 1.0f : scale_at<SDT>(ta.Bs, (ta.n0 >> 7) * ta.kblocks + kb);

        // operand fragments: lane reads 32 bytes of its row per 64-wide K half
        i32x8 wf[2][2], af[2][2];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int kh = 0; kh < 2; ++kh) {
                const int koff = kh * 64 + lhi * 32;
                const uint8_t *wp = sm.b[buf] + (wn * 64 + blk * 32 + l32) * LDS_ROW + koff;
                const uint8_t *ap = sm.a[buf] + (wm * 64 + blk * 32 + l32) * LDS_ROW + koff;
                u32x4 w0 = *(const u32x4 *)wp, w1 = *(const u32x4 *)(wp + 16);
                u32x4 a0 = *(const u32x4 *)ap, a1 = *(const u32x4 *)(ap + 16);
                wf[blk][kh] = i32x8{(int)w0.x, (int)w0.y, (int)w0.z, (int)w0.w, (int)w1.x, (int)w1.y, (int)w1.z, (int)w1.w};
                af[blk][kh] = i32x8{(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, (int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
            }
        // four 32 x 32 blocks; the fold of block i is issued after the MFMAs of block i+1
        // so that VALU work overlaps the matrix pipe
        const float sc0 = sm.as[buf][wm * 64 + l32] * bscale;
        const float sc1 = sm.as[buf][wm * 64 + 32 + l32] * bscale;
        const f32x16 zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        f32x16 p[4];
#pragma unroll
        for (int blk = 0; blk < 4; ++blk) {
            const int mb = blk >> 1, nb = blk & 1;
            p[blk] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[nb][0], af[mb][0], zero, 0, 0, 0, 0, 0, 0);
            p[blk] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[nb][1], af[mb][1], p[blk], 0, 0, 0, 0, 0, 0);
            if (blk > 0) {
                const int pm = (blk - 1) >> 1, pn = (blk - 1) & 1;
                const float sc = pm ? sc1 : sc0;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    // element r of a 32 x 32 block sits in weight row 8 (r / 4) + 4 (lane / 32) + r % 4
                    const float sr = BROW ? sc * sm.bs[buf][wn * 64 + pn * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3)] : sc;
                    acc.v[pm][pn][r] = __builtin_fmaf(p[blk - 1][r], sr, acc.v[pm][pn][r]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float sr = BROW ? sc1 * sm.bs[buf][wn * 64 + 32 + 8 * (r >> 2) + 4 * lhi + (r & 3)] : sc1;
            acc.v[1][1][r] = __builtin_fmaf(p[3][r], sr, acc.v[1][1][r]);
        }
        if (more) sstore(buf ^ 1);
        __syncthreads();
    }
}

// element (mb, nb, r) of a lane's accumulator sits at
//   m = m0 + wm*64 + mb*32 + lane%32
//   n = n0 + wn*64 + nb*32 + 8*(r/4) + 4*(lane/32) + r%4
template <typename F>
__device__ __forceinline__ void for_each_quad(const Acc &acc, int64_t m0, int64_t n0, F &&f)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
        const int64_t m = m0 + wm * 64 + mb * 32 + (lane & 31);
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int64_t n = n0 + wn * 64 + nb * 32 + 8 * g + 4 * (lane >> 5);
                f(m, n, acc.v[mb][nb][4 * g], acc.v[mb][nb][4 * g + 1], acc.v[mb][nb][4 * g + 2], acc.v[mb][nb][4 * g + 3]);
            }
    }
}

__device__ __forceinline__ void store_tile(const Acc &acc, int64_t m0, int64_t m_end, int64_t n0, int64_t ldc, void *C,
                                           int out_dtype)
{
    for_each_quad(acc, m0, n0, [&](int64_t m, int64_t n, float a, float b, float c, float d) {
        if (m >= m_end) return;
        if (out_dtype == LP_BF16) {
            u32x2 o = {pack_bf16(a, b), pack_bf16(c, d)};
            *(u32x2 *)((uint16_t *)C + m * ldc + n) = o;
        } else {
            u32x4 o = {f2u(a), f2u(b), f2u(c), f2u(d)};
            *(u32x4 *)((float *)C + m * ldc + n) = o;
        }
    });
}

template <int SDT, bool BROW = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_dense(const uint8_t *__restrict__ Aq, const void *__restrict__ As,
                                                  const uint8_t *__restrict__ Bq, const void *__restrict__ Bs,
                                                  int scale_dtype, int64_t M, int64_t N, int64_t K, int64_t tiles_m,
                                                  int64_t tiles_n, void *__restrict__ C, int64_t ldc, int out_dtype)
{
    __shared__ Smem sm;
    int64_t tm, tn;
    if (!tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
    TileArgs ta;
    ta.Aq = Aq; ta.As = As; ta.Bq = Bq; ta.Bs = Bs; ta.scale_dtype = scale_dtype;
    ta.K = K; ta.kblocks = K / TK; ta.m0 = tm * TM; ta.m_end = M; ta.n0 = tn * TN;
    ta.kb_begin = 0; ta.kb_end = (int)(K / TK);
    Acc acc;
    gemm_tile<SDT, BROW>(ta, sm, acc);
    store_tile(acc, ta.m0, M, ta.n0, ldc, C, out_dtype);
}

// Row-scaled problems that share M and N and differ in K, one launch (see gemm_asm_rowscale_grouped for `groups`).
template <int SDT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_rowscale_grouped(
    const uint8_t *__restrict__ Aq, const void *__restrict__ As, const uint8_t *__restrict__ Bq, const void *__restrict__ Bs,
    int scale_dtype, const int32_t *__restrict__ groups, int64_t M, int64_t N, int64_t tiles_m, int64_t tiles_n, int64_t per_group,
    void *__restrict__ C, int out_dtype, int max_k_blocks)
{
    __shared__ Smem sm;
    const int64_t g = blockIdx.x / per_group, local = blockIdx.x - g * per_group;
    int64_t tm, tn;
    if (!tile_coords(local, tiles_m, tiles_n, tm, tn)) return;
    const int64_t slot = groups[4 * g], kb = groups[4 * g + 1], before = groups[4 * g + 2];
    // an entry that breaks the caller's promise (more K blocks than max_k_blocks, on which the host checked the operand
    // sizes; a negative slot or offset) writes nothing
    if (kb <= 0 || kb > max_k_blocks || slot < 0 || before < 0) return;
    const int64_t ssz = SDT == LP_F32 ? 4 : 1;
    TileArgs ta;
    ta.Aq = Aq + M * 128 * before; ta.As = (const char *)As + M * before * ssz;
    ta.Bq = Bq + N * 128 * before; ta.Bs = (const char *)Bs + N * before * ssz;
    ta.scale_dtype = scale_dtype;
    ta.K = kb * 128; ta.kblocks = kb; ta.m0 = tm * TM; ta.m_end = M; ta.n0 = tn * TN;
    ta.kb_begin = 0; ta.kb_end = (int)kb;
    Acc acc;
    gemm_tile<SDT, true>(ta, sm, acc);
    store_tile(acc, ta.m0, M, ta.n0, N, (char *)C + slot * M * N * (out_dtype == LP_BF16 ? 2 : 4), out_dtype);
}

// ------------------------------------------------------------------ split-K
// Skinny problems (few output tiles) are weight-streaming bound: K is cut into
// `splits` contiguous ranges so that every CU pulls HBM; each range writes an
// fp32 partial tile to the workspace and a second kernel adds the ranges in a
// fixed order (deterministic) and narrows.

template <int SDT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_splitk(const uint8_t *__restrict__ Aq, const void *__restrict__ As,
                                                   const uint8_t *__restrict__ Bq, const void *__restrict__ Bs,
                                                   int scale_dtype, int64_t M, int64_t N, int64_t K, int64_t tiles_m,
                                                   int64_t tiles_n, int splits, int kb_per_split, float *__restrict__ ws)
{
    __shared__ Smem sm;
    const int64_t tile = blockIdx.x / splits;
    const int split = (int)(blockIdx.x - tile * splits);
    const int64_t tn = tile / tiles_m, tm = tile - tn * tiles_m;
    TileArgs ta;
    ta.Aq = Aq; ta.As = As; ta.Bq = Bq; ta.Bs = Bs; ta.scale_dtype = scale_dtype;
    ta.K = K; ta.kblocks = K / TK; ta.m0 = tm * TM; ta.m_end = M; ta.n0 = tn * TN;
    ta.kb_begin = split * kb_per_split;
    const int kb_all = (int)(K / TK);
    ta.kb_end = ta.kb_begin + kb_per_split < kb_all ? ta.kb_begin + kb_per_split : kb_all;
    Acc acc;
    if (ta.kb_begin < ta.kb_end) {
        gemm_tile<SDT>(ta, sm, acc);
    } else {
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc.v[mb][nb][r] = 0.0f;
    }
    store_tile(acc, ta.m0, M, ta.n0, N, ws + (int64_t)split * M * N, LP_F32);
}

// The ranges are added in their order.  All loads are issued before the first addition (a range past the last is read
// from the last and not added): a thread's time is one trip to memory instead of one per range, which is what a
// reduction of a few MB costs.
__global__ __launch_bounds__(256) void splitk_reduce(const float *__restrict__ ws, int splits, int64_t mn,
                                                     void *__restrict__ C, int out_dtype)
{
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= mn) return;
    f32x4 s = *(const f32x4 *)(ws + i);
    for (int k0 = 1; k0 < splits; k0 += 8) {
        f32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int k = k0 + j < splits ? k0 + j : splits - 1;
            v[j] = *(const f32x4 *)(ws + (int64_t)k * mn + i);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const bool on = k0 + j < splits;
            s.x += on ? v[j].x : 0.0f; s.y += on ? v[j].y : 0.0f; s.z += on ? v[j].z : 0.0f; s.w += on ? v[j].w : 0.0f;
        }
    }
    if (out_dtype == LP_BF16) {
        u32x2 o = {pack_bf16(s.x, s.y), pack_bf16(s.z, s.w)};
        *(u32x2 *)((uint16_t *)C + i) = o;
    } else {
        *(f32x4 *)((float *)C + i) = s;
    }
}

// how many K ranges to use: aim at >= 2 workgroups per CU (256 CUs).  Only for at most 32 tiles: with more, the
// hand-scheduled 128 x 128 kernel (which splits K inside the workgroup) is ahead of this kernel pair (one MI355X, us per
// call, pair against that kernel, fp32 / e8m0 scales: 16 tiles, 512 x 512 x 7168, 21.4 / 22.1 against 27.6 / 24.2; 32 tiles,
// 1024 x 512 x 7168, 22.4 / 23.5 against 29.5 / 26.0; 64 tiles, 2048 x 512 x 4096, 26.0 / 27.8 against 20.2 / 17.2; 72 tiles,
// 384 x 3072 x 4096, 30.7 / 32.5 against 20.4 / 17.7; 80 tiles, 640 x 2048 x 7168, 42.5 / 46.1 against 30.6 / 26.4; the pair's
// figures are from before its reduction issued all its loads at once, which took 1 - 2 us off: 4 tiles 14.4 -> 12.5).
// K ranges on the hand-scheduled 128 x 128 loop instead of this compiler-scheduled kernel were built and measured: level
// (4 tiles 12.2 against 12.5, 16 tiles 18.9 against 20.2, 32 tiles 22.7 against 22.4, 2000 x 128 x 7168 19.0 against 18.5) and,
// with more tiles, behind the single launch like this pair -- one workgroup per CU already keeps half of the CU's matrix
// rate, so two ranges that land on one CU take as long as the unsplit tile.
int choose_splits(int64_t tiles, int64_t kblocks)
{
    if (tiles > 32 || kblocks < 32) return 1;                 // short K: the second launch costs more than the split gains
    int64_t s = (512 + tiles - 1) / tiles;
    if (s > kblocks / 4) s = kblocks / 4;     // keep >= 4 K steps per range
    if (s > 16) s = 16;
    return s < 1 ? 1 : (int)s;
}

// ------------------------------------------------------------------ grouped
// Rows are sorted by expert; expert e owns rows m_offsets[e] .. m_offsets[e+1]-1.
// The grid is sized from an upper bound on the number of 128-row tiles; every
// workgroup finds its (expert, tile) from the offsets with a block-wide scan.

template <int SDT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_grouped(const uint8_t *__restrict__ Aq, const void *__restrict__ As,
                                                    const uint8_t *__restrict__ Bq, const void *__restrict__ Bs,
                                                    int scale_dtype, const int32_t *__restrict__ m_offsets, int E,
                                                    int64_t M_total, int64_t N, int64_t K, int64_t max_mtiles, int64_t tiles_n,
                                                    void *__restrict__ C, int out_dtype)
{
    __shared__ Smem sm;
    __shared__ int scan[256];
    __shared__ int found_e, found_first;
    int64_t gmt, tn;
    const bool in_range = tile_coords(blockIdx.x, max_mtiles, tiles_n, gmt, tn);
    const int t = threadIdx.x;
    if (t == 0) found_e = -1;
    __syncthreads();
    // inclusive scan of per-expert tile counts, 256 experts per round
    int base = 0;
    for (int e0 = 0; e0 < E; e0 += 256) {
        const int e = e0 + t;
        int cnt = 0;
        int64_t unused;
        if (e < E) cnt = (lowp::gemm::expert_rows(m_offsets, e, M_total, unused) + TM - 1) / TM;
        scan[t] = cnt;
        __syncthreads();
        for (int off = 1; off < 256; off <<= 1) {
            int v = t >= off ? scan[t - off] : 0;
            __syncthreads();
            scan[t] += v;
            __syncthreads();
        }
        const int incl = base + scan[t], excl = incl - cnt;
        if (in_range && e < E && gmt >= excl && gmt < incl) { found_e = e; found_first = excl; }
        base += scan[255];
        __syncthreads();
    }
    if (!in_range || found_e < 0) return;
    const int e = found_e;
    int64_t row_begin;
    const int64_t row_end = lowp::gemm::expert_rows(m_offsets, e, M_total, row_begin) + row_begin;
    const int64_t kblocks = K / TK;
    TileArgs ta;
    ta.Aq = Aq; ta.As = As; ta.scale_dtype = scale_dtype;
    ta.Bq = Bq + (int64_t)e * N * K;
    ta.Bs = (const char *)Bs + (int64_t)e * (N / 128) * kblocks * (scale_dtype == LP_F32 ? 4 : 1);
    ta.K = K; ta.kblocks = kblocks;
    ta.m0 = row_begin + (gmt - found_first) * TM; ta.m_end = row_end; ta.n0 = tn * TN;
    ta.kb_begin = 0; ta.kb_end = (int)kblocks;
    Acc acc;
    gemm_tile<SDT>(ta, sm, acc);
    store_tile(acc, ta.m0, row_end, ta.n0, N, C, out_dtype);
}

}  // namespace

// e8m0 scale bytes -> fp32, for the kernels that only read fp32 scales
__global__ __launch_bounds__(256) void scales_to_f32(const uint8_t *__restrict__ a, int64_t na, const uint8_t *__restrict__ b,
                                                     int64_t nb, float *__restrict__ out_a, float *__restrict__ out_b)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < na) out_a[i] = gemm::scale_at<LP_E8M0>(a, i);
    else if (i < na + nb) out_b[i - na] = gemm::scale_at<LP_E8M0>(b, i - na);
}

static int64_t round_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

// fp32 copies of e8m0 scales sit at the start of the workspace (activation scales, then weight scales)
static int64_t scale_copy_bytes(int64_t M, int64_t N, int64_t K)
{
    return M > 64 && K % 512 == 0 ? round_up(M * (K / 128) * 4, 256) + round_up((N / 128) * (K / 128) * 4, 256) : 0;
}

static int64_t split_bytes(int64_t M, int64_t N, int64_t K);

extern "C" int64_t lp_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K)
{
    if (M <= 0 || N <= 0 || K <= 0 || N % 128 || K % 128) return 0;
    return scale_copy_bytes(M, N, K) + split_bytes(M, N, K);
}

static int64_t split_bytes(int64_t M, int64_t N, int64_t K)
{
    // shapes the single-launch decode kernels take never reach the K split
    static const bool no_thin = getenv("LP_GEMM_NO_THIN") != nullptr;
    if (!no_thin && (gemm::thin_ok(M, N, K) || gemm::thin_rows_ok(M, N, K))) return 0;
    static const bool skinny = getenv("LP_GEMM_SKINNY") != nullptr && getenv("LP_GEMM_NO_SKINNY") == nullptr;
    if (M <= 64 && skinny) {
        int sp, per;
        gemm::skinny_plan(N, K, sp, per);
        if (per <= gemm::kSkinnyBlocks) return gemm::skinny_workspace_bytes(N, sp);
    }
    const int64_t tiles = ((M + TM - 1) / TM) * (N / TN);
    const int splits = choose_splits(tiles, K / TK);
    return splits > 1 ? (int64_t)splits * M * N * 4 : 0;
}

static int check_gemm_args(const char *name, const void *Aq, const void *As, const void *Bq, const void *Bs,
                           int scale_dtype, int64_t M, int64_t N, int64_t K, const void *C, int out_dtype)
{
    LP_REQUIRE(scale_dtype == LP_F32 || scale_dtype == LP_E8M0, "%s: scale_dtype must be LP_F32 or LP_E8M0", name);
    LP_REQUIRE(out_dtype == LP_BF16 || out_dtype == LP_F32, "%s: out_dtype must be LP_BF16 or LP_F32", name);
    LP_REQUIRE(M >= 0 && N >= 0 && K >= 0, "%s: negative dimension", name);
    LP_REQUIRE(K % 128 == 0, "%s: K (%lld) must be a multiple of 128", name, (long long)K);
    LP_REQUIRE(N % 128 == 0, "%s: N (%lld) must be a multiple of 128", name, (long long)N);
    if (M == 0 || N == 0) return 1;
    LP_REQUIRE(K > 0, "%s: K must be positive", name);
    LP_REQUIRE(Aq && As && Bq && Bs && C, "%s: null pointer", name);
    LP_REQUIRE((uintptr_t)Aq % 16 == 0 && (uintptr_t)Bq % 16 == 0 && (uintptr_t)C % 16 == 0,
               "%s: operands must be 16-byte aligned", name);
    return LP_OK;
}

// One launch of the 128 x 128 kernel on columns [0, N) of a problem whose C has row stride ldc.
static int launch_small(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M,
                        int64_t N, int64_t K, void *C, int64_t ldc, int out_dtype, hipStream_t st)
{
    static const char *mid_min = getenv("LP_GEMM_MID_MIN_M");       // tuning aid
    if (M >= (mid_min ? atoi(mid_min) : 1) && gemm::mid_asm_ok(As, Bs, scale_dtype, M, N, K))
        return gemm::launch_mid_asm(Aq, As, Bq, Bs, scale_dtype, M, N, K, C, ldc, out_dtype, st);
    const int64_t tiles_m = (M + TM - 1) / TM, tiles_n = N / TN;
    const int64_t grid = padded_grid(tiles_m, tiles_n);
    LP_REQUIRE(grid <= 0x7FFFFFFF, "lp_gemm_fp8_block: problem too large");
    if (scale_dtype == LP_F32)
        hipLaunchKernelGGL(gemm_dense<LP_F32>, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq, As,
                           (const uint8_t *)Bq, Bs, scale_dtype, M, N, K, tiles_m, tiles_n, C, ldc, out_dtype);
    else
        hipLaunchKernelGGL(gemm_dense<LP_E8M0>, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq, As,
                           (const uint8_t *)Bq, Bs, scale_dtype, M, N, K, tiles_m, tiles_n, C, ldc, out_dtype);
    return check_launch("lp_gemm_fp8_block");
}

extern "C" int lp_gemm_fp8_rowscale(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M,
                                    int64_t N, int64_t K, void *C, int out_dtype, lp_stream_t stream)
{
    int rc = check_gemm_args("lp_gemm_fp8_rowscale", Aq, As, Bq, Bs, scale_dtype, M, N, K, C, out_dtype);
    if (rc) return rc > 0 ? LP_OK : rc;
    const int64_t tiles_m = (M + TM - 1) / TM, tiles_n = N / TN;
    const int64_t grid = padded_grid(tiles_m, tiles_n);
    LP_REQUIRE(grid <= 0x7FFFFFFF, "lp_gemm_fp8_rowscale: problem too large");
    hipStream_t st = (hipStream_t)stream;
    // one or two K blocks: the kernel without a K loop (the grouped entry uses it for such problems too: same bits)
    if (scale_dtype == LP_E8M0 && (K == 128 || K == 256) && M % 128 == 0 && N % 128 == 0 && ((uintptr_t)As | (uintptr_t)Bs) % 2 == 0 &&
        ((uintptr_t)Aq | (uintptr_t)Bq) % 16 == 0)
        return gemm::launch_rowscale_small(Aq, As, Bq, Bs, nullptr, 1, (int)(K / 128), M, N, C, out_dtype, st);
    if (gemm::rowscale_asm_ok(As, Bs, scale_dtype, M, N, K)) return gemm::launch_rowscale_asm(Aq, As, Bq, Bs, M, N, K, C, out_dtype, st);
    if (scale_dtype == LP_F32)
        hipLaunchKernelGGL((gemm_dense<LP_F32, true>), dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq, As,
                           (const uint8_t *)Bq, Bs, scale_dtype, M, N, K, tiles_m, tiles_n, C, N, out_dtype);
    else
        hipLaunchKernelGGL((gemm_dense<LP_E8M0, true>), dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq, As,
                           (const uint8_t *)Bq, Bs, scale_dtype, M, N, K, tiles_m, tiles_n, C, N, out_dtype);
    return check_launch("lp_gemm_fp8_rowscale");
}

extern "C" int lp_gemm_fp8_rowscale_grouped(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype,
                                            const int32_t *groups, int G, int max_k_blocks, int k_blocks_multiple, int64_t M, int64_t N,
                                            void *C, int out_dtype, lp_stream_t stream)
{
    LP_REQUIRE(G >= 0 && max_k_blocks >= 0 && k_blocks_multiple >= 1, "lp_gemm_fp8_rowscale_grouped: bad group description");
    if (G == 0 || max_k_blocks == 0) return LP_OK;
    int rc = check_gemm_args("lp_gemm_fp8_rowscale_grouped", Aq, As, Bq, Bs, scale_dtype, M, N, (int64_t)max_k_blocks * 128, C, out_dtype);
    if (rc) return rc > 0 ? LP_OK : rc;
    LP_REQUIRE(groups, "lp_gemm_fp8_rowscale_grouped: null pointer");
    LP_REQUIRE(M % 128 == 0, "lp_gemm_fp8_rowscale_grouped: M (%lld) must be a multiple of 128", (long long)M);
    hipStream_t st = (hipStream_t)stream;
    // problems of exactly one or exactly two K blocks (short experts): no K loop, several workgroups per CU
    if (scale_dtype == LP_E8M0 && (max_k_blocks == 1 || max_k_blocks == 2) && k_blocks_multiple == max_k_blocks && N % 128 == 0 &&
        ((uintptr_t)As | (uintptr_t)Bs) % 2 == 0 && ((uintptr_t)Aq | (uintptr_t)Bq) % 16 == 0)
        return gemm::launch_rowscale_small(Aq, As, Bq, Bs, groups, G, max_k_blocks, M, N, C, out_dtype, st);
    // every problem's K a multiple of 512 (promised by the caller: k_blocks_multiple), e8m0 scales: the hand-scheduled loop
    if (k_blocks_multiple % 4 == 0 && gemm::rowscale_asm_ok(As, Bs, scale_dtype, M, N, (int64_t)max_k_blocks * 128))
        return gemm::launch_rowscale_grouped_asm(Aq, As, Bq, Bs, groups, G, max_k_blocks, M, N, C, out_dtype, st);
    const int64_t tiles_m = M / TM, tiles_n = N / TN;
    const int64_t per_group = padded_grid(tiles_m, tiles_n), grid = per_group * G;
    LP_REQUIRE(grid <= 0x7FFFFFFF, "lp_gemm_fp8_rowscale_grouped: problem too large");
    if (scale_dtype == LP_F32)
        hipLaunchKernelGGL(gemm_rowscale_grouped<LP_F32>, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq, As,
                           (const uint8_t *)Bq, Bs, scale_dtype, groups, M, N, tiles_m, tiles_n, per_group, C, out_dtype, max_k_blocks);
    else
        hipLaunchKernelGGL(gemm_rowscale_grouped<LP_E8M0>, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq, As,
                           (const uint8_t *)Bq, Bs, scale_dtype, groups, M, N, tiles_m, tiles_n, per_group, C, out_dtype, max_k_blocks);
    return check_launch("lp_gemm_fp8_rowscale_grouped");
}

extern "C" int lp_gemm_fp8_block(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype,
                                 int64_t M, int64_t N, int64_t K, void *C, int out_dtype, void *workspace,
                                 int64_t workspace_bytes, lp_stream_t stream)
{
    int rc = check_gemm_args("lp_gemm_fp8_block", Aq, As, Bq, Bs, scale_dtype, M, N, K, C, out_dtype);
    if (rc) return rc > 0 ? LP_OK : rc;
    hipStream_t st = (hipStream_t)stream;
    // e8m0 scales normally go to the kernels whose matrix instructions apply them.  LP_GEMM_E8M0_EXPAND=1 (tuning
    // aid) instead expands them to fp32 in the caller's scratch and runs the fp32-scale kernels.
    static const bool expand = getenv("LP_GEMM_E8M0_EXPAND") != nullptr;
    const int64_t sc_bytes = scale_copy_bytes(M, N, K);
    if (expand && scale_dtype == LP_E8M0 && sc_bytes > 0 && workspace && workspace_bytes >= sc_bytes && (uintptr_t)workspace % 256 == 0) {
        const int64_t na = M * (K / 128), nb = (N / 128) * (K / 128);
        float *fa = (float *)workspace, *fb = (float *)((char *)workspace + round_up(na * 4, 256));
        hipLaunchKernelGGL(scales_to_f32, dim3((unsigned)((na + nb + 255) / 256)), dim3(256), 0, st, (const uint8_t *)As, na,
                           (const uint8_t *)Bs, nb, fa, fb);
        rc = check_launch("lp_gemm_fp8_block(scales)");
        if (rc) return rc;
        return lp_gemm_fp8_block(Aq, fa, Bq, fb, LP_F32, M, N, K, C, out_dtype, (char *)workspace + sc_bytes,
                                 workspace_bytes - sc_bytes, stream);
    }
    // The K-split weight-streaming kernel pair is opt-in (LP_GEMM_SKINNY=1): on every decode shape measured since
    // the single-launch kernels above and the 128-row tile kernel exist it is level with them or behind (two launches).
    static const bool no_skinny = getenv("LP_GEMM_SKINNY") == nullptr || getenv("LP_GEMM_NO_SKINNY") != nullptr;
    static const bool no_thin = getenv("LP_GEMM_NO_THIN") != nullptr;           // tuning aid
    if (!no_thin && gemm::thin_rows_ok(M, N, K)) return gemm::launch_thin_rows(Aq, As, Bq, Bs, scale_dtype, M, N, K, C, out_dtype, st);
    if (!no_thin && gemm::thin_ok(M, N, K)) return gemm::launch_thin(Aq, As, Bq, Bs, scale_dtype, M, N, K, C, out_dtype, st);
    if (M <= 64 && !no_skinny) {
        // decode-sized: the weight-streaming kernel, when the caller gave scratch for its K ranges and one range
        // fits its window of K blocks (longer ranges are better served by the tiled kernels below)
        int sp, per;
        gemm::skinny_plan(N, K, sp, per);
        const bool ws_ok = sp == 1 || (workspace && workspace_bytes >= gemm::skinny_workspace_bytes(N, sp) &&
                                       (uintptr_t)workspace % 16 == 0);
        if (per <= gemm::kSkinnyBlocks && ws_ok)
            return gemm::launch_skinny(Aq, As, Bq, Bs, scale_dtype, M, N, K, C, out_dtype, (float *)workspace, sp, per, st);
    }
    const int64_t tiles_m = (M + TM - 1) / TM, tiles_n = N / TN;
    int splits = choose_splits(tiles_m * tiles_n, K / TK);
    if (splits > 1 && (!workspace || workspace_bytes < (int64_t)splits * M * N * 4 || (uintptr_t)workspace % 16)) splits = 1;
    if (splits > 1) {
        const int kb_all = (int)(K / TK);
        const int per = (kb_all + splits - 1) / splits;
        splits = (kb_all + per - 1) / per;
        if (scale_dtype == LP_F32)
            hipLaunchKernelGGL(gemm_splitk<LP_F32>, dim3((unsigned)(tiles_m * tiles_n * splits)), dim3(256), 0, st, (const uint8_t *)Aq,
                               As, (const uint8_t *)Bq, Bs, scale_dtype, M, N, K, tiles_m, tiles_n, splits, per, (float *)workspace);
        else
            hipLaunchKernelGGL(gemm_splitk<LP_E8M0>, dim3((unsigned)(tiles_m * tiles_n * splits)), dim3(256), 0, st, (const uint8_t *)Aq,
                               As, (const uint8_t *)Bq, Bs, scale_dtype, M, N, K, tiles_m, tiles_n, splits, per, (float *)workspace);
        rc = check_launch("lp_gemm_fp8_block(split-K)");
        if (rc) return rc;
        const int64_t mn = M * N;
        hipLaunchKernelGGL(splitk_reduce, dim3((unsigned)((mn / 4 + 255) / 256)), dim3(256), 0, st, (const float *)workspace,
                           splits, mn, C, out_dtype);
        return check_launch("lp_gemm_fp8_block(reduce)");
    }
    // Prefill-sized problems go to the 256-row kernel.  Its 256 x 256 tiles are dealt to the 256 CUs in
    // rounds; when the last round would be mostly empty, the columns it would cover are given to the
    // 128 x 128 kernel instead, whose smaller tiles fill the machine.
    // LP_GEMM_FORCE_SMALL=1 keeps the 128 x 128 kernel, LP_GEMM_TN forces the big kernel's tile width (tuning aids).
    static const bool force_small = getenv("LP_GEMM_FORCE_SMALL") != nullptr;
    static const char *force_tn = getenv("LP_GEMM_TN");
    const int esz = out_dtype == LP_BF16 ? 2 : 4, ssz = scale_dtype == LP_F32 ? 4 : 1;
    // 256-row tiles from 800 tiles of 128 x 128 on, and already above the 512 that fit the chip at once when the 256-row
    // tiles fill most of one round: more than 192 of them.  With fewer, the 128 x 128 tiles are ahead although they need a
    // second, short round (K = 7168, fp32 / e8m0 scales, us as 256-row tiles -> 128 x 128: 2304 x 4096, 144 big tiles, 96.6
    // -> 87.1 / 83.5 -> 74.7; 2560 x 4096, 160: 92.8 -> 87.4 / 80.2 -> 73.7; 2816 x 4096, 176: 91.1 -> 88.7 / 79.3 -> 75.0; the
    // other way at 1664 x 7168, 196: 86.4 <- 88.9, and 2048 x 7168, 224: 92.2 <- 107.5).
    const int64_t small_tiles = tiles_m * tiles_n, big_tiles = ((M + 255) / 256) * ((N + 255) / 256);
    if (!force_small && M >= 192 && (small_tiles >= 800 || (small_tiles > 512 && big_tiles > 192 && big_tiles <= 256))) {
        if (force_tn) return gemm::launch_big(Aq, As, Bq, Bs, scale_dtype, M, N, K, C, N, out_dtype, atoi(force_tn), st);
        if (gemm::launch_wide(Aq, As, Bq, Bs, scale_dtype, M, N, K, C, N, out_dtype, st, &rc)) return rc;
        const int64_t bm = (M + 255) / 256, bn = (N + 255) / 256, tiles = bm * bn;
        const int64_t full = tiles / 256, rem = tiles % 256;
        int64_t n_big = N;                                   // columns given to the big kernel
        if (full >= 1 && rem > 0 && rem < 160) n_big = (full * 256 / bm) * 256;
        if (n_big > N) n_big = N;
        if (n_big > 0 && n_big < N && gemm::launch_mixed(Aq, As, Bq, Bs, scale_dtype, M, N, K, n_big, C, N, out_dtype, st, &rc)) return rc;
        if (n_big > 0) {
            rc = gemm::launch_big(Aq, As, Bq, Bs, scale_dtype, M, n_big, K, C, N, out_dtype, 256, st);
            if (rc) return rc;
        }
        if (n_big < N)
            return launch_small(Aq, As, (const uint8_t *)Bq + n_big * K, (const char *)Bs + (n_big / 128) * (K / 128) * ssz,
                                scale_dtype, M, N - n_big, K, (char *)C + n_big * esz, N, out_dtype, st);
        return LP_OK;
    }
    return launch_small(Aq, As, Bq, Bs, scale_dtype, M, N, K, C, N, out_dtype, st);
}

extern "C" int lp_gemm_fp8_grouped(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype,
                                   const int32_t *m_offsets, int E, int64_t M_total, int64_t N, int64_t K, void *C,
                                   int out_dtype, lp_stream_t stream)
{
    LP_REQUIRE(E >= 0, "lp_gemm_fp8_grouped: negative expert count");
    int rc = check_gemm_args("lp_gemm_fp8_grouped", Aq, As, Bq, Bs, scale_dtype, M_total, N, K, C, out_dtype);
    if (rc) return rc > 0 ? LP_OK : rc;
    if (E == 0) return LP_OK;
    LP_REQUIRE(m_offsets, "lp_gemm_fp8_grouped: null m_offsets");
    // many rows per expert on average: 256-row tiles on the hand-scheduled kernel
    if (gemm::big_grouped_ok(As, Bs, scale_dtype, M_total, N, K))
        return gemm::launch_big_grouped(Aq, As, Bq, Bs, scale_dtype, m_offsets, E, M_total, N, K, C, out_dtype, (hipStream_t)stream);
    const int64_t max_mtiles = M_total / TM + E, tiles_n = N / TN;
    const int64_t grid = padded_grid(max_mtiles, tiles_n);
    LP_REQUIRE(grid <= 0x7FFFFFFF, "lp_gemm_fp8_grouped: problem too large");
    if (scale_dtype == LP_F32)
        hipLaunchKernelGGL(gemm_grouped<LP_F32>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, (const uint8_t *)Aq, As,
                           (const uint8_t *)Bq, Bs, scale_dtype, m_offsets, E, M_total, N, K, max_mtiles, tiles_n, C, out_dtype);
    else
        hipLaunchKernelGGL(gemm_grouped<LP_E8M0>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, (const uint8_t *)Aq, As,
                           (const uint8_t *)Bq, Bs, scale_dtype, m_offsets, E, M_total, N, K, max_mtiles, tiles_n, C, out_dtype);
    return check_launch("lp_gemm_fp8_grouped");
}

extern "C" int lp_gemm_fp8_grouped_nn(const void *Aq, const void *As, const void *Wq, const void *Ws, int scale_dtype,
                                      const int32_t *m_offsets, int E, int64_t M_total, int64_t N, int64_t K, void *C,
                                      int out_dtype, lp_stream_t stream)
{
    LP_REQUIRE(E >= 0, "lp_gemm_fp8_grouped_nn: negative expert count");
    int rc = check_gemm_args("lp_gemm_fp8_grouped_nn", Aq, As, Wq, Ws, scale_dtype, M_total, N, K, C, out_dtype);
    if (rc) return rc > 0 ? LP_OK : rc;
    if (E == 0) return LP_OK;
    LP_REQUIRE(m_offsets, "lp_gemm_fp8_grouped_nn: null m_offsets");
    LP_REQUIRE(scale_dtype == LP_E8M0, "lp_gemm_fp8_grouped_nn: power-of-two (LP_E8M0) scales only");
    if (!gemm::grouped_nn_ok(As, Ws, scale_dtype, E, M_total, N, K))
        return fail(LP_ERR_UNSUPPORTED,
                    "lp_gemm_fp8_grouped_nn: needs N %% 512 == 0, K %% 512 == 0, 4-byte aligned scale tables, at most 512 experts and "
                    "operands below 4 GiB (got E=%d M=%lld N=%lld K=%lld): transpose the weights and call lp_gemm_fp8_grouped",
                    E, (long long)M_total, (long long)N, (long long)K);
    return gemm::launch_grouped_nn(Aq, As, Wq, Ws, m_offsets, E, M_total, N, K, C, out_dtype, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------------------------
// lp_gemm_fp8_block for callers that cannot allocate device memory: the K-split partial sums go to a buffer that is
// part of the library's device image instead of a caller workspace.  Each GPU the process uses holds its own copy
// of the array at its own address; in host code the array's name is only a handle for hipGetSymbolAddress, so the
// device address is looked up once per device (with that device current) and everything below uses that pointer.
constexpr int64_t kStaticScratchBytes = 32ll << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

extern "C" int64_t lp_gemm_static_scratch_bytes(void) { return kStaticScratchBytes; }

namespace {
constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices];            // device address of `scratch` per device ordinal, nullptr = not looked up yet
pthread_mutex_t g_scratch_lock = PTHREAD_MUTEX_INITIALIZER;

int static_scratch(void **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(LP_ERR_HIP, "lp_gemm_fp8_block_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_block_static: device ordinal %d out of range", dev);
    pthread_mutex_lock(&g_scratch_lock);
    void *p = g_scratch_ptr[dev];
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e == hipSuccess && p) g_scratch_ptr[dev] = p;
    }
    pthread_mutex_unlock(&g_scratch_lock);
    if (e != hipSuccess || !p)
        return fail(LP_ERR_HIP, "lp_gemm_fp8_block_static: hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    *out = p;
    return LP_OK;
}
}  // namespace

extern "C" int lp_gemm_fp8_block_static(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype,
                                        int64_t M, int64_t N, int64_t K, void *C, int out_dtype, lp_stream_t stream)
{
    int rc = check_gemm_args("lp_gemm_fp8_block_static", Aq, As, Bq, Bs, scale_dtype, M, N, K, C, out_dtype);
    if (rc) return rc > 0 ? LP_OK : rc;
    // Only the K-split pair uses scratch (fp32 partial tiles, every one of them written before the reduction reads
    // it, so the buffer's previous contents never matter and nothing is cleared).
    // (decode shapes are served by the single-launch kernels before the K split is considered: no scratch, never refused).
    // The pair is taken for at most 32 tiles of 128 x 128 in at most 16 K ranges: 32 MiB, the buffer's size, so the
    // size test below guards against a dispatcher that changes rather than against any shape of today's.
    const int64_t need = split_bytes(M, N, K);
    LP_REQUIRE(need <= kStaticScratchBytes,
               "lp_gemm_fp8_block_static: M=%lld N=%lld K=%lld needs %lld bytes of K-split scratch, the built-in buffer holds %lld; "
               "call lp_gemm_fp8_block with a workspace of lp_gemm_workspace_bytes()",
               (long long)M, (long long)N, (long long)K, (long long)need, (long long)kStaticScratchBytes);
    void *ws = nullptr;
    if (need > 0) {
        rc = static_scratch(&ws);
        if (rc) return rc;
    }
    return lp_gemm_fp8_block(Aq, As, Bq, Bs, scale_dtype, M, N, K, C, out_dtype, ws, need, stream);
}

