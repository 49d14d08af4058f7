// Decode-sized block-scaled FP8 GEMM (at most 64 activation rows) for gfx950: a weight-streaming kernel.
//
// With so few rows the problem is the HBM read of the weights (M = 64, N = 4096, K = 7168: 29 MB of weights
// against 0.5 MB of activations), so the kernel is built around getting every CU's share of the weight bytes
// in flight at once:
//   * a workgroup (4 waves) owns 128 weight rows x up to 7 K blocks of 128; each wave's 32 rows x 7 blocks go
//     from HBM into VGPRs with non-temporal 16-byte loads, four blocks (16 loads per lane) ahead of the block
//     being multiplied, which keeps about 64 KB per CU in flight without parking the waves in the issue queue
//     (requesting the whole share up front leaves the arithmetic of all blocks for after the stream).  The loads are laid out
//     for the memory system (8 lanes cover one 128-byte row segment); each block is then turned into MFMA
//     fragments (a lane needs 32 bytes of one row) through a small wave-private LDS buffer, without barriers;
//   * the activations of those K blocks (64 rows, 56 KB, served by L2 after the first workgroup) and their
//     scales are requested first, staged through LDS (XOR-swizzled 16-byte chunks) and shared by the waves;
//   * K is cut into contiguous ranges so that there is at least one workgroup per CU; each range writes an fp32
//     partial tile to the workspace and the ranges are added in a fixed order by splitk_reduce (deterministic).
// The matrix cores do the arithmetic (v_mfma_f32_16x16x128_f8f6f4, zero C per scale block, result folded into
// the accumulators with As * Bs); at this size they are idle most of the time.
#include "gemm_common.h"

using namespace lowp;

namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4v __attribute__((ext_vector_type(4)));

constexpr int JB = lowp::gemm::kSkinnyBlocks;    // K blocks per workgroup and round
constexpr int KB = 128;
constexpr int DEPTH = 4;            // weight blocks requested ahead of the one being multiplied

__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row >> 1) & 7); }

template <int SDT>
__global__ __launch_bounds__(256) void gemm_skinny(const uint8_t *__restrict__ Aq, const void *__restrict__ As,
                                                   const uint8_t *__restrict__ Bq, const void *__restrict__ Bs, int M,
                                                   int64_t N, int64_t K, int n_tiles, int per, float *__restrict__ ws,
                                                   void *__restrict__ C, int out_dtype)
{
    __shared__ __attribute__((aligned(1024))) uint8_t sA[JB * 64 * KB];
    __shared__ float sS[512];                    // JB x 64 scales, padded so that every thread writes
    __shared__ __attribute__((aligned(1024))) uint8_t sW[4][2][32 * KB];      // per wave: two blocks of 32 weight rows

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l16 = lane & 15, lq = lane >> 4;
    const int tn = blockIdx.x % n_tiles, split = blockIdx.x / n_tiles;
    const int kblocks = (int)(K / KB);
    const int kb_begin = split * per;
    const int kb_end = kb_begin + per < kblocks ? kb_begin + per : kblocks;
    const int64_t n_base = (int64_t)tn * 128 + wave * 32;

    f32x4v acc[4][2];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) acc[mb][nb] = f32x4v{0.0f, 0.0f, 0.0f, 0.0f};
    const f32x4v zero = {0.0f, 0.0f, 0.0f, 0.0f};

    for (int kb0 = kb_begin; kb0 < kb_end; kb0 += JB) {
        const int nblk = kb_end - kb0 < JB ? kb_end - kb0 : JB;
        // ---- requests, oldest first: weight scales (uniform), activation scales, activations, weights.
        // Blocks past the end of the range repeat the last valid one (loaded, never used).
        float bs[JB];
#pragma unroll
        for (int j = 0; j < JB; ++j)
            bs[j] = gemm::scale_at<SDT>(Bs, (int64_t)tn * kblocks + kb0 + (j < nblk ? j : nblk - 1));
        float sv[2];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int idx = t + 256 * q, j = idx & 7, row = idx >> 3;            // j = 7 is padding
            const int jj = j < nblk ? j : nblk - 1, rr = row < M ? row : M - 1;
            sv[q] = gemm::scale_at<SDT>(As, (int64_t)rr * kblocks + kb0 + jj);
        }
        u32x4 av[14];
#pragma unroll
        for (int i = 0; i < 14; ++i) {
            const int c = t + 256 * i, j = c >> 9, row = (c >> 3) & 63, slot = c & 7;
            const int jj = j < nblk ? j : nblk - 1, rr = row < M ? row : M - 1;
            av[i] = *(const u32x4 *)(Aq + (int64_t)rr * K + (int64_t)(kb0 + jj) * KB + slot * 16);
        }
        u32x4 w[JB][4];                             // block j, rows 8 i + lane / 8 of the wave's 32, chunk lane % 8
        auto request = [&](int j) {
            const int jj = j < nblk ? j : nblk - 1;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                w[j][i] = __builtin_nontemporal_load(
                    (const u32x4 *)(Bq + (n_base + 8 * i + (lane >> 3)) * K + (int64_t)(kb0 + jj) * KB + (lane & 7) * 16));
        };
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) request(j);
        __builtin_amdgcn_sched_barrier(0);          // everything above is issued before anything below

        // ---- stage activations and their scales for the four waves
#pragma unroll
        for (int q = 0; q < 2; ++q)
            sS[((t + 256 * q) & 7) * 64 + ((t + 256 * q) >> 3)] = sv[q];
#pragma unroll
        for (int i = 0; i < 14; ++i) {
            const int c = t + 256 * i, j = c >> 9, row = (c >> 3) & 63, slot = c & 7;
            *(u32x4 *)(sA + j * 64 * KB + row * KB + swz(row, slot) * 16) = av[i];
        }
        // LDS writes done, then barrier; the weight loads stay in flight (no wait on the vector-memory counter)
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);

        // ---- arithmetic, one scale block at a time as its weights arrive.  No branches here (the compiler
        // would sink the weight loads into them): blocks past the end of the range get a zero scale.
#pragma unroll
        for (int j = 0; j < JB; ++j) {
            const uint8_t *sa = sA + j * 64 * KB;
            const float bsj = j < nblk ? bs[j] : 0.0f;
            // weights of this block: registers -> wave-private LDS -> fragments (in-order within the wave)
            uint8_t *sw = sW[wave][j & 1];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = 8 * i + (lane >> 3);
                *(u32x4 *)(sw + row * KB + swz(row, lane & 7) * 16) = w[j][i];
            }
            i32x8 wf[2];
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                const int row = nb * 16 + l16;
                const u32x4 y0 = *(const u32x4 *)(sw + row * KB + swz(row, 2 * lq) * 16);
                const u32x4 y1 = *(const u32x4 *)(sw + row * KB + swz(row, 2 * lq + 1) * 16);
                wf[nb] = i32x8{(int)y0.x, (int)y0.y, (int)y0.z, (int)y0.w, (int)y1.x, (int)y1.y, (int)y1.z, (int)y1.w};
            }
            i32x8 af[4];
            float sc[4];
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
                const int row = mb * 16 + l16;
                const u32x4 x0 = *(const u32x4 *)(sa + row * KB + swz(row, 2 * lq) * 16);
                const u32x4 x1 = *(const u32x4 *)(sa + row * KB + swz(row, 2 * lq + 1) * 16);
                af[mb] = i32x8{(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
                sc[mb] = sS[j * 64 + row] * bsj;
            }
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int mb = 0; mb < 4; ++mb) {
                    const f32x4v p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[nb], af[mb], zero, 0, 0, 0, 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[mb][nb][r] = __builtin_fmaf(p[r], sc[mb], acc[mb][nb][r]);
                }
            // keep the window full: the requests of a later block go out between the math of two blocks, so the
            // wave is never stuck issuing its whole share while data it could already multiply sits in registers
            __builtin_amdgcn_sched_barrier(0);
            if (j + DEPTH < JB) request(j + DEPTH);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (kb0 + JB < kb_end) __syncthreads();     // the next round overwrites the staged activations
    }

    // lane owns activation row mb * 16 + l16 and weight rows n_base + nb * 16 + 4 lq .. + 3
    if (ws != nullptr) {
        // partial sums go to the workspace in the order the lanes hold them, [split][tile][wave][mb][nb][lane] x 4
        // floats: every store instruction writes 1 KB of consecutive bytes (row-major partial tiles would be
        // written in 64-byte pieces).  skinny_reduce reads them back the same way.
        float *part = ws + (((int64_t)split * n_tiles + tn) * 4 + wave) * (8 * 256);
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                const f32x4v v = acc[mb][nb];
                u32x4 o = {f2u(v[0]), f2u(v[1]), f2u(v[2]), f2u(v[3])};
                __builtin_nontemporal_store(o, (u32x4 *)(part + (mb * 2 + nb) * 256 + lane * 4));
            }
        return;
    }
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
        const int m = mb * 16 + l16;
        if (m >= M) continue;
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const int64_t n = n_base + nb * 16 + 4 * lq;
            const f32x4v v = acc[mb][nb];
            if (out_dtype == LP_F32) {
                u32x4 o = {f2u(v[0]), f2u(v[1]), f2u(v[2]), f2u(v[3])};
                *(u32x4 *)((float *)C + (int64_t)m * N + n) = o;
            } else {
                u32x2 o = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
                *(u32x2 *)((uint16_t *)C + (int64_t)m * N + n) = o;
            }
        }
    }
}

// Adds the K ranges in a fixed order and writes C.  One thread per (tile, wave, mb, nb, lane) group of 4 values.
__global__ __launch_bounds__(256) void skinny_reduce(const float *__restrict__ ws, int splits, int n_tiles, int M, int64_t N,
                                                     void *__restrict__ C, int out_dtype)
{
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;          // group index inside one split
    const int64_t per_split = (int64_t)n_tiles * 4 * 8 * 64;
    if (g >= per_split) return;
    f32x4 s = *(const f32x4 *)(ws + g * 4);
    for (int k = 1; k < splits; ++k) {
        const f32x4 v = *(const f32x4 *)(ws + ((int64_t)k * per_split + g) * 4);
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    const int lane = (int)(g & 63), nb = (int)((g >> 6) & 1), mb = (int)((g >> 7) & 3), wave = (int)((g >> 9) & 3);
    const int64_t tn = g >> 11;
    const int m = mb * 16 + (lane & 15);
    if (m >= M) return;
    const int64_t n = tn * 128 + wave * 32 + nb * 16 + 4 * (lane >> 4);
    if (out_dtype == LP_BF16) {
        u32x2 o = {pack_bf16(s.x, s.y), pack_bf16(s.z, s.w)};
        *(u32x2 *)((uint16_t *)C + (int64_t)m * N + n) = o;
    } else {
        *(f32x4 *)((float *)C + (int64_t)m * N + n) = s;
    }
}

}  // namespace

namespace lowp {
namespace gemm {

// K ranges for the skinny kernel: at least one workgroup per CU when K allows it.
void skinny_plan(int64_t N, int64_t K, int &splits, int &per)
{
    const int n_tiles = (int)(N / 128), kblocks = (int)(K / KB);
    int s = (256 + n_tiles - 1) / n_tiles;
    if (s > kblocks) s = kblocks;
    if (s < 1) s = 1;
    per = (kblocks + s - 1) / s;
    splits = (kblocks + per - 1) / per;
}

int64_t skinny_workspace_bytes(int64_t N, int splits) { return splits > 1 ? (int64_t)splits * (N / 128) * 8192 * 4 : 0; }

int launch_skinny(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N,
                  int64_t K, void *C, int out_dtype, float *ws, int splits, int per, hipStream_t st)
{
    const int n_tiles = (int)(N / 128);
    const int64_t grid = (int64_t)n_tiles * splits;
    if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_block: problem too large");
    if (scale_dtype == LP_F32)
        hipLaunchKernelGGL(gemm_skinny<LP_F32>, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq, As,
                           (const uint8_t *)Bq, Bs, (int)M, N, K, n_tiles, per, splits > 1 ? ws : nullptr, C, out_dtype);
    else
        hipLaunchKernelGGL(gemm_skinny<LP_E8M0>, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq, As,
                           (const uint8_t *)Bq, Bs, (int)M, N, K, n_tiles, per, splits > 1 ? ws : nullptr, C, out_dtype);
    int rc = check_launch("lp_gemm_fp8_block(skinny)");
    if (rc || splits == 1) return rc;
    const int64_t groups = (int64_t)n_tiles * 2048;
    hipLaunchKernelGGL(skinny_reduce, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, st, (const float *)ws, splits,
                       n_tiles, (int)M, N, C, out_dtype);
    return check_launch("lp_gemm_fp8_block(skinny reduce)");
}

}  // namespace gemm
}  // namespace lowp
