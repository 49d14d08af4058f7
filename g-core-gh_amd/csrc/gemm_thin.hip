// Block-scaled FP8 GEMM for at most 16 activation rows (single-token decode batches) on gfx950.
//
// The problem is one pass over the weights (M = 16, N = 4096, K = 7168: 29 MB against 0.1 MB of activations),
// so the kernel is cut for the memory system rather than for the matrix cores:
//   * a workgroup owns 16 weight rows (16 output columns) over the whole of K, which gives N / 16 workgroups
//     (256 for N = 4096: one per CU) without cutting K across workgroups, so there are no partial tiles to
//     write, no second kernel and no workspace;
//   * its 8 waves take contiguous runs of at most 7 K blocks each.  A wave requests its whole run at once,
//     weights (non-temporal) and activations (served by L2 after the first workgroups), 28 16-byte loads per
//     lane, so every byte the CU needs is in flight within the first few hundred cycles;
//   * the loads land in MFMA operand layout directly: lane (row r = lane % 16, part c = lane / 16) reads bytes
//     [16 c, 16 c + 16) and [64 + 16 c, 64 + 16 c + 16) of its row's 128-byte K block.  That is a permutation
//     of K inside the block compared with the canonical layout, the same one for both operands, and a dot
//     product does not care;
//   * v_mfma_f32_16x16x128_f8f6f4 with a zero C per scale block, folded into the accumulators with As * Bs;
//     the 8 partial sums of a workgroup are added through LDS in wave order (deterministic).
#include "gemm_common.h"

using namespace lowp;

namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4v __attribute__((ext_vector_type(4)));

constexpr int kThinWaves = 8;
constexpr int kThinRun = 7;          // K blocks per wave

template <int SDT, int PER>
__global__ __launch_bounds__(64 * kThinWaves) void gemm_thin(const uint8_t *__restrict__ Aq, const void *__restrict__ As,
                                                             const uint8_t *__restrict__ Bq, const void *__restrict__ Bs,
                                                             int M, int64_t N, int64_t K, void *__restrict__ C, int out_dtype)
{
    constexpr int per = PER;                              // K blocks per wave (compile time: no branch between the loads)
    __shared__ f32x4v red[kThinWaves][64];
    __shared__ float sSa[2 * 64 * kThinWaves];           // activation scales, [row][K block] as in memory (896 used at most)
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);        // uniform, so that the weight scales are scalar loads
    const int l16 = lane & 15, lq = lane >> 4;
    const int kblocks = (int)(K / 128);
    const int64_t n0 = (int64_t)blockIdx.x * 16;
    const int kb0 = wave * per;
    const int m = l16 < M ? l16 : M - 1;                 // rows past M repeat the last one; never stored

    // ---- every request of the wave, oldest first: weights, activations, scales.  Blocks past the end of K
    // repeat the last valid one and get a zero scale below.
    // activation scales: the workgroup copies the [16, kblocks] table with consecutive lanes on consecutive
    // addresses (rows past M repeat the last one) instead of 16-row gathers by every wave
    float sv[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const int i = t + 64 * kThinWaves * q;
        const int last = M * kblocks - 1;
        sv[q] = gemm::scale_at<SDT>(As, i < last ? i : last);
    }
    __builtin_amdgcn_sched_barrier(0);                    // these two stay the oldest requests
    float sb[PER];
    u32x4 a0[PER], a1[PER], b0[PER], b1[PER];
    const uint8_t *ap = Aq + (int64_t)m * K + lq * 16;
    const uint8_t *bp = Bq + (n0 + l16) * K + lq * 16;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
        b0[j] = __builtin_nontemporal_load((const u32x4 *)(bp + (int64_t)kb * 128));
        b1[j] = __builtin_nontemporal_load((const u32x4 *)(bp + (int64_t)kb * 128 + 64));
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
        a0[j] = *(const u32x4 *)(ap + (int64_t)kb * 128);
        a1[j] = *(const u32x4 *)(ap + (int64_t)kb * 128 + 64);
        sb[j] = gemm::scale_at<SDT>(Bs, (n0 >> 7) * kblocks + kb);
    }
    // the staged activation scales were requested first, so writing them to LDS waits for nothing else
#pragma unroll
    for (int q = 0; q < 2; ++q)
        sSa[t + 64 * kThinWaves * q] = sv[q];            // unconditional: a guarded store would pull its load down here
    // keep the scheduler from trading requests in flight for registers: nothing below moves above this line
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    f32x4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
    const f32x4v zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const bool valid = kb0 + j < kblocks;
        const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
        const float s = valid ? sSa[m * kblocks + kb] * sb[j] : 0.0f;
        const i32x8 wf = {(int)b0[j].x, (int)b0[j].y, (int)b0[j].z, (int)b0[j].w, (int)b1[j].x, (int)b1[j].y, (int)b1[j].z, (int)b1[j].w};
        const i32x8 af = {(int)a0[j].x, (int)a0[j].y, (int)a0[j].z, (int)a0[j].w, (int)a1[j].x, (int)a1[j].y, (int)a1[j].z, (int)a1[j].w};
        // rows of the result follow the first operand: p[i] belongs to weight row 4 * (lane / 16) + i, activation row lane % 16
        const f32x4v p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af, zero, 0, 0, 0, 0, 0, 0);
        acc.x = __builtin_fmaf(p.x, s, acc.x);
        acc.y = __builtin_fmaf(p.y, s, acc.y);
        acc.z = __builtin_fmaf(p.z, s, acc.z);
        acc.w = __builtin_fmaf(p.w, s, acc.w);
    }
    red[wave][lane] = acc;
    __syncthreads();
    if (wave != 0 || l16 >= M) return;
    f32x4v sum = red[0][lane];
#pragma unroll
    for (int w = 1; w < kThinWaves; ++w) {
        const f32x4v v = red[w][lane];
        sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
    }
    const int64_t n = n0 + 4 * lq;
    if (out_dtype == LP_BF16) {
        const u32x2 o = {pack_bf16(sum.x, sum.y), pack_bf16(sum.z, sum.w)};
        *(u32x2 *)((uint16_t *)C + (int64_t)l16 * N + n) = o;
    } else {
        *(f32x4v *)((float *)C + (int64_t)l16 * N + n) = sum;
    }
}

}  // namespace

namespace lowp {
namespace gemm {

bool thin_ok(int64_t M, int64_t N, int64_t K)
{
    // one run of K blocks per wave; enough workgroups to cover the chip (fewer are better served by the K-split kernels)
    return M >= 1 && M <= 16 && N % 16 == 0 && K % 128 == 0 && K / 128 <= kThinWaves * kThinRun && N / 16 >= 192 &&
           N / 16 <= 0x7FFFFFFF;
}

template <int SDT, int PER>
void launch_thin_per(const void *Aq, const void *As, const void *Bq, const void *Bs, int64_t M, int64_t N, int64_t K, void *C,
                     int out_dtype, int per, hipStream_t st)
{
    if constexpr (PER > 1) {
        if (per < PER) return launch_thin_per<SDT, PER - 1>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, per, st);
    }
    hipLaunchKernelGGL((gemm_thin<SDT, PER>), dim3((unsigned)(N / 16)), dim3(64 * kThinWaves), 0, st, (const uint8_t *)Aq, As,
                       (const uint8_t *)Bq, Bs, (int)M, N, K, C, out_dtype);
}

int launch_thin(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K,
                void *C, int out_dtype, hipStream_t st)
{
    const int kblocks = (int)(K / 128);
    const int per = (kblocks + kThinWaves - 1) / kThinWaves;
    if (scale_dtype == LP_F32) launch_thin_per<LP_F32, kThinRun>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, per, st);
    else launch_thin_per<LP_E8M0, kThinRun>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, per, st);
    return check_launch("lp_gemm_fp8_block(thin)");
}

}  // namespace gemm
}  // namespace lowp
