// Row-scaled FP8 GEMM for problems of one or two K blocks: the weight gradients dW_e = dY_e^T X_e of experts with at most
// 256 rows (gpatch_v4/models/deepseek_v4/fp8.py:325-341), which are most experts of a routed batch.  Such a problem is a
// write of M x N results more than a GEMM: a 128 x 128 tile reads 32 KB (or 64 KB) and writes 32 KB of bf16.  No K loop
// and no pipeline inside a workgroup: it requests its whole operand tiles (LDS-direct loads, 8 rows x 128 bytes per
// request), waits once, multiplies with the scale bytes of both operands applied by the matrix cores, stages the results
// through the same LDS and stores whole 128-byte lines.  What overlaps one workgroup's wait and stores is the other
// workgroups of its CU: 36 KB of LDS and 64 accumulators per lane let four of them (one K block) or two (two blocks)
// share it.  LDS rows and chunks are laid out as in gemm_fp8_big.hip (the 16 lanes of a fragment read cover whole
// 256-byte lines).
#include "gemm_common.h"
#include <utility>

using namespace lowp;

namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4v __attribute__((ext_vector_type(4)));

#define LDS_PTR(p) ((void __attribute__((address_space(3))) *)(p))
#define GLB_PTR(p) ((const void __attribute__((address_space(1))) *)(p))

// LDS row that holds tile row r, the tile row an LDS row holds, and the slot of chunk c of tile row r
__device__ __forceinline__ int lds_row(int r) { return (r & ~15) | ((r & 7) << 1) | ((r >> 3) & 1); }
__device__ __forceinline__ int tile_row(int p) { return (p & ~15) | ((p >> 1) & 7) | ((p & 1) << 3); }
__device__ __forceinline__ int swz(int r, int chunk) { return chunk ^ (r & 7); }

// bf16 results of a wave's 64 x 64 sub-tile through LDS: row pitch 128 + 16 bytes, written per accumulator block (mb, nb)
// by lane (l16, lq) -- row 16 mb + l16, columns 16 nb + 4 lq .. + 3 -- and read back in 16-byte chunks of 8 columns, 8
// lanes to a row, so that a store instruction writes 8 whole rows of 128 bytes.
constexpr int kPitch = 64 * 2 + 16, kWaveStage = 64 * kPitch;

// Tried: two to four K blocks passing one after the other through one block's worth of LDS (four workgroups per CU whatever
// the K): the weight gradient of config 4's layer 4.31 ms against 4.21 with both blocks requested at once, and four-block
// problems 4.74 against 4.21 on the hand-scheduled loop.
template <int KBS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(KBS == 1 ? 4 : 2, KBS == 1 ? 4 : 2))) void gemm_rowscale_small(const uint8_t *__restrict__ Aq, const uint8_t *__restrict__ As,
                                                           const uint8_t *__restrict__ Bq, const uint8_t *__restrict__ Bs,
                                                           const int32_t *__restrict__ groups, int64_t M, int64_t N, int64_t tiles_m,
                                                           int64_t tiles_n, int64_t per_group, void *__restrict__ C, int out_dtype)
{
    constexpr int TILE = 128 * 128, OPER = KBS * TILE, PITCH = KBS * 128;
    constexpr int LDS_BYTES = 2 * OPER > 4 * kWaveStage ? 2 * OPER : 4 * kWaveStage;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[LDS_BYTES];
    const int64_t g = blockIdx.x / per_group, local = blockIdx.x - g * per_group;
    int64_t tm, tn;
    if (!gemm::tile_coords(local, tiles_m, tiles_n, tm, tn)) return;
    // no table: one problem of KBS blocks
    const int64_t slot = groups ? groups[4 * g] : 0, kb = groups ? groups[4 * g + 1] : KBS, before = groups ? groups[4 * g + 2] : 0;
    // an entry of another size (or one that breaks the caller's promises) is not this launch's: nothing is written
    if (kb != KBS || slot < 0 || before < 0) return;
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave >> 1, wn = wave & 1, l16 = lane & 15, lq = lane >> 4;
    const int64_t m0 = tm * 128, n0 = tn * 128;
    const uint8_t *a_g = Aq + M * 128 * before + m0 * PITCH, *b_g = Bq + N * 128 * before + n0 * PITCH;
    const uint8_t *as_g = As + M * before + m0 * KBS, *bs_g = Bs + N * before + n0 * KBS;

    // requests: group q of 8 LDS rows of an operand block is wave q % 4's; lane -> row lane / 8 of the group, slot lane % 8
    const int ld_row = lane >> 3, ld_slot = lane & 7;
    uint32_t off[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = tile_row(8 * (wave + 4 * i) + ld_row);
        off[i] = (uint32_t)(row * PITCH + swz(row, ld_slot) * 16);
    }
    auto request = [&](int j, int buf) {                 // K block j of both operands into block buffer buf
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int q = wave + 4 * i;
            __builtin_amdgcn_global_load_lds(GLB_PTR(a_g + off[i] + j * 128), LDS_PTR(smem + buf * TILE + q * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds(GLB_PTR(b_g + off[i] + j * 128), LDS_PTR(smem + OPER + buf * TILE + q * 1024), 16, 0, 0);
        }
    };
#pragma unroll
    for (int j = 0; j < KBS; ++j) request(j, j);
    // scale bytes of the lane's rows: byte j of the register = K block j (picked by the instruction's op_sel)
    int sa[4], sb[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const int ra = wm * 64 + b * 16 + l16, rb = wn * 64 + b * 16 + l16;
        if (KBS == 1) { sa[b] = as_g[ra]; sb[b] = bs_g[rb]; }
        else { sa[b] = *(const uint16_t *)(as_g + 2 * ra); sb[b] = *(const uint16_t *)(bs_g + 2 * rb); }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    f32x4v acc[4][4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) acc[mb][nb] = f32x4v{0.0f, 0.0f, 0.0f, 0.0f};
    auto frag = [&](const uint8_t *base, int row) -> i32x8 {
        const u32x4 x0 = *(const u32x4 *)(base + lds_row(row) * 128 + swz(row, 2 * lq) * 16);
        const u32x4 x1 = *(const u32x4 *)(base + lds_row(row) * 128 + swz(row, 2 * lq + 1) * 16);
        return i32x8{(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
    };
    auto block = [&](auto jc) {
        constexpr int j = decltype(jc)::value, buf = j;
        // fragments are read where they are used (the activation side four times over): registers for four workgroups per CU
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
            const i32x8 bf = frag(smem + OPER + buf * TILE, wn * 64 + nb * 16 + l16);
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
                const i32x8 af = frag(smem + buf * TILE, wm * 64 + mb * 16 + l16);
                acc[mb][nb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf, af, acc[mb][nb], 0, 0, j, sb[nb], j, sa[mb]);
            }
        }
    };
    block(std::integral_constant<int, 0>{});
    if constexpr (KBS == 2) block(std::integral_constant<int, 1>{});

    const int64_t row0 = m0 + wm * 64, col0 = n0 + wn * 64;
    char *c_g = (char *)C + slot * M * N * (out_dtype == LP_BF16 ? 2 : 4);
    if (out_dtype == LP_BF16) {
        __syncthreads();                                 // every wave has read its fragments: the tile memory is free
        uint8_t *stage = smem + wave * kWaveStage;
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
                const u32x2 o = {pack_bf16(acc[mb][nb].x, acc[mb][nb].y), pack_bf16(acc[mb][nb].z, acc[mb][nb].w)};
                *(u32x2 *)(stage + (mb * 16 + l16) * kPitch + (nb * 16 + 4 * lq) * 2) = o;
            }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // a wave reads back only what it wrote
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            const int row = p * 8 + (lane >> 3), chunk = lane & 7;
            const u32x4 v = *(const u32x4 *)(stage + row * kPitch + chunk * 16);
            __builtin_nontemporal_store(v, (u32x4 *)((uint16_t *)c_g + (row0 + row) * N + col0 + chunk * 8));
        }
        return;
    }
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
            const u32x4 o = {f2u(acc[mb][nb].x), f2u(acc[mb][nb].y), f2u(acc[mb][nb].z), f2u(acc[mb][nb].w)};
            *(u32x4 *)((float *)c_g + (row0 + mb * 16 + l16) * N + col0 + nb * 16 + 4 * lq) = o;
        }
}

}  // namespace

namespace lowp {
namespace gemm {

// Every entry of `groups` has k_blocks K blocks (1 or 2): e8m0 scales, M and N multiples of 128.  groups == nullptr: one
// problem (G = 1) written at C.
int launch_rowscale_small(const void *Aq, const void *As, const void *Bq, const void *Bs, const int32_t *groups, int G, int k_blocks,
                          int64_t M, int64_t N, void *C, int out_dtype, hipStream_t st)
{
    const int64_t tiles_m = M / 128, tiles_n = N / 128;
    const int64_t per_group = padded_grid(tiles_m, tiles_n), grid = per_group * G;
    if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_rowscale_grouped: problem too large");
    auto go = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq, (const uint8_t *)As, (const uint8_t *)Bq,
                           (const uint8_t *)Bs, groups, M, N, tiles_m, tiles_n, per_group, C, out_dtype);
    };
    if (k_blocks == 1) go(gemm_rowscale_small<1>);
    else go(gemm_rowscale_small<2>);
    return check_launch("lp_gemm_fp8_rowscale_grouped(small K)");
}

}  // namespace gemm
}  // namespace lowp
