// Unscaled C = A B^T with fp32 accumulation, fp8 (e4m3fn) or bf16 operands, for gfx950.
//
// Same data movement as the block-scaled kernels: a K step is 128 bytes of every operand row
// (128 fp8 or 64 bf16 values), copied HBM/L2 -> LDS by global_load_lds_dwordx4 into one of two
// stages, 16-byte chunks XOR-swizzled by row so that both the linear copies and the fragment
// reads are conflict free.  The matrix cores accumulate in place (no scales to fold), so the
// compiler's schedule is adequate here: v_mfma_f32_16x16x128_f8f6f4 for fp8 (one per K step and
// 16 x 16 block), two v_mfma_f32_16x16x32_bf16 for bf16.  The weight fragment is the MFMA A
// operand, the activation fragment the B operand: a lane then holds 4 consecutive output columns
// of one output row, which makes the stores 8 / 16 bytes wide.
#include <pthread.h>
#include <stdlib.h>

#include "gemm_common.h"

using namespace lowp;

namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int KB = 128;             // bytes per operand row and K step

#define LDS_PTR(p) ((void __attribute__((address_space(3))) *)(p))
#define GLB_PTR(p) ((const void __attribute__((address_space(1))) *)(p))

// LDS layout of a stage (rows of 128 bytes), the one of the block-scaled loops: tile row r sits at LDS row lds_row(r) and
// its 16-byte chunk c in slot c ^ (r & 7), so that the 16 lanes of a ds_read_b128 phase (rows l16 and l16 + 8 side by
// side, eight different slots) cover whole 256-byte lines; tile_row is the inverse of lds_row.
__device__ __forceinline__ int lds_row(int r) { return (r & ~15) | ((r & 7) << 1) | ((r >> 3) & 1); }
__device__ __forceinline__ int tile_row(int p) { return (p & ~15) | ((p >> 1) & 7) | ((p & 1) << 3); }
__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ (row & 7); }

// fp32 -> e4m3fn with saturation to +-448 (the conversion a GPU tile compiler emits for an fp8 output
// tile); NaN stays NaN.
__device__ __forceinline__ float sat448(float x)
{
    const float c = __builtin_fminf(__builtin_fmaxf(x, -kE4M3Max), kE4M3Max);
    return x != x ? x : c;
}

// Tile TM x TN, (TM / 64) x 2 waves, a wave owns 64 rows x TN / 2 columns.
template <bool IS_BF16, int TM, int TN>
__global__ __launch_bounds__(TM * 2) void gemm_nt_kernel(const uint8_t *__restrict__ A, const uint8_t *__restrict__ B,
                                                         int64_t M, int64_t N, int64_t row_bytes, int64_t tiles_m,
                                                         int64_t tiles_n, void *__restrict__ C, int out_dtype)
{
    constexpr int WAVES = TM / 64 * 2, NBW = TN / 32;
    constexpr int A_BYTES = TM * KB, B_BYTES = TN * KB, STAGE = A_BYTES + B_BYTES;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[2 * STAGE];

    int64_t tm, tn;
    if (!gemm::tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
    const int64_t m0 = tm * TM, n0 = tn * TN;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l16 = lane & 15, lq = lane >> 4;
    const int ksteps = (int)(row_bytes / KB);

    // copy plan: wave w, instruction i fills LDS rows 8 * (w + WAVES * i) .. + 7 (1 KB) with the tile rows that belong
    // there; rows past the end of a matrix are clamped to its last row (they only feed outputs that are never stored)
    const int ld_row = lane >> 3, ld_slot = lane & 7;
    const uint8_t *a_src[TM / 8 / WAVES];
    const uint8_t *b_src[TN / 8 / WAVES];
#pragma unroll
    for (int i = 0; i < TM / 8 / WAVES; ++i) {
        const int row = tile_row(8 * (wave + WAVES * i) + ld_row);
        const int64_t m = m0 + row < M ? m0 + row : M - 1;
        a_src[i] = A + m * row_bytes + swz(row, ld_slot) * 16;
    }
#pragma unroll
    for (int i = 0; i < TN / 8 / WAVES; ++i) {
        const int row = tile_row(8 * (wave + WAVES * i) + ld_row);
        const int64_t n = n0 + row < N ? n0 + row : N - 1;
        b_src[i] = B + n * row_bytes + swz(row, ld_slot) * 16;
    }
    auto issue_stage = [&](int ks, int stage) {
        uint8_t *sa = smem + stage * STAGE, *sb = sa + A_BYTES;
#pragma unroll
        for (int i = 0; i < TM / 8 / WAVES; ++i)
            __builtin_amdgcn_global_load_lds(GLB_PTR(a_src[i] + (int64_t)ks * KB), LDS_PTR(sa + (wave + WAVES * i) * 1024), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < TN / 8 / WAVES; ++i)
            __builtin_amdgcn_global_load_lds(GLB_PTR(b_src[i] + (int64_t)ks * KB), LDS_PTR(sb + (wave + WAVES * i) * 1024), 16, 0, 0);
    };

    f32x4v acc[4][NBW];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) acc[mb][nb] = f32x4v{0.0f, 0.0f, 0.0f, 0.0f};

    issue_stage(0, 0);
    __syncthreads();

    for (int ks = 0; ks < ksteps; ++ks) {
        const int stage = ks & 1;
        if (ks + 1 < ksteps) issue_stage(ks + 1, stage ^ 1);
        const uint8_t *sa = smem + stage * STAGE, *sb = sa + A_BYTES;
        if constexpr (!IS_BF16) {
            // lane reads 32 bytes (chunks 2 lq, 2 lq + 1) of its row: K bytes 32 lq .. 32 lq + 31
            i32x8 af[4];
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
                const int row = wm * 64 + mb * 16 + l16;
                const u32x4 x0 = *(const u32x4 *)(sa + lds_row(row) * KB + swz(row, 2 * lq) * 16);
                const u32x4 x1 = *(const u32x4 *)(sa + lds_row(row) * KB + swz(row, 2 * lq + 1) * 16);
                af[mb] = i32x8{(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
            }
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) {
                const int row = wn * (TN / 2) + nb * 16 + l16;
                const u32x4 y0 = *(const u32x4 *)(sb + lds_row(row) * KB + swz(row, 2 * lq) * 16);
                const u32x4 y1 = *(const u32x4 *)(sb + lds_row(row) * KB + swz(row, 2 * lq + 1) * 16);
                const i32x8 wf = i32x8{(int)y0.x, (int)y0.y, (int)y0.z, (int)y0.w, (int)y1.x, (int)y1.y, (int)y1.z, (int)y1.w};
#pragma unroll
                for (int mb = 0; mb < 4; ++mb)
                    acc[mb][nb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af[mb], acc[mb][nb], 0, 0, 0, 0, 0, 0);
            }
        } else {
            // two MFMAs of 32 values: lane holds values 8 lq .. 8 lq + 7 of each half (chunk 4 h + lq)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                bf16x8 af[4];
#pragma unroll
                for (int mb = 0; mb < 4; ++mb) {
                    const int row = wm * 64 + mb * 16 + l16;
                    af[mb] = *(const bf16x8 *)(sa + lds_row(row) * KB + swz(row, 4 * h + lq) * 16);
                }
#pragma unroll
                for (int nb = 0; nb < NBW; ++nb) {
                    const int row = wn * (TN / 2) + nb * 16 + l16;
                    const bf16x8 wf = *(const bf16x8 *)(sb + lds_row(row) * KB + swz(row, 4 * h + lq) * 16);
#pragma unroll
                    for (int mb = 0; mb < 4; ++mb)
                        acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, af[mb], acc[mb][nb], 0, 0, 0);
                }
            }
        }
        __syncthreads();      // the next stage has landed and every wave has left this one
    }

    // lane owns row m = .. + l16 and, per block, columns 4 lq .. 4 lq + 3
    const int64_t wcol0 = n0 + wn * (TN / 2);
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
        const int64_t m = m0 + wm * 64 + mb * 16 + l16;
        if (m >= M) continue;
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
            const int64_t n = wcol0 + nb * 16 + 4 * lq;
            if (n >= N) continue;
            const f32x4v v = acc[mb][nb];
            if (out_dtype == LP_BF16) {
                u32x2 o = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
                *(u32x2 *)((uint16_t *)C + m * N + n) = o;
            } else if (out_dtype == LP_F32) {
                u32x4 o = {f2u(v[0]), f2u(v[1]), f2u(v[2]), f2u(v[3])};
                *(u32x4 *)((float *)C + m * N + n) = o;
            } else {
                *(uint32_t *)((uint8_t *)C + m * N + n) = cvt4(sat448(v[0]), sat448(v[1]), sat448(v[2]), sat448(v[3]));
            }
        }
    }
}

template <bool IS_BF16, int TM, int TN>
int launch(const void *A, const void *B, int64_t M, int64_t N, int64_t row_bytes, void *C, int out_dtype, hipStream_t st)
{
    const int64_t tiles_m = (M + TM - 1) / TM, tiles_n = (N + TN - 1) / TN;
    const int64_t grid = gemm::padded_grid(tiles_m, tiles_n);
    if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_nt: problem too large");
    hipLaunchKernelGGL((gemm_nt_kernel<IS_BF16, TM, TN>), dim3((unsigned)grid), dim3(TM * 2), 0, st, (const uint8_t *)A,
                       (const uint8_t *)B, M, N, row_bytes, tiles_m, tiles_n, C, out_dtype);
    return check_launch("lp_gemm_nt");
}

// Unit scales for routing fp8 problems through the block-scaled kernels (below): 1 MiB of e8m0 bytes 0x7F (= 2^0) in the
// library's device image, one copy per GPU, filled by a small kernel at a GPU's first use.  Host code reaches the array
// through the address hipGetSymbolAddress returns for the current device.
constexpr int64_t kUnitScaleBytes = 1 << 20;
__device__ __align__(256) uint8_t unit_scales[kUnitScaleBytes];
constexpr int kMaxDevices = 64;
void *g_unit_ptr[kMaxDevices];               // device address per device ordinal once the array is filled
pthread_mutex_t g_unit_lock = PTHREAD_MUTEX_INITIALIZER;

__global__ __launch_bounds__(256) void fill_bytes(u32x4 *dst, uint32_t word)
{
    dst[(int64_t)blockIdx.x * 256 + threadIdx.x] = u32x4{word, word, word, word};
}

// nullptr when the array cannot be used for this call: device ordinal out of range, a HIP error, or the first use on
// this device falls inside a stream capture (the fill must have run before anything reads the array).
const void *unit_scale_array(hipStream_t st)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    pthread_mutex_lock(&g_unit_lock);
    void *p = g_unit_ptr[dev];
    if (!p) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        void *q = nullptr;
        if (hipStreamIsCapturing(st, &cap) == hipSuccess && cap == hipStreamCaptureStatusNone &&
            hipGetSymbolAddress(&q, HIP_SYMBOL(unit_scales)) == hipSuccess && q) {
            hipLaunchKernelGGL(fill_bytes, dim3((unsigned)(kUnitScaleBytes / 16 / 256)), dim3(256), 0, st, (u32x4 *)q, 0x7F7F7F7Fu);
            // the fill is ordered before this call's kernels on `st`; other streams may only use the array once it is
            // complete, so the address is published after the stream has drained (once per device and process)
            if (hipGetLastError() == hipSuccess && hipStreamSynchronize(st) == hipSuccess) g_unit_ptr[dev] = p = q;
        } else {
            (void)hipGetLastError();
        }
    }
    pthread_mutex_unlock(&g_unit_lock);
    return p;
}

}  // namespace

extern "C" int lp_gemm_nt(const void *A, const void *B, int in_dtype, int64_t M, int64_t N, int64_t K, void *C,
                          int out_dtype, lp_stream_t stream)
{
    LP_REQUIRE(in_dtype == LP_E4M3 || in_dtype == LP_BF16, "lp_gemm_nt: in_dtype must be LP_E4M3 or LP_BF16");
    LP_REQUIRE(out_dtype == LP_E4M3 || out_dtype == LP_BF16 || out_dtype == LP_F32,
               "lp_gemm_nt: out_dtype must be LP_E4M3, LP_BF16 or LP_F32");
    LP_REQUIRE(M >= 0 && N >= 0 && K > 0, "lp_gemm_nt: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    const int64_t esz = in_dtype == LP_BF16 ? 2 : 1;
    LP_REQUIRE((K * esz) % KB == 0, "lp_gemm_nt: K must be a multiple of %d for this operand type (got %lld)",
               (int)(KB / esz), (long long)K);
    LP_REQUIRE(N % 16 == 0, "lp_gemm_nt: N must be a multiple of 16 (got %lld)", (long long)N);
    if (M == 0 || N == 0) return LP_OK;
    LP_REQUIRE(A && B && C, "lp_gemm_nt: null pointer");
    LP_REQUIRE((uintptr_t)A % 16 == 0 && (uintptr_t)B % 16 == 0 && (uintptr_t)C % 16 == 0,
               "lp_gemm_nt: operands must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    // fp8 operands with bf16 or fp32 results, K and N in whole scale blocks: the block-scaled GEMM itself with every scale
    // 2^0 (e8m0 scales are applied inside the matrix instruction at no cost), i.e. its whole choice of kernels by shape --
    // the decode kernels, the hand-scheduled 128 x 128 and 256-row loops -- instead of the compiler-scheduled kernel below.
    // Same bits on every shape compared; one MI355X, us per call, that kernel -> this route: 64 x 4096 x 7168 43.1 -> 12.4,
    // 128 x 4096 x 2048 17.7 -> 9.5, 512 x 1024 x 4096 28.8 -> 15.4, 2048 x 4096 x 1024 15.8 -> 11.7, 1024 x 4096 x 4096 30.5 ->
    // 18.8, 2048 x 4096 x 4096 36.3 -> 30.3, 2048 x 18432 x 1024 49.9 -> 42.4; level from 4096^3 on, where both end in the
    // same loop.  LP_GEMM_NT_PLAIN=1 or LP_GEMM_NT_BLOCK=0 (tuning aids) keep it off.
    static const bool plain_early = getenv("LP_GEMM_NT_PLAIN") != nullptr;
    static const bool via_block = !(getenv("LP_GEMM_NT_BLOCK") && atoi(getenv("LP_GEMM_NT_BLOCK")) == 0);
    if (!plain_early && via_block && in_dtype == LP_E4M3 && out_dtype != LP_E4M3 && K % 128 == 0 && N % 128 == 0 &&
        M * (K / 128) <= kUnitScaleBytes && (N / 128) * (K / 128) <= kUnitScaleBytes) {
        const void *ones = unit_scale_array(st);
        if (ones) return lp_gemm_fp8_block(A, ones, B, ones, LP_E8M0, M, N, K, C, out_dtype, nullptr, 0, stream);
    }
    // e4m3 results (and whatever the route above leaves): K in whole groups of 512, enough tiles: the block-scaled GEMM's hand-scheduled
    // loop with every scale 2^0 (e8m0 scales are applied inside the matrix instruction at no cost), instead of the
    // compiler-scheduled kernel below.  LP_GEMM_NT_PLAIN=1 keeps that one.
    static const bool plain = getenv("LP_GEMM_NT_PLAIN") != nullptr;
    // (N >= 128: the loop indexes weight scales by 128-row block and needs at least one whole block)
    // From the point on where the 128 x 128 tiles of the kernel below no longer fit the chip at once (two workgroups per
    // CU: 512): 2048 x 4096 x 4096, 512 tiles, 36.9 us there against 47.5 on the loop; 2304 x 4096 x 4096, 576 tiles, 58.8
    // against 45.9 (bf16: 99.0 against 80.3).  LP_GEMM_NT_ASM_FROM = n (tuning aid): from n tiles of 128 x 128 instead.
    static const int64_t asm_from = getenv("LP_GEMM_NT_ASM_FROM") ? atoi(getenv("LP_GEMM_NT_ASM_FROM")) : 513;
    const int64_t small_tiles = ((M + 127) / 128) * ((N + 127) / 128);
    if (!plain && in_dtype == LP_E4M3 && K % 512 == 0 && N % 16 == 0 && N >= 128 && small_tiles >= asm_from &&
        M * (K / 128) <= kUnitScaleBytes && ((N + 127) / 128) * (K / 128) <= kUnitScaleBytes) {
        const void *ones = unit_scale_array(st);
        if (ones && gemm::nt_unit_scales_ok(ones, M, N, K)) return gemm::launch_nt_unit_scales(A, B, ones, M, N, K, C, out_dtype, st);
    }
    // bf16 operands on the same loop (two bf16 matrix instructions per fp8 one): K counted in bytes
    if (!plain && in_dtype == LP_BF16 && (2 * K) % 512 == 0 && N % 16 == 0 && N >= 128 && small_tiles >= asm_from &&
        M * (2 * K / 128) <= kUnitScaleBytes && ((N + 127) / 128) * (2 * K / 128) <= kUnitScaleBytes) {
        const void *ones = unit_scale_array(st);
        if (ones && gemm::nt_unit_scales_ok(ones, M, N, 2 * K)) return gemm::launch_nt_unit_scales(A, B, ones, M, N, 2 * K, C, out_dtype, st, true);
    }
    // 256 x 256 tiles once they fill the machine about twice, 128 x 128 otherwise
    // (bf16: from one round of tiles on -- 4096^3, 256 tiles: 127.5 us against 141.5 on 128 x 128 tiles)
    const bool big = M >= 192 && ((M + 255) / 256) * ((N + 255) / 256) >= (in_dtype == LP_BF16 ? 200 : 400);
    if (in_dtype == LP_BF16)
        return big ? launch<true, 256, 256>(A, B, M, N, K * 2, C, out_dtype, st)
                   : launch<true, 128, 128>(A, B, M, N, K * 2, C, out_dtype, st);
    return big ? launch<false, 256, 256>(A, B, M, N, K, C, out_dtype, st)
               : launch<false, 128, 128>(A, B, M, N, K, C, out_dtype, st);
}
