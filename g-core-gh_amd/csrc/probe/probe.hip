// The measurement and test aids of include/lowp_probe.h, built into a library of their own (liblowp_probe.so):
// on-device checks of the gfx950 conversion instructions against the software casts in lowp_math.h, bulk casts
// used by tests, and the bare-stream / matrix-pipe / copy-path probes the benchmark times beside the kernels.
#include "../lowp_device.h"
#include "../../../include/lowp_probe.h"

using namespace lowp;

namespace lowp {
// this library's own message buffer (the product library has its own behind lp_last_error)
char *error_buffer()
{
    static thread_local char buf[kErrorBufferSize] = {0};
    return buf;
}
}  // namespace lowp

extern "C" const char *lp_probe_last_error(void) { return lowp::error_buffer(); }

namespace {

__device__ __forceinline__ void count(uint64_t *out, bool bad)
{
    unsigned long long b = __ballot(bad);
    if ((threadIdx.x & 63) == 0 && b) atomicAdd((unsigned long long *)out, (unsigned long long)__popcll(b));
}

// which 0: every fp32 pattern; patterns with |x| > 464 (or NaN) are skipped
// (448 < |x| <= 464 must round down to 448, which is what lets kernels skip a clamp)
__global__ __launch_bounds__(256) void st_cvt_fp8(uint64_t *out)
{
    const uint32_t base = (blockIdx.x * 256u + threadIdx.x) * 16u;
    bool bad = false;
    for (uint32_t i = 0; i < 16u; i += 2) {
        uint32_t u0 = base + i, u1 = base + i + 1;
        float a = u2f(u0), b = u2f(u1);
        bool ok0 = (u0 & 0x7FFFFFFFu) <= 0x43E80000u, ok1 = (u1 & 0x7FFFFFFFu) <= 0x43E80000u;
        int w = __builtin_amdgcn_cvt_pk_fp8_f32(ok0 ? a : 0.0f, ok1 ? b : 0.0f, 0, false);
        int w2 = __builtin_amdgcn_cvt_pk_fp8_f32(ok1 ? b : 0.0f, ok0 ? a : 0.0f, 0, true);
        if (ok0) bad |= (uint8_t)w != sw_f32_to_e4m3fn(a) || (uint8_t)(w2 >> 24) != sw_f32_to_e4m3fn(a);
        if (ok1) bad |= (uint8_t)(w >> 8) != sw_f32_to_e4m3fn(b) || (uint8_t)(w2 >> 16) != sw_f32_to_e4m3fn(b);
    }
    count(out, bad);
}

// which 1: 256 codes through all four byte positions
__global__ __launch_bounds__(256) void st_cvt_from_fp8(uint64_t *out)
{
    const uint32_t c = threadIdx.x;
    bool bad = false;
    if ((c & 0x7Fu) != 0x7Fu) {
        uint32_t w = c | ((c ^ 0x55u) << 8) | (c << 16) | ((c ^ 0x33u) << 24);
        f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
        f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
        bad |= f2u(lo.x) != f2u(sw_e4m3fn_to_f32((uint8_t)c));
        bad |= f2u(hi.x) != f2u(sw_e4m3fn_to_f32((uint8_t)c));
        uint32_t c1 = c ^ 0x55u, c3 = c ^ 0x33u;
        if ((c1 & 0x7Fu) != 0x7Fu) bad |= f2u(lo.y) != f2u(sw_e4m3fn_to_f32((uint8_t)c1));
        if ((c3 & 0x7Fu) != 0x7Fu) bad |= f2u(hi.y) != f2u(sw_e4m3fn_to_f32((uint8_t)c3));
    }
    count(out, bad);
}

// which 2: packed fp32 -> bf16 over every non-NaN fp32
__global__ __launch_bounds__(256) void st_cvt_bf16(uint64_t *out)
{
    const uint32_t base = (blockIdx.x * 256u + threadIdx.x) * 16u;
    bool bad = false;
    for (uint32_t i = 0; i < 16u; i += 2) {
        uint32_t u0 = base + i, u1 = base + i + 1;
        bool ok0 = (u0 & 0x7FFFFFFFu) <= 0x7F800000u, ok1 = (u1 & 0x7FFFFFFFu) <= 0x7F800000u;
        uint32_t p = pack_bf16(ok0 ? u2f(u0) : 0.0f, ok1 ? u2f(u1) : 0.0f);
        if (ok0) bad |= (p & 0xFFFFu) != sw_f32_to_bf16(u2f(u0));
        if (ok1) bad |= (p >> 16) != sw_f32_to_bf16(u2f(u1));
    }
    count(out, bad);
}

// which 3: every packed byte in every byte position, scale operand 1.0
__global__ __launch_bounds__(256) void st_cvt_fp4(uint64_t *out)
{
    const uint32_t b = threadIdx.x;
    bool bad = false;
    for (int pos = 0; pos < 4; ++pos) {
        uint32_t w = (b << (8 * pos)) | (0xA5C3961Eu & ~(0xFFu << (8 * pos)));
        float v[8];
        fp4_decode8(w, v);
        bad |= f2u(v[2 * pos]) != f2u(sw_e2m1_to_f32(b & 0xFu, true));
        bad |= f2u(v[2 * pos + 1]) != f2u(sw_e2m1_to_f32(b >> 4, true));
        float z[8];
        fp4_decode8(fp4_pos_zero(w), z);
        bad |= f2u(z[2 * pos]) != f2u(sw_e2m1_to_f32(b & 0xFu, false));
        bad |= f2u(z[2 * pos + 1]) != f2u(sw_e2m1_to_f32(b >> 4, false));
    }
    count(out, bad);
}

// self test: hardware conversion with the tie adjustment == software rounding, every finite fp32, three scales
__global__ __launch_bounds__(256) void st_cvt_to_fp4(uint64_t *out)
{
    const uint32_t base = (blockIdx.x * 256u + threadIdx.x) * 16u;
    bool bad = false;
    for (int k = 0; k < 3; ++k) {
        const int e = k == 0 ? 0 : (k == 1 ? -7 : 9);
        const uint32_t eb = (uint32_t)e << 23;
        const uint32_t t0 = 0x3F400000u + eb, t1 = 0x3FE00000u + eb, t2 = 0x40600000u + eb;
        const float s = u2f((uint32_t)(e + 127) << 23);
        for (uint32_t i = 0; i < 16u; i += 2) {
            uint32_t b0 = base + i, b1 = base + i + 1;
            const uint32_t a0 = b0 & 0x7FFFFFFFu, a1 = b1 & 0x7FFFFFFFu;
            const bool ok0 = a0 < 0x7F800000u, ok1 = a1 < 0x7F800000u;
            const uint32_t want0 = sw_f32_to_e2m1_half_down(u2f(b0) / s), want1 = sw_f32_to_e2m1_half_down(u2f(b1) / s);
            b0 -= (a0 == t0) | (a0 == t1) | (a0 == t2);
            b1 -= (a1 == t0) | (a1 == t1) | (a1 == t2);
            const uint32_t w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(0u, ok0 ? u2f(b0) : 0.0f, ok1 ? u2f(b1) : 0.0f, s, 0);
            if (ok0) bad |= (w & 15u) != want0;
            if (ok1) bad |= ((w >> 4) & 15u) != want1;
        }
    }
    unsigned long long b = __ballot(bad);
    if ((threadIdx.x & 63) == 0 && b) atomicAdd((unsigned long long *)out, (unsigned long long)__popcll(b));
}

__global__ __launch_bounds__(256) void debug_cast(int kind, const float *__restrict__ x, void *__restrict__ out, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        float v = x[i];
        if (kind == 0) ((uint8_t *)out)[i] = sw_f32_to_e4m3fn(v);
        else if (kind == 1) ((uint8_t *)out)[i] = (uint8_t)__builtin_amdgcn_cvt_pk_fp8_f32(clamp448(v), 0.0f, 0, false);
        else if (kind == 2) ((uint8_t *)out)[i] = f32_to_e8m0(v);
        else if (kind == 3) ((uint16_t *)out)[i] = sw_f32_to_bf16(v);
        else if (kind == 4) ((uint8_t *)out)[i] = (uint8_t)__builtin_amdgcn_cvt_scalef32_pk_fp4_f32(0u, v, v, 1.0f, 0);
        else ((uint8_t *)out)[i] = (uint8_t)__builtin_amdgcn_cvt_scalef32_pk_fp4_f32(0u, v, v, 4.0f, 0);
    }
}

// Stream probe: each of the launch's workgroups reads a contiguous share of `src` with 16-byte non-temporal loads
// (all lanes of a wave on consecutive addresses, 8 loads in flight per lane) and writes a share of `dst` with 16-byte
// stores whose value depends on what was read, so neither side can be dropped.  No arithmetic to speak of: what
// it takes is what the memory system and the launch take for that many bytes.
__global__ __launch_bounds__(256) void stream_probe(const u32x4 *__restrict__ src, int64_t read_vecs, u32x4 *__restrict__ dst,
                                                    int64_t write_vecs)
{
    const int64_t wgs = gridDim.x, wg = blockIdx.x;
    const int64_t r_per = (read_vecs + wgs - 1) / wgs, w_per = (write_vecs + wgs - 1) / wgs;
    const int64_t r0 = wg * r_per, r1 = r0 + r_per < read_vecs ? r0 + r_per : read_vecs;
    u32x4 acc = {0u, 0u, 0u, 0u};
    for (int64_t i = r0 + threadIdx.x; i < r1; i += 256 * 8) {
        u32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = i + 256 * j < r1 ? __builtin_nontemporal_load(src + i + 256 * j) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < 8; ++j) { acc.x ^= v[j].x; acc.y ^= v[j].y; acc.z ^= v[j].z; acc.w ^= v[j].w; }
    }
    const int64_t w0 = wg * w_per, w1 = w0 + w_per < write_vecs ? w0 + w_per : write_vecs;
    for (int64_t i = w0 + threadIdx.x; i < w1; i += 256) {
        acc.x += 1u;
        __builtin_nontemporal_store(acc, dst + i);
    }
}

// Matrix-pipe probe: the fp8 16x16x128 matrix instruction in a register-only loop, FMAS fp32 FMAs after each (0, 2, 4, 6
// or 8: the fp32-scaled GEMM loops fold with four), eight waves per workgroup = two per SIMD, no LDS and no memory traffic
// inside the loop.  The operand registers v[0:15] hold 64 bytes per lane from `operands` (e4m3 codes), or zeros.  What it
// takes is what the chip's clock under that arithmetic allows: the ceiling of any kernel built from these instructions.
#define LP_PROBE_CLOBBERS                                                                                                       \
    "v0", "v1", "v2", "v3", "v4", "v5", "v6", "v7", "v8", "v9", "v10", "v11", "v12", "v13", "v14", "v15", "v20", "v32", "v33", "v34", "v35",   \
        "v36", "v37", "v38", "v39", "v40", "v41", "v42", "v43", "v44", "v45", "v46", "v47", "v48", "v49", "v50", "v51", "v52", "v53", "v54",   \
        "v55", "v56", "v57", "v58", "v59", "v60", "v61", "v62", "v63", "v64", "v65", "v66", "v67", "v68", "v69", "v70", "v71", "v72", "v73",   \
        "v74", "v75", "v76", "v77", "v78", "v79", "v80", "v81", "v82", "v83", "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92",   \
        "v93", "v94", "v95", "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109",      \
        "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123", "v124", "v125",     \
        "v126", "v127"
template <int FMAS>
__global__ __launch_bounds__(512) void probe_mfma(const uint8_t *__restrict__ operands, int iters)
{
    const uint8_t *p = operands + (size_t)(threadIdx.x & 63) * 64;
    if (operands != nullptr)
        asm volatile("global_load_dwordx4 v[0:3], %0, off\n\tglobal_load_dwordx4 v[4:7], %0, off offset:16\n\t"
                     "global_load_dwordx4 v[8:11], %0, off offset:32\n\tglobal_load_dwordx4 v[12:15], %0, off offset:48\n\t"
                     "s_waitcnt vmcnt(0)\n\tv_mov_b32 v20, 0x3f8ccccd\n\tv_mov_b32 v21, 0x7f7f7f7f" ::"v"(p) : "memory", LP_PROBE_CLOBBERS);
    else
        asm volatile("v_mov_b32 v0, 0\n\tv_mov_b32 v1, 0\n\tv_mov_b32 v2, 0\n\tv_mov_b32 v3, 0\n\tv_mov_b32 v4, 0\n\tv_mov_b32 v5, 0\n\t"
                     "v_mov_b32 v6, 0\n\tv_mov_b32 v7, 0\n\tv_mov_b32 v8, 0\n\tv_mov_b32 v9, 0\n\tv_mov_b32 v10, 0\n\tv_mov_b32 v11, 0\n\t"
                     "v_mov_b32 v12, 0\n\tv_mov_b32 v13, 0\n\tv_mov_b32 v14, 0\n\tv_mov_b32 v15, 0\n\tv_mov_b32 v20, 0\n\tv_mov_b32 v21, 0x7f7f7f7f" ::: LP_PROBE_CLOBBERS);
    for (int i = 0; i < iters; ++i) {
        if constexpr (FMAS == 0) asm volatile(
#include "probe_mfma_body0.inc"
            ::: LP_PROBE_CLOBBERS);
        else if constexpr (FMAS == 2) asm volatile(
#include "probe_mfma_body2.inc"
            ::: LP_PROBE_CLOBBERS);
        else if constexpr (FMAS == 4) asm volatile(
#include "probe_mfma_body4.inc"
            ::: LP_PROBE_CLOBBERS);
        else if constexpr (FMAS == 6) asm volatile(
#include "probe_mfma_body6.inc"
            ::: LP_PROBE_CLOBBERS);
        else if constexpr (FMAS == 8) asm volatile(
#include "probe_mfma_body8.inc"
            ::: LP_PROBE_CLOBBERS);
        else if constexpr (FMAS == -1) asm volatile(
#include "probe_mfma_body_scaled.inc"
            ::: LP_PROBE_CLOBBERS);
        else asm volatile(
#include "probe_mfma_body_inplace.inc"
            ::: LP_PROBE_CLOBBERS);
    }
}

#define LDS_PTR(p) ((void __attribute__((address_space(3))) *)(p))
#define GLB_PTR(p) ((const void __attribute__((address_space(1))) *)(p))

// What a CU's copy path out of the L2 delivers, in the shape the GEMM loops use it: every wave issues eight 1 KB requests
// per step (8 rows x 128 bytes each, rows row_stride apart, 16 bytes per lane), two steps' worth of LDS, one step kept in
// flight behind a wait and a workgroup barrier.  The source is four regions of 512 rows; the workgroups of an XCD read the
// same region and every step moves on by 128 bytes inside the rows (eight windows, then again), so after the first pass
// everything is served by the L2.  TO_LDS: global_load_lds (no registers); otherwise 16-byte loads into registers.
template <int WAVES, bool TO_LDS>
__global__ __launch_bounds__(WAVES * 64) void probe_copy(const uint8_t *__restrict__ src, int steps, int64_t row_stride, uint32_t *sink)
{
    __shared__ __attribute__((aligned(1024))) uint8_t lds[2 * WAVES * 8 * 1024];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const uint8_t *base = src + (int64_t)((blockIdx.x >> 3) & 3) * 512 * row_stride;
    const int row = lane >> 3, chunk = lane & 7;
    u32x4 acc = {0, 0, 0, 0};
    for (int s = 0; s < steps; ++s) {
        const int64_t win = (int64_t)(s & 7) * 128;
        uint8_t *stage = lds + (s & 1) * (WAVES * 8 * 1024);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int r = 8 * (wave + WAVES * i) + row;                     // < 512
            const uint8_t *g = base + (int64_t)r * row_stride + win + chunk * 16;
            if constexpr (TO_LDS) __builtin_amdgcn_global_load_lds(GLB_PTR(g), LDS_PTR(stage + (wave + WAVES * i) * 1024), 16, 0, 0);
            else { const u32x4 v = *(const u32x4 *)g; acc += v; }
        }
        if constexpr (TO_LDS) {
            asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            __builtin_amdgcn_s_barrier();
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (!TO_LDS && acc.x == 0x12345678u && acc.y == 0x9abcdef0u) sink[t] = acc.z + acc.w;      // keeps the loads alive
}

}  // namespace

extern "C" int lp_probe_copy(int to_lds, int waves, int steps, const void *src, int64_t src_bytes, int64_t row_stride, void *sink,
                             int workgroups, lp_stream_t stream)
{
    LP_REQUIRE(waves == 4 || waves == 8, "lp_probe_copy: 4 or 8 waves per workgroup");
    LP_REQUIRE(steps >= 1 && steps <= (1 << 24), "lp_probe_copy: 1 .. 2^24 steps");
    LP_REQUIRE(workgroups >= 1 && workgroups <= (1 << 20), "lp_probe_copy: 1 .. 2^20 workgroups");
    LP_REQUIRE(row_stride >= 1024 && row_stride % 16 == 0, "lp_probe_copy: row_stride must be a multiple of 16, at least 1024");
    LP_REQUIRE(src && sink && (uintptr_t)src % 16 == 0, "lp_probe_copy: src (16-byte aligned) and sink (2048 bytes) must be given");
    LP_REQUIRE(src_bytes >= 4 * 512 * row_stride, "lp_probe_copy: src must hold 4 x 512 rows of row_stride bytes");
    hipStream_t st = (hipStream_t)stream;
    const uint8_t *p = (const uint8_t *)src;
    uint32_t *sk = (uint32_t *)sink;
    if (waves == 8 && to_lds) hipLaunchKernelGGL((probe_copy<8, true>), dim3((unsigned)workgroups), dim3(512), 0, st, p, steps, row_stride, sk);
    else if (waves == 8) hipLaunchKernelGGL((probe_copy<8, false>), dim3((unsigned)workgroups), dim3(512), 0, st, p, steps, row_stride, sk);
    else if (to_lds) hipLaunchKernelGGL((probe_copy<4, true>), dim3((unsigned)workgroups), dim3(256), 0, st, p, steps, row_stride, sk);
    else hipLaunchKernelGGL((probe_copy<4, false>), dim3((unsigned)workgroups), dim3(256), 0, st, p, steps, row_stride, sk);
    return check_launch("lp_probe_copy");
}

extern "C" int lp_probe_mfma(int fmas_per_instruction, int iters, const void *operands, int workgroups, lp_stream_t stream)
{
    LP_REQUIRE(fmas_per_instruction == 0 || fmas_per_instruction == 2 || fmas_per_instruction == 4 || fmas_per_instruction == 6 ||
                   fmas_per_instruction == 8 || (fmas_per_instruction <= -1 && fmas_per_instruction >= -4),
               "lp_probe_mfma: 0, 2, 4, 6 or 8 FMAs per matrix instruction, or -1 .. -4");
    LP_REQUIRE(iters >= 1 && iters <= (1 << 24), "lp_probe_mfma: 1 .. 2^24 iterations");
    LP_REQUIRE(workgroups >= 1 && workgroups <= (1 << 20), "lp_probe_mfma: 1 .. 2^20 workgroups");
    LP_REQUIRE((uintptr_t)operands % 16 == 0, "lp_probe_mfma: operands must be 16-byte aligned (4096 bytes, or NULL)");
    hipStream_t st = (hipStream_t)stream;
    const uint8_t *ops = (const uint8_t *)operands;
    switch (fmas_per_instruction) {
    case 0: hipLaunchKernelGGL(probe_mfma<0>, dim3((unsigned)workgroups), dim3(512), 0, st, ops, iters); break;
    case 2: hipLaunchKernelGGL(probe_mfma<2>, dim3((unsigned)workgroups), dim3(512), 0, st, ops, iters); break;
    case 4: hipLaunchKernelGGL(probe_mfma<4>, dim3((unsigned)workgroups), dim3(512), 0, st, ops, iters); break;
    case 6: hipLaunchKernelGGL(probe_mfma<6>, dim3((unsigned)workgroups), dim3(512), 0, st, ops, iters); break;
    case -1: hipLaunchKernelGGL(probe_mfma<-1>, dim3((unsigned)workgroups), dim3(512), 0, st, ops, iters); break;
    case -2: hipLaunchKernelGGL(probe_mfma<-2>, dim3((unsigned)workgroups), dim3(512), 0, st, ops, iters); break;
    case -3: hipLaunchKernelGGL(probe_mfma<-1>, dim3((unsigned)workgroups), dim3(256), 0, st, ops, iters); break;
    case -4: hipLaunchKernelGGL(probe_mfma<-2>, dim3((unsigned)workgroups), dim3(256), 0, st, ops, iters); break;
    default: hipLaunchKernelGGL(probe_mfma<8>, dim3((unsigned)workgroups), dim3(512), 0, st, ops, iters); break;
    }
    return check_launch("lp_probe_mfma");
}

extern "C" int lp_probe_stream(const void *src, int64_t read_bytes, void *dst, int64_t write_bytes, int workgroups, lp_stream_t stream)
{
    LP_REQUIRE(read_bytes >= 0 && write_bytes >= 0 && read_bytes % 16 == 0 && write_bytes % 16 == 0,
               "lp_probe_stream: byte counts must be non-negative multiples of 16");
    LP_REQUIRE(workgroups >= 1 && workgroups <= (1 << 20), "lp_probe_stream: 1 .. 2^20 workgroups");
    LP_REQUIRE((read_bytes == 0 || src) && (write_bytes == 0 || dst), "lp_probe_stream: null pointer");
    LP_REQUIRE(((uintptr_t)src | (uintptr_t)dst) % 16 == 0, "lp_probe_stream: buffers must be 16-byte aligned");
    hipLaunchKernelGGL(stream_probe, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream, (const u32x4 *)src, read_bytes / 16,
                       (u32x4 *)dst, write_bytes / 16);
    return check_launch("lp_probe_stream");
}

extern "C" int lp_selftest(int which, uint64_t *mismatches, lp_stream_t stream)
{
    LP_REQUIRE(mismatches, "lp_selftest: null pointer");
    LP_REQUIRE(which >= 0 && which <= 4, "lp_selftest: which must be 0..4");
    hipStream_t st = (hipStream_t)stream;
    hipError_t e = hipMemsetAsync(mismatches, 0, sizeof(uint64_t), st);
    if (e != hipSuccess) return fail(LP_ERR_HIP, "lp_selftest: %s", hipGetErrorString(e));
    const unsigned all = (1u << 20);   // 2^20 workgroups x 256 threads x 16 patterns = 2^32
    if (which == 0) hipLaunchKernelGGL(st_cvt_fp8, dim3(all), dim3(256), 0, st, mismatches);
    else if (which == 1) hipLaunchKernelGGL(st_cvt_from_fp8, dim3(1), dim3(256), 0, st, mismatches);
    else if (which == 2) hipLaunchKernelGGL(st_cvt_bf16, dim3(all), dim3(256), 0, st, mismatches);
    else if (which == 3) hipLaunchKernelGGL(st_cvt_fp4, dim3(1), dim3(256), 0, st, mismatches);
    else hipLaunchKernelGGL(st_cvt_to_fp4, dim3(all), dim3(256), 0, st, mismatches);
    return check_launch("lp_selftest");
}

extern "C" int lp_debug_cast(int kind, const float *x, void *out, int64_t n, lp_stream_t stream)
{
    LP_REQUIRE(kind >= 0 && kind <= 5, "lp_debug_cast: kind must be 0..5");
    LP_REQUIRE(n >= 0, "lp_debug_cast: negative length");
    if (n == 0) return LP_OK;
    LP_REQUIRE(x && out, "lp_debug_cast: null pointer");
    unsigned wgs = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
    hipLaunchKernelGGL(debug_cast, dim3(wgs), dim3(256), 0, (hipStream_t)stream, kind, x, out, n);
    return check_launch("lp_debug_cast");
}
