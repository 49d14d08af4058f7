// Block-scaled FP8 GEMM for at most 16 activation rows (single-token decode batches) on gfx950.
//
// The problem is one pass over the weights (M = 16, N = 4096, K = 7168: 29 MB against 0.1 MB of activations),
// so the kernels are cut for the memory system rather than for the matrix cores.  Common to both:
//   * a workgroup owns 16 weight rows (16 output columns) over the whole of K, which gives N / 16 workgroups
//     (256 for N = 4096: one per CU) without cutting K across workgroups, so there are no partial tiles to
//     write, no second kernel and no workspace;
//   * its 8 waves take contiguous runs of at most 7 K blocks each;
//   * v_mfma_f32_16x16x128_f8f6f4 with a zero C per scale block, folded into the accumulators with As * Bs;
//     the 8 partial sums of a workgroup are added through LDS in wave order (deterministic).
// gemm_thin_ring moves the operands with LDS-direct loads: a request covers 8 rows x 128 contiguous bytes
// (8 cache lines per instruction, the cheapest shape for the address path) and lands in a wave-private ring of
// K-block slots in LDS, from where two 16-byte reads per operand give the MFMA layout.  No barrier is involved,
// a wave waits on its own request counter only, and a slot is requested again as soon as it has been read.
// gemm_thin loads straight into MFMA operand layout instead (lane = one row, so 16 cache lines per
// instruction): fewer steps, but its requests cost the address path about twice as much; it is kept for
// comparison behind LP_GEMM_THIN_DIRECT.
#include "gemm_common.h"
#include <utility>

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

#define LDS_PTR(p) ((void __attribute__((address_space(3))) *)(p))
#define GLB_PTR(p) ((const void __attribute__((address_space(1))) *)(p))

__device__ __forceinline__ u32x4 lds_read16(uint32_t addr)
{
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr));
    return v;
}

template <int N>
__device__ __forceinline__ void wait_requests()          // at most N of the wave's global requests still in flight
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// K longer than the 8 x kThinRun blocks a workgroup's waves take in one run: the workgroup walks K in `rounds` rounds of
// round_blocks K blocks -- scale table, requests and the unrolled run of every wave once per round, the accumulators kept
// across them -- so nothing is added up outside the kernel and no scratch is needed; a round's start-up (the rings drain
// and fill again) is paid rounds - 1 times more.  The operands and scale tables move on by a round's blocks, their row
// pitches stay those of the whole K.  Sets kblocks to the K blocks of this round.
#define LP_THIN_ROUND(SDT)                                                                                         \
    const int rb = LONGK && rounds > 1 ? round_blocks : row_blocks;                                                \
    if (LONGK && rd) {                                                                                                      \
        Aq += (int64_t)rb * 128;                                                                                   \
        Bq += (int64_t)rb * 128;                                                                                   \
        As = (const char *)As + (int64_t)rb * ((SDT) == LP_F32 ? 4 : 1);                                           \
        Bs = (const char *)Bs + (int64_t)rb * ((SDT) == LP_F32 ? 4 : 1);                                           \
        __syncthreads(); /* every wave has its scales of the last round in registers before the table is rewritten */ \
    }                                                                                                              \
    const int kblocks = !LONGK ? row_blocks : (row_blocks - rd * rb < rb ? row_blocks - rd * rb : rb);

// entry i of a workgroup's activation-scale table [M, kblocks] (its K blocks of every row, rows row_blocks entries apart
// in memory)
template <bool LONGK>
__device__ __forceinline__ int table_index(int i, int M, int kblocks, int row_blocks)
{
    const int last = M * kblocks - 1;
    const int c = i < last ? i : last;
    if (!LONGK || kblocks == row_blocks) return c;       // (one pass over the whole K: the table is the one in memory)
    const int row = c / kblocks;
    return row * row_blocks + (c - row * kblocks);
}

template <class F, int... J>
__device__ __forceinline__ void unrolled(F &&f, std::integer_sequence<int, J...>)
{
    (f(std::integral_constant<int, J>{}), ...);
}

// SLOTS K blocks of (16 weight rows + 16 activation rows) x 128 bytes per wave: 4 KB a slot.
template <int SDT, int PER, int SLOTS, bool LONGK = false>
__global__ __launch_bounds__(64 * kThinWaves) void gemm_thin_ring(const uint8_t *__restrict__ Aq, const void *__restrict__ As,
                                                                  const uint8_t *__restrict__ Bq, const void *__restrict__ Bs,
                                                                  int M, int64_t N, int64_t K, void *__restrict__ C,
                                                                  int out_dtype, int rounds, int round_blocks)
{
    constexpr int S0 = SLOTS < PER ? SLOTS : PER;        // blocks requested before the first one is used
    __shared__ __attribute__((aligned(1024))) uint8_t ring[kThinWaves * SLOTS * 4096];
    __shared__ f32x4v red[kThinWaves][64];
    __shared__ float sSa[2 * 64 * kThinWaves];           // activation scales, [row][K block] as in memory (896 used at most)
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l16 = lane & 15, lq = lane >> 4;
    const int row_blocks = (int)(K / 128);
    const int64_t n0 = (int64_t)blockIdx.x * 16;
    const int kb0 = wave * PER;
    const int m = l16 < M ? l16 : M - 1;
    f32x4v acc;                                          // zeroed where the first round's run begins
    auto round = [&](const int rd) {
    LP_THIN_ROUND(SDT)

    // The activation-scale table [16, kblocks] goes through LDS (consecutive lanes on consecutive addresses
    // instead of 16-row gathers by every wave).  Its two requests per lane and everything that touches LDS before
    // the rings are drained are written as asm with hand-placed waits: the compiler waits for every LDS-direct
    // request in flight before anything of its own that depends on the request counter.
    uint32_t sv[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const int idx = table_index<LONGK>(t + 64 * kThinWaves * q, M, kblocks, row_blocks);
        if (SDT == LP_F32) asm volatile("global_load_dword %0, %1, off" : "=v"(sv[q]) : "v"((const float *)As + idx));
        else asm volatile("global_load_ubyte %0, %1, off" : "=v"(sv[q]) : "v"((const uint8_t *)As + idx));
    }
    // request plan: lane = (row lane / 8 of the 8 rows of one request, 16-byte position lane % 8); the position
    // holds chunk position ^ row, so that the operand reads below (16 rows, one chunk each) spread over the banks
    const int ld_row = lane >> 3, chunk = (lane & 7) ^ ld_row;
    const uint8_t *bsrc = Bq + (n0 + ld_row) * K + chunk * 16;
    const int ma0 = ld_row < M ? ld_row : M - 1, ma1 = ld_row + 8 < M ? ld_row + 8 : M - 1;
    const uint8_t *asrc0 = Aq + (int64_t)ma0 * K + chunk * 16, *asrc1 = Aq + (int64_t)ma1 * K + chunk * 16;
    uint8_t *wring = ring + wave * (SLOTS * 4096);
    auto request = [&](int j) {                          // block j of the run into slot j % SLOTS: 4 requests
        const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
        uint8_t *dst = wring + (j % SLOTS) * 4096;
        const int64_t off = (int64_t)kb * 128;
        __builtin_amdgcn_global_load_lds(GLB_PTR(bsrc + off), LDS_PTR(dst), 16, 0, 2);                   // weights: streaming hint
        __builtin_amdgcn_global_load_lds(GLB_PTR(bsrc + 8 * K + off), LDS_PTR(dst + 1024), 16, 0, 2);
        __builtin_amdgcn_global_load_lds(GLB_PTR(asrc0 + off), LDS_PTR(dst + 2048), 16, 0, 0);
        __builtin_amdgcn_global_load_lds(GLB_PTR(asrc1 + off), LDS_PTR(dst + 3072), 16, 0, 0);
    };
#pragma unroll
    for (int j = 0; j < S0; ++j) request(j);

    float sb[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
        sb[j] = gemm::scale_at<SDT>(Bs, (n0 >> 7) * row_blocks + kb);
    }
    const uint32_t ssa0 = (uint32_t)(uintptr_t)LDS_PTR(sSa);
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(sv[0]), "+v"(sv[1]) : "n"(4 * S0) : "memory");          // the two oldest requests
    if (SDT != LP_F32) {
#pragma unroll
        for (int q = 0; q < 2; ++q) sv[q] = sv[q] == 0u ? 0x00400000u : (sv[q] == 0xFFu ? 0x7FC00000u : sv[q] << 23);   // e8m0 -> fp32 bits
    }
    asm volatile("ds_write_b32 %0, %1\n\tds_write_b32 %0, %2 offset:2048\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier"
                 :: "v"(ssa0 + 4 * t), "v"(sv[0]), "v"(sv[1]) : "memory");
    float sa[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
        asm volatile("ds_read_b32 %0, %1" : "=v"(sa[j]) : "v"(ssa0 + 4 * (m * kblocks + kb)));
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(sa[j])::"memory");
        sa[j] = kb0 + j < kblocks ? sa[j] * sb[j] : 0.0f;
    }
    __builtin_amdgcn_sched_barrier(0);

    // operand reads: lane (row lane % 16, part lane / 16) takes chunks 2 part and 2 part + 1 of its row
    const uint32_t ring0 = (uint32_t)(uintptr_t)LDS_PTR(wring);
    const uint32_t rd0 = ring0 + l16 * 128 + (((2 * lq) ^ (l16 & 7)) << 4), rd1 = ring0 + l16 * 128 + (((2 * lq + 1) ^ (l16 & 7)) << 4);
    if (!LONGK || rd == 0) acc = f32x4v{0.0f, 0.0f, 0.0f, 0.0f};
    const f32x4v zero = {0.0f, 0.0f, 0.0f, 0.0f};
    auto step = [&](auto jc) {
        constexpr int j = decltype(jc)::value;
        // requests made so far: blocks 0 .. min(PER, S0 + j) - 1; block j has landed when at most the
        // 4 * (that - (j + 1)) younger ones are still in flight
        constexpr int issued = (S0 + j < PER ? S0 + j : PER);
        wait_requests<4 * (issued - (j + 1))>();
        const uint32_t so = (j % SLOTS) * 4096;
        u32x4 w0 = lds_read16(rd0 + so), w1 = lds_read16(rd1 + so), x0 = lds_read16(rd0 + so + 2048), x1 = lds_read16(rd1 + so + 2048);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(w0), "+v"(w1), "+v"(x0), "+v"(x1)::"memory");
        if constexpr (j + SLOTS < PER) request(j + SLOTS);        // the slot has been read: ask for its next block
        const i32x8 wf = {(int)w0.x, (int)w0.y, (int)w0.z, (int)w0.w, (int)w1.x, (int)w1.y, (int)w1.z, (int)w1.w};
        const i32x8 af = {(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
        const f32x4v p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af, zero, 0, 0, 0, 0, 0, 0);
        acc.x = __builtin_fmaf(p.x, sa[j], acc.x);
        acc.y = __builtin_fmaf(p.y, sa[j], acc.y);
        acc.z = __builtin_fmaf(p.z, sa[j], acc.z);
        acc.w = __builtin_fmaf(p.w, sa[j], acc.w);
    };
    unrolled(step, std::make_integer_sequence<int, PER>{});
    };
    if constexpr (LONGK) {
        for (int rd = 0; rd < rounds; ++rd) round(rd);
    } else {
        round(0);
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

// ---------------------------------------------------------------------------------------------------------
// 17 to 64 activation rows: the same cut (16 weight rows x all of K per workgroup), but the activations of a K
// block are now 2 to 4 row groups of 16, up to 8 KB against 2 KB of weights, and would fill a common ring with
// bytes that come from L2.  So the two operands get rings of their own: weights BS K blocks deep (HBM
// latency), activations AD units of 32 rows (L2 latency), a K block being one or two units (BS = 4, AD = 2, or 3 and 3).
// Plan of the requests of one wave, in issue order, so that every wait can name how many younger requests may
// still be in flight: weight blocks 0 .. BS-1 (2 requests each), activation units 0 .. AD-1 (4 each); then at
// step u, after the reads, unit u + AD and, on the first unit of a block j, weight block j + BS.
template <int PER, int U, int BS, int AD>
struct RingPlan {
    int a_end[PER * U];          // requests issued up to and including activation unit u
    int b_end[PER];              // ... weight block j
    int before[PER * U];         // requests issued before the wait of step u
    constexpr RingPlan() : a_end{}, b_end{}, before{}
    {
        int n = 0;
        for (int j = 0; j < (BS < PER ? BS : PER); ++j) { n += 2; b_end[j] = n; }
        for (int u = 0; u < (AD < PER * U ? AD : PER * U); ++u) { n += 4; a_end[u] = n; }
        for (int u = 0; u < PER * U; ++u) {
            before[u] = n;
            if (u + AD < PER * U) { n += 4; a_end[u + AD] = n; }
            if (u % U == 0 && u / U + BS < PER) { n += 2; b_end[u / U + BS] = n; }
        }
    }
};

template <int SDT, int PER, int MB, int BS = 4, int AD = 2, bool LONGK = false>
__global__ __launch_bounds__(64 * kThinWaves) void gemm_thin_ring2(const uint8_t *__restrict__ Aq, const void *__restrict__ As,
                                                                   const uint8_t *__restrict__ Bq, const void *__restrict__ Bs,
                                                                   int M, int64_t N, int64_t K, void *__restrict__ C,
                                                                   int out_dtype, int rounds, int round_blocks)
{
    constexpr int U = (MB + 1) / 2, UNITS = PER * U;
    constexpr int B0 = BS < PER ? BS : PER, A0 = AD < UNITS ? AD : UNITS;
    constexpr int SV = (16 * MB * kThinWaves * kThinRun + 64 * kThinWaves - 1) / (64 * kThinWaves);      // table entries per lane
    constexpr RingPlan<PER, U, BS, AD> plan{};
    __shared__ __attribute__((aligned(1024))) uint8_t bring[kThinWaves * BS * 2048];
    __shared__ __attribute__((aligned(1024))) uint8_t aring[kThinWaves * AD * 4096];     // later: the waves' partial sums
    __shared__ float sSa[SV * 64 * kThinWaves];          // activation scales, [row][K block] as in memory
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l16 = lane & 15, lq = lane >> 4;
    const int row_blocks = (int)(K / 128);
    const int64_t n0 = (int64_t)blockIdx.x * 16;
    const int kb0 = wave * PER;
    f32x4v acc[MB];                                      // zeroed where the first round's run begins
    auto round = [&](const int rd) {
    LP_THIN_ROUND(SDT)

    // scale table through LDS, requests and LDS accesses as asm with hand-placed waits (see gemm_thin_ring)
    uint32_t sv[SV];
#pragma unroll
    for (int q = 0; q < SV; ++q) {
        const int idx = table_index<LONGK>(t + 64 * kThinWaves * q, M, kblocks, row_blocks);
        if (SDT == LP_F32) asm volatile("global_load_dword %0, %1, off" : "=v"(sv[q]) : "v"((const float *)As + idx));
        else asm volatile("global_load_ubyte %0, %1, off" : "=v"(sv[q]) : "v"((const uint8_t *)As + idx));
    }

    const int ld_row = lane >> 3, chunk = (lane & 7) ^ ld_row;
    const uint8_t *bsrc = Bq + (n0 + ld_row) * K + chunk * 16;
    uint8_t *wb = bring + wave * (BS * 2048), *wa = aring + wave * (AD * 4096);
    auto request_b = [&](int j) {
        const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
        uint8_t *dst = wb + (j % BS) * 2048;
        // the weights are read once by the whole launch: with the streaming hint (last argument) they pass the L2 without
        // pushing out the activations every workgroup reads (13.2 -> 13.0 us on M = 64, N = 4096, K = 7168)
        __builtin_amdgcn_global_load_lds(GLB_PTR(bsrc + (int64_t)kb * 128), LDS_PTR(dst), 16, 0, 2);
        __builtin_amdgcn_global_load_lds(GLB_PTR(bsrc + 8 * K + (int64_t)kb * 128), LDS_PTR(dst + 1024), 16, 0, 2);
    };
    auto request_a = [&](int u) {                        // unit u: rows 32 (u % U) .. + 31 of block u / U
        const int j = u / U, v = u % U;
        const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
        uint8_t *dst = wa + (u % AD) * 4096;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = 32 * v + 8 * i + ld_row;
            const uint8_t *src = Aq + (int64_t)(row < M ? row : M - 1) * K + chunk * 16 + (int64_t)kb * 128;
            __builtin_amdgcn_global_load_lds(GLB_PTR(src), LDS_PTR(dst + i * 1024), 16, 0, 0);
        }
    };
#pragma unroll
    for (int j = 0; j < B0; ++j) request_b(j);
#pragma unroll
    for (int u = 0; u < A0; ++u) request_a(u);

    float sb[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
        sb[j] = gemm::scale_at<SDT>(Bs, (n0 >> 7) * row_blocks + kb);
    }
    const uint32_t ssa0 = (uint32_t)(uintptr_t)LDS_PTR(sSa);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * B0 + 4 * A0) : "memory");          // the table requests are the oldest
#pragma unroll
    for (int q = 0; q < SV; ++q) {
        asm volatile("" : "+v"(sv[q]));
        if (SDT != LP_F32) sv[q] = sv[q] == 0u ? 0x00400000u : (sv[q] == 0xFFu ? 0x7FC00000u : sv[q] << 23);       // e8m0 -> fp32 bits
        asm volatile("ds_write_b32 %0, %1" ::"v"(ssa0 + 4 * (t + 64 * kThinWaves * q)), "v"(sv[q]) : "memory");
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    float sa[MB][PER];
#pragma unroll
    for (int g = 0; g < MB; ++g) {
        const int m = 16 * g + l16 < M ? 16 * g + l16 : M - 1;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
            asm volatile("ds_read_b32 %0, %1" : "=v"(sa[g][j]) : "v"(ssa0 + 4 * (m * kblocks + kb)));
        }
    }
#pragma unroll
    for (int g = 0; g < MB; ++g)
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(sa[g][j])::"memory");
            sa[g][j] = kb0 + j < kblocks ? sa[g][j] * sb[j] : 0.0f;
        }
    __builtin_amdgcn_sched_barrier(0);

    const uint32_t rdo0 = l16 * 128 + (((2 * lq) ^ (l16 & 7)) << 4), rdo1 = l16 * 128 + (((2 * lq + 1) ^ (l16 & 7)) << 4);
    const uint32_t wb0 = (uint32_t)(uintptr_t)LDS_PTR(wb), wa0 = (uint32_t)(uintptr_t)LDS_PTR(wa);
    if (!LONGK || rd == 0) {
#pragma unroll
        for (int g = 0; g < MB; ++g) acc[g] = f32x4v{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const f32x4v zero = {0.0f, 0.0f, 0.0f, 0.0f};
    u32x4 w0, w1;                                        // weight fragment of the current block, kept over its units
    auto step = [&](auto uc) {
        constexpr int u = decltype(uc)::value, j = u / U, v = u % U;
        constexpr int need = (v == 0 && plan.b_end[j] > plan.a_end[u]) ? plan.b_end[j] : plan.a_end[u];
        wait_requests<plan.before[u] - need>();
        constexpr bool two = 2 * v + 1 < MB;             // the unit holds a second row group
        const uint32_t ao = wa0 + (u % AD) * 4096;
        u32x4 x0 = lds_read16(ao + rdo0), x1 = lds_read16(ao + rdo1), y0 = x0, y1 = x1;
        if constexpr (two) { y0 = lds_read16(ao + 2048 + rdo0); y1 = lds_read16(ao + 2048 + rdo1); }
        if constexpr (v == 0) { w0 = lds_read16(wb0 + (j % BS) * 2048 + rdo0); w1 = lds_read16(wb0 + (j % BS) * 2048 + rdo1); }
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(x0), "+v"(x1), "+v"(y0), "+v"(y1), "+v"(w0), "+v"(w1)::"memory");
        if constexpr (u + AD < UNITS) request_a(u + AD);
        if constexpr (v == 0 && j + BS < PER) request_b(j + BS);
        const i32x8 wf = {(int)w0.x, (int)w0.y, (int)w0.z, (int)w0.w, (int)w1.x, (int)w1.y, (int)w1.z, (int)w1.w};
        {
            constexpr int g = 2 * v;
            const i32x8 af = {(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
            const f32x4v p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af, zero, 0, 0, 0, 0, 0, 0);
            acc[g].x = __builtin_fmaf(p.x, sa[g][j], acc[g].x);
            acc[g].y = __builtin_fmaf(p.y, sa[g][j], acc[g].y);
            acc[g].z = __builtin_fmaf(p.z, sa[g][j], acc[g].z);
            acc[g].w = __builtin_fmaf(p.w, sa[g][j], acc[g].w);
        }
        if constexpr (two) {
            constexpr int g = 2 * v + 1;
            const i32x8 af = {(int)y0.x, (int)y0.y, (int)y0.z, (int)y0.w, (int)y1.x, (int)y1.y, (int)y1.z, (int)y1.w};
            const f32x4v p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af, zero, 0, 0, 0, 0, 0, 0);
            acc[g].x = __builtin_fmaf(p.x, sa[g][j], acc[g].x);
            acc[g].y = __builtin_fmaf(p.y, sa[g][j], acc[g].y);
            acc[g].z = __builtin_fmaf(p.z, sa[g][j], acc[g].z);
            acc[g].w = __builtin_fmaf(p.w, sa[g][j], acc[g].w);
        }
    };
    unrolled(step, std::make_integer_sequence<int, UNITS>{});
    };
    if constexpr (LONGK) {
        for (int rd = 0; rd < rounds; ++rd) round(rd);
    } else {
        round(0);
    }

    // partial sums into the wave's own (drained) activation ring, then row group g is added up by wave g
    f32x4v *red = (f32x4v *)aring;                       // [wave][4 AD][lane]: the first 4 KB of each wave's own ring
#pragma unroll
    for (int g = 0; g < MB; ++g) red[(wave * 4 * AD + g) * 64 + lane] = acc[g];
    __syncthreads();
    if (wave >= MB) return;
    const int row = 16 * wave + l16;
    f32x4v sum = red[wave * 64 + lane];                  // wave 0's partial of group `wave`
#pragma unroll
    for (int w = 1; w < kThinWaves; ++w) {
        const f32x4v x = red[(w * 4 * AD + wave) * 64 + lane];
        sum.x += x.x; sum.y += x.y; sum.z += x.z; sum.w += x.w;
    }
    if (row >= M) return;
    const int64_t n = n0 + 4 * lq;
    if (out_dtype == LP_BF16) {
        const u32x2 o = {pack_bf16(sum.x, sum.y), pack_bf16(sum.z, sum.w)};
        *(u32x2 *)((uint16_t *)C + (int64_t)row * N + n) = o;
    } else {
        *(f32x4v *)((float *)C + (int64_t)row * N + n) = sum;
    }
}

// ---------------------------------------------------------------------------------------------------------
// 9 to 64 activation rows against many weight rows (more than one group of 16 per CU), and 65 to 128 rows against at
// most 8192 weight rows (where 128 x 128 tiles would leave most CUs without one; R = 2 or 4, U = 4): a workgroup owns 8 R weight
// rows (R = 2 .. 10: N / (8 R) workgroups, e.g. 256 of 72 rows for N = 18432) over the whole of K, so the 64 activation
// rows a workgroup pulls through its CU's copy path are shared by 4 R / 8 times the weight bytes of the 16-row cut.
// Same scheme as gemm_thin_ring2 otherwise: the 8 waves take runs of PER K blocks, wave-private rings fed by LDS-direct
// loads (a request = 8 rows x 128 bytes), hand-counted waits, no barrier inside the loop, partial sums added through LDS
// in wave order.  A K block of a wave is R weight requests (one block in flight: R KB) and two activation units of 32
// rows (4 requests each, two units in flight), 144 KB per workgroup at R = 10.  The rows are cut into (R + 1) / 2 blocks
// of 16 for the matrix instruction; with odd R the last block's upper 8 rows are never loaded and its upper 8 columns
// never stored (a column of the result depends on its own weight row only).  8 R is not a multiple of 128, so a
// block of 16 rows can straddle two weight-scale blocks: every lane takes the scale of its own four columns.
// U: activation units of 32 rows per K block (1 for at most 32 activation rows, 2 up to 64, 4 up to 128 and for slices of
// 128 rows of more, one slice per blockIdx.y); two units are in flight.  One MI355X, us per call with fp32 scales, split-K pair or tiles -> U = 4: 128 x 4096 x 4096 20.6 -> 16.1,
// 96 x 7168 x 2048 13.5 -> 9.1, 128 x 8192 x 4096 23.3 -> 17.3, 128 x 4096 x 7168 22.0 -> 21.7; beyond 8192 weight rows
// the tiles are ahead (128 x 12288 x 4096: 23.5 against 31.7).
template <int PER, int R, int U>
struct RowsPlan {
    int a_end[PER * U];          // requests issued up to and including activation unit u
    int b_end[PER];              // ... weight block j
    int before[PER * U];         // requests issued before the wait of step u
    constexpr RowsPlan() : a_end{}, b_end{}, before{}
    {
        int n = R;
        b_end[0] = n;
        for (int u = 0; u < 2 && u < PER * U; ++u) { n += 4; a_end[u] = n; }
        for (int u = 0; u < PER * U; ++u) {
            before[u] = n;
            if (u + 2 < PER * U) { n += 4; a_end[u + 2] = n; }
            if (u % U == 0 && u / U + 1 < PER) { n += R; b_end[u / U + 1] = n; }
        }
    }
};

template <int SDT, int PER, int R, int U = 2, bool LONGK = false>
__global__ __launch_bounds__(64 * kThinWaves) void gemm_thin_rows(const uint8_t *__restrict__ Aq, const void *__restrict__ As,
                                                                  const uint8_t *__restrict__ Bq, const void *__restrict__ Bs,
                                                                  int M, int64_t N, int64_t K, void *__restrict__ C,
                                                                  int out_dtype, int rounds, int round_blocks)
{
    constexpr int MB = 2 * U, NBK = (R + 1) / 2, UNITS = PER * U, A0 = UNITS < 2 ? UNITS : 2;
    constexpr int SV = (16 * MB * kThinWaves * kThinRun + 64 * kThinWaves - 1) / (64 * kThinWaves);      // table entries per lane
    constexpr int WAVE_LDS = R * 1024 + 2 * 4096;
    constexpr RowsPlan<PER, R, U> plan{};
    __shared__ __attribute__((aligned(1024))) uint8_t ring[kThinWaves * WAVE_LDS];       // per wave: R KB of weights, two activation units
    __shared__ float sSa[SV * 64 * kThinWaves];          // activation scales, [row][K block] as in memory
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int l16 = lane & 15, lq = lane >> 4;
    const int row_blocks = (int)(K / 128);
    const int64_t n0 = (int64_t)blockIdx.x * (8 * R);
    const int kb0 = wave * PER;
    if constexpr (U == 4) {
        // more than 128 activation rows: blockIdx.y picks a slice of 128 (the last one may be shorter)
        const int64_t r0 = (int64_t)blockIdx.y * 128;
        Aq += r0 * K;
        As = (const char *)As + r0 * row_blocks * (SDT == LP_F32 ? 4 : 1);
        C = (char *)C + r0 * N * (out_dtype == LP_BF16 ? 2 : 4);
        M = M - (int)r0 < 128 ? M - (int)r0 : 128;
    }
    f32x4v acc[MB][NBK];                                 // zeroed where the first round's run begins
    auto round = [&](const int rd) {
    LP_THIN_ROUND(SDT)

    uint32_t sv[SV];
#pragma unroll
    for (int q = 0; q < SV; ++q) {
        const int idx = table_index<LONGK>(t + 64 * kThinWaves * q, M, kblocks, row_blocks);
        if (SDT == LP_F32) asm volatile("global_load_dword %0, %1, off" : "=v"(sv[q]) : "v"((const float *)As + idx));
        else asm volatile("global_load_ubyte %0, %1, off" : "=v"(sv[q]) : "v"((const uint8_t *)As + idx));
    }

    const int ld_row = lane >> 3, chunk = (lane & 7) ^ ld_row;
    uint8_t *wb = ring + wave * WAVE_LDS, *wa = wb + R * 1024;
    // weight rows past the end of the matrix (last workgroup) are read from the last row and never stored
    uint32_t boff[R];                                    // N K < 2^32 (checked on the host)
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int64_t row = n0 + 8 * i + ld_row;
        boff[i] = (uint32_t)((row < N ? row : N - 1) * K + chunk * 16);
    }
    auto request_b = [&](int j) {
        const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
#pragma unroll
        for (int i = 0; i < R; ++i)              // read once by the whole launch: streamed past the L2's resident lines
            __builtin_amdgcn_global_load_lds(GLB_PTR(Bq + boff[i] + (uint32_t)kb * 128u), LDS_PTR(wb + i * 1024), 16, 0, 2);
    };
    auto request_a = [&](int u) {                        // unit u: rows 32 (u % U) .. + 31 of block u / U, into slot u % 2
        const int j = u / U, v = u % U;
        const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
        uint8_t *dst = wa + (u % 2) * 4096;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = 32 * v + 8 * i + ld_row;
            const uint8_t *src = Aq + (int64_t)(row < M ? row : M - 1) * K + chunk * 16 + (int64_t)kb * 128;
            __builtin_amdgcn_global_load_lds(GLB_PTR(src), LDS_PTR(dst + i * 1024), 16, 0, 0);
        }
    };
    request_b(0);
#pragma unroll
    for (int u = 0; u < A0; ++u) request_a(u);

    // weight scales of the lane's own four columns of every block of 16
    float sb[NBK][PER];
    const int64_t last_blk = (N >> 7) - 1;
#pragma unroll
    for (int nb = 0; nb < NBK; ++nb) {
        int64_t blk = (n0 + 16 * nb + 4 * lq) >> 7;
        if (blk > last_blk) blk = last_blk;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
            sb[nb][j] = gemm::scale_at<SDT>(Bs, blk * row_blocks + kb);
        }
    }
    const uint32_t ssa0 = (uint32_t)(uintptr_t)LDS_PTR(sSa);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(R + 4 * A0) : "memory");          // the table requests are the oldest
#pragma unroll
    for (int q = 0; q < SV; ++q) {
        asm volatile("" : "+v"(sv[q]));
        if (SDT != LP_F32) sv[q] = sv[q] == 0u ? 0x00400000u : (sv[q] == 0xFFu ? 0x7FC00000u : sv[q] << 23);       // e8m0 -> fp32 bits
        asm volatile("ds_write_b32 %0, %1" ::"v"(ssa0 + 4 * (t + 64 * kThinWaves * q)), "v"(sv[q]) : "memory");
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    float sa[MB][PER];
#pragma unroll
    for (int g = 0; g < MB; ++g) {
        const int m = 16 * g + l16 < M ? 16 * g + l16 : M - 1;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int kb = kb0 + j < kblocks ? kb0 + j : kblocks - 1;
            asm volatile("ds_read_b32 %0, %1" : "=v"(sa[g][j]) : "v"(ssa0 + 4 * (m * kblocks + kb)));
        }
    }
#pragma unroll
    for (int g = 0; g < MB; ++g)
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(sa[g][j])::"memory");
            if (kb0 + j >= kblocks) sa[g][j] = 0.0f;     // a K block past the end (the last wave's run) adds nothing
        }
    // the weight scales are in their registers before the loop: inside it every wait on the request counter is counted by hand
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int nb = 0; nb < NBK; ++nb)
#pragma unroll
        for (int j = 0; j < PER; ++j) asm volatile("" : "+v"(sb[nb][j]));
    __builtin_amdgcn_sched_barrier(0);

    const uint32_t rdo0 = l16 * 128 + (((2 * lq) ^ (l16 & 7)) << 4), rdo1 = l16 * 128 + (((2 * lq + 1) ^ (l16 & 7)) << 4);
    const uint32_t wb0 = (uint32_t)(uintptr_t)LDS_PTR(wb), wa0 = (uint32_t)(uintptr_t)LDS_PTR(wa);
    if (!LONGK || rd == 0) {
#pragma unroll
        for (int g = 0; g < MB; ++g)
#pragma unroll
            for (int nb = 0; nb < NBK; ++nb) acc[g][nb] = f32x4v{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const f32x4v zero = {0.0f, 0.0f, 0.0f, 0.0f};
    i32x8 wf[NBK];                                       // weight fragments of the current block, kept over its units
    auto step = [&](auto uc) {
        constexpr int u = decltype(uc)::value, j = u / U, v = u % U;
        constexpr int need = (v == 0 && plan.b_end[j] > plan.a_end[u]) ? plan.b_end[j] : plan.a_end[u];
        wait_requests<plan.before[u] - need>();
        const uint32_t ao = wa0 + (u % 2) * 4096;
        u32x4 x0 = lds_read16(ao + rdo0), x1 = lds_read16(ao + rdo1);
        u32x4 y0 = lds_read16(ao + 2048 + rdo0), y1 = lds_read16(ao + 2048 + rdo1);
        u32x4 w0[NBK], w1[NBK];
        if constexpr (v == 0) {
#pragma unroll
            for (int nb = 0; nb < NBK; ++nb) { w0[nb] = lds_read16(wb0 + nb * 2048 + rdo0); w1[nb] = lds_read16(wb0 + nb * 2048 + rdo1); }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(x0), "+v"(x1), "+v"(y0), "+v"(y1)::"memory");
        if constexpr (v == 0) {
#pragma unroll
            for (int nb = 0; nb < NBK; ++nb) {
                asm volatile("" : "+v"(w0[nb]), "+v"(w1[nb]));          // used after the wait above, not before
                wf[nb] = i32x8{(int)w0[nb].x, (int)w0[nb].y, (int)w0[nb].z, (int)w0[nb].w, (int)w1[nb].x, (int)w1[nb].y, (int)w1[nb].z, (int)w1[nb].w};
            }
        }
        if constexpr (u + 2 < UNITS) request_a(u + 2);
        if constexpr (v == 0 && j + 1 < PER) request_b(j + 1);
        const i32x8 af0 = {(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
        const i32x8 af1 = {(int)y0.x, (int)y0.y, (int)y0.z, (int)y0.w, (int)y1.x, (int)y1.y, (int)y1.z, (int)y1.w};
#pragma unroll
        for (int nb = 0; nb < NBK; ++nb) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                constexpr int g0 = 2 * v;
                const int g = g0 + h;
                const f32x4v p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[nb], h ? af1 : af0, zero, 0, 0, 0, 0, 0, 0);
                const float sc = sa[g][j] * sb[nb][j];
                acc[g][nb].x = __builtin_fmaf(p.x, sc, acc[g][nb].x);
                acc[g][nb].y = __builtin_fmaf(p.y, sc, acc[g][nb].y);
                acc[g][nb].z = __builtin_fmaf(p.z, sc, acc[g][nb].z);
                acc[g][nb].w = __builtin_fmaf(p.w, sc, acc[g][nb].w);
            }
        }
    };
    unrolled(step, std::make_integer_sequence<int, UNITS>{});
    };
    if constexpr (LONGK) {
        for (int rd = 0; rd < rounds; ++rd) round(rd);
    } else {
        round(0);
    }

    // partial sums through the (drained) rings, as many row groups at a time as fit a wave's own ring (all of them in one pass
    // where they do: every pass costs two barriers at which the waves wait for the slowest): pair (g, nb) of the pass is
    // added up by wave pair % 8 over the waves in their order
    f32x4v *red = (f32x4v *)ring;                        // [wave][GP NBK][lane], GP NBK KB per wave <= its ring
    constexpr int FIT = WAVE_LDS / 1024 / NBK;           // row groups whose partial sums fit
    constexpr int GP = FIT >= MB ? MB : (FIT >= 4 && MB % 4 == 0 ? 4 : 2);
    static_assert(GP * NBK * 1024 <= WAVE_LDS && MB % GP == 0, "a wave's partial sums of a pass fit its own ring");
#pragma unroll
    for (int pass = 0; pass < MB / GP; ++pass) {
        __syncthreads();                                 // every wave is done with its ring (or with the previous pass)
#pragma unroll
        for (int h = 0; h < GP; ++h)
#pragma unroll
            for (int nb = 0; nb < NBK; ++nb) red[(wave * (WAVE_LDS / 1024) + h * NBK + nb) * 64 + lane] = acc[GP * pass + h][nb];
        __syncthreads();
        for (int pair = wave; pair < GP * NBK; pair += kThinWaves) {
            const int h = pair / NBK, nb = pair % NBK;
            f32x4v sum = red[(h * NBK + nb) * 64 + lane];
#pragma unroll
            for (int w = 1; w < kThinWaves; ++w) {
                const f32x4v x = red[(w * (WAVE_LDS / 1024) + h * NBK + nb) * 64 + lane];
                sum.x += x.x; sum.y += x.y; sum.z += x.z; sum.w += x.w;
            }
            const int row = 16 * (GP * pass + h) + l16, col = 16 * nb + 4 * lq;
            const int64_t n = n0 + col;
            if (row >= M || col >= 8 * R || n >= N) continue;
            if (out_dtype == LP_BF16) {
                const u32x2 o = {pack_bf16(sum.x, sum.y), pack_bf16(sum.z, sum.w)};
                *(u32x2 *)((uint16_t *)C + (int64_t)row * N + n) = o;
            } else {
                *(f32x4v *)((float *)C + (int64_t)row * N + n) = sum;
            }
        }
    }
}

}  // namespace

namespace lowp {
namespace gemm {

// K longer than one run of the workgroup's waves (8 x kThinRun blocks = 7168): rounds of equal length inside the workgroup,
// at most kThinMaxRounds of them (K <= 57344).  Returns the number of rounds and the K blocks of one.
constexpr int kThinMaxRounds = 8;
static int thin_rounds(int64_t K, int *round_blocks)
{
    const int64_t kblocks = K / 128, whole = kThinWaves * kThinRun;
    const int rounds = (int)((kblocks + whole - 1) / whole);
    *round_blocks = rounds <= 1 ? 0 : (int)((kblocks + rounds - 1) / rounds);
    return rounds < 1 ? 1 : rounds;
}

// Which shapes of a long K the decode kernels take (one MI355X, us per call, tiled kernels or K-split pair -> rounds): up to
// 16 rows all from 4096 weight rows and, with fewer, up to two rounds (1 x 7168 x 18432 64.1 -> 23.8, 8 x 7168 x 8192 32.5 -> 13.4,
// 12 x 12288 x 8192 35.5 -> 20.0, 16 x 18432 x 8192 37.8 -> 29.7, 16 x 4096 x 16384 18.7 -> 18.3, 2 x 512 x 8192 9.1 -> 8.0); up to 64 rows from
// 5120 weight rows (64 x 7168 x 18432 70.4 -> 44.6, 64 x 5120 x 14336 55.8 -> 31.8, 64 x 6144 x 8192 34.9 -> 22.2, 64 x 8192 x 8192
// 35.7 -> 24.0, 32 x 12288 x 14336 56.0 -> 35.2, 24 x 36864 x 8192 78.9 -> 57.1, 64 x 12288 x 8192 37.0 -> 28.7; but 64 x 4096 x
// 8192 18.0 -> 17.8, 32 x 2048 x 16384 15.6 -> 17.8, and above 32 rows 48 x 18432 x 8192 36.3 -> 47.9, see below);
// not above 64 rows (128 x 4096 x 14336 28.2 -> 39.7, 100 x 3072 x 9216 20.7 -> 26.1; the gains at 7168 weight rows and more
// came from a variant that spilled).  LP_GEMM_THIN_LONG_K = 0 / 1 (tuning aid): none / all of them up to 64 rows.
// Weight rows per workgroup of the many-rows kernel, / 8: the R for which rounds of 256 workgroups x bytes a workgroup pulls
// are fewest (the larger R when they tie); *wgs_out = its workgroups.
static int choose_rows_r(int64_t M, int64_t N, bool long_k, int64_t *wgs_out)
{
    int best = 10;
    int64_t best_cost = INT64_MAX, best_wgs = 0;
    const int64_t slices = M > 64 ? (M + 127) / 128 : 1;
    for (int r : {2, 4, 6, 8, 9, 10}) {
        if (M > 64 ? r > 4 : r < 4) continue;
        if (long_k && M > 32 && r > 6) continue;        // (no long-K variant with two activation units and more rows)
        // a workgroup's time goes with the bytes it pulls: 8 r weight rows and, from 65 rows on, 128 activation rows
        const int64_t wgs = slices * ((N + 8 * r - 1) / (8 * r)), cost = ((wgs + 255) / 256) * (M > 64 ? 16 + r : r);
        if (cost < best_cost || (cost == best_cost && r > best)) { best_cost = cost; best = r; best_wgs = wgs; }
    }
    if (wgs_out) *wgs_out = best_wgs;
    return best;
}

static bool long_k_ok(int64_t M, int64_t N, int64_t K)
{
    static const char *env = getenv("LP_GEMM_THIN_LONG_K");
    if (K / 128 <= kThinWaves * kThinRun) return true;
    if (K / 128 > kThinMaxRounds * kThinWaves * kThinRun || M > 64) return false;
    if (env) return atoi(env) != 0;
    if (M <= 16) return N >= 4096 || K / 128 <= 2 * kThinWaves * kThinRun;        // (16 x 1024 x 20480, three rounds on 64 workgroups: 15.1 -> 17.6)
    if (N < 5120) return false;
    if (M <= 32) return true;
    // 33 .. 64 rows take at most 48 weight rows per workgroup here: not where that leaves the last round of workgroups badly
    // filled (N = 18432: 384 workgroups; 48 x 18432 x 8192 36.3 -> 47.9 us, where 12288 rows, 256 workgroups, go 36.2 -> 27.0)
    int64_t wgs = 0;
    (void)choose_rows_r(M, N, true, &wgs);
    if (M <= 64) return wgs <= 256 || wgs * 100 >= ((wgs + 255) / 256) * 256 * 85;
    return false;          // (65 .. 128 rows: 128 x 7168 x 18432 81.4 -> 70.5 us with a variant that spills registers; not kept, see LP_LAUNCH_LONGK)
}

bool thin_ok(int64_t M, int64_t N, int64_t K)
{
    // one run of K blocks per wave.  Above 16 rows a workgroup holds 128 KB of LDS and its activations (M / 16 times the
    // bytes of its weights) come through the same request path, so beyond about two workgroups per CU the
    // K-split kernel, which shares the activations between 128 weight rows, is ahead (measured at N = 18432).
    // No lower limit on the weight rows: with fewer workgroups than CUs this one launch is still ahead of the K-split
    // pair's two (one MI355X, us per call, pair -> this kernel: 32 x 2048 x 1024 8.8 -> 4.0, 64 x 2048 x 7168 16.0 -> 11.8,
    // 8 x 512 x 4096 10.1 -> 5.3, 16 x 128 x 7168 11.2 -> 5.3, 64 x 128 x 7168 12.4 -> 11.0).  LP_GEMM_THIN_FROM = n
    // (tuning aid): only from n groups of 16 weight rows.
    if (M < 1 || M > 64 || N % 16 != 0 || K % 128 != 0 || !long_k_ok(M, N, K)) return false;
    const int64_t groups = N / 16;
    static const int64_t min_groups = getenv("LP_GEMM_THIN_FROM") ? atoi(getenv("LP_GEMM_THIN_FROM")) : 1;
    return groups >= min_groups && groups <= (M <= 16 ? 0x7FFFFFFF : 512);
}

// 9 .. 64 activation rows against more weight rows than one 16-row workgroup per CU: 8 R rows per workgroup, R from {4, 6, 8, 9,
// 10} (65 .. 128 activation rows: from {2, 4}) such that the rounds of 256 workgroups times R are fewest (18432 rows: R = 9, 256 workgroups).
// Groups of 16 weight rows from which the many-rows kernel takes over from the 16-row cut at more than 16 activation rows
// (one MI355X, M = 64, K = 7168, us per call, 16-row cut or 128 x 128 tiles -> 8 R rows: N = 6144 23.1 -> 16.9, 8192 24.2 ->
// 17.8, 12288 36.3 -> 22.0, 18432 38.4 -> 29.3, 36864 73.3 -> 60.7; N = 4096 is one 16-row workgroup per CU either way).
constexpr int64_t kRowsFromGroups = 256;

bool thin_rows_ok(int64_t M, int64_t N, int64_t K)
{
    static const bool off = getenv("LP_GEMM_THIN_ROWS") && atoi(getenv("LP_GEMM_THIN_ROWS")) == 0;       // tuning aid
    static const int64_t min_groups = getenv("LP_GEMM_THIN_ROWS_FROM") ? atoi(getenv("LP_GEMM_THIN_ROWS_FROM")) : kRowsFromGroups;
    // from 9 activation rows: at 16 rows it is 8 % ahead of the 16-row ring kernel from N = 18432 (28.2 -> 25.9 us at K = 7168),
    // at 8 rows level with it (25.1 / 25.5), at 1 row behind (23.6 / 25.4)
    static const int64_t min_m = getenv("LP_GEMM_THIN_ROWS_MIN_M") ? atoi(getenv("LP_GEMM_THIN_ROWS_MIN_M")) : 9;
    // 65 .. 128 rows (four activation units per K block): where the tiled kernels would leave most CUs without a tile.  Up to
    // 4096 weight rows a workgroup takes 16 of them (R = 2: 256 workgroups at N = 4096; 128 x 4096 x 4096 16.6 -> 15.3 us,
    // 96 x 3072 x 2048 8.3 -> 7.5), and there is no lower limit on the weight rows either (tiles or K-split pair -> this
    // kernel: 128 x 2048 x 7168 21.5 -> 14.2, 128 x 2048 x 2048 12.9 -> 7.9, 128 x 512 x 1024 8.9 -> 6.0, 128 x 128 x 7168
    // 13.7 -> 13.1).  LP_GEMM_THIN_ROWS_WIDE_FROM = n (tuning aid): only from n groups of 16 weight rows.
    static const int64_t max_m = getenv("LP_GEMM_THIN_ROWS_MAX_M") ? atoi(getenv("LP_GEMM_THIN_ROWS_MAX_M")) : 128;
    static const int64_t wide_max_n = getenv("LP_GEMM_THIN_ROWS_WIDE_N") ? atoi(getenv("LP_GEMM_THIN_ROWS_WIDE_N")) : 8192;
    if (off || N % 16 != 0 || K % 128 != 0 || !long_k_ok(M, N, K) || N * K >= 0xFFFFFFFFll) return false;
    static const int64_t wide_min_groups = getenv("LP_GEMM_THIN_ROWS_WIDE_FROM") ? atoi(getenv("LP_GEMM_THIN_ROWS_WIDE_FROM")) : 1;
    if (M > 128) {
        // slices of 128 rows (blockIdx.y) in one launch, where all workgroups run at once and the tiled kernels would give most
        // CUs no tile, so that a tile's chain of K steps is the whole time (0.7 us per step of 128): one MI355X, us per call,
        // tiles or K-split pair -> slices: 512 x 2048 x 4096 26.8 -> 16.3, 256 x 4096 x 4096 23.9 -> 17.5, 1024 x 1024 x 7168
        // 28.6 -> 22.7, 512 x 2048 x 1024 10.2 -> 7.5, 256 x 2048 x 2048 13.6 -> 8.5.  Not with two rounds of workgroups (512 x
        // 3072 x 4096: 22.0 -> 29.6), not at K = 512 (level), not with few weight rows and a long K (256 x 256 x 7168: 14.4 ->
        // 16.7).  The longer K, the fewer rows: up to 8192 at K <= 2048 (2048 x 512 x 2048: 13.3 -> 10.7, 4096 x 128 x 1024: 10.7 ->
        // 7.5), up to 2048 at K <= 4096 and from 256 weight rows (1280 x 512 x 4096: 20.1 -> 17.5, but 4096 x 256 x 4096: 20.6 ->
        // 28.2 and 1280 x 128 x 4096: 13.9 -> 15.7), up to 1024 beyond.
        // LP_GEMM_THIN_ROWS_SLICES_MAX_M = n (tuning aid): up to n rows at most, 128 switches the slices off.
        static const int64_t slices_max_m = getenv("LP_GEMM_THIN_ROWS_SLICES_MAX_M") ? atoi(getenv("LP_GEMM_THIN_ROWS_SLICES_MAX_M")) : 8192;
        const int64_t rows_at_k = K <= 2048 ? 8192 : K <= 4096 ? 2048 : 1024;
        const int64_t weight_rows_at_k = K <= 2048 ? 128 : K <= 4096 ? 256 : 1024;
        return M <= slices_max_m && M <= rows_at_k && N >= weight_rows_at_k && max_m >= 128 && K >= 1024 &&
               ((M + 127) / 128) * ((N + 31) / 32) <= 256;
    }
    if (M > 64) return M <= max_m && N / 16 >= wide_min_groups && N <= wide_max_n;
    // up to 16 rows the 16-row ring kernel stays ahead while it has at most two workgroups per CU and K is short (9 .. 16 x 5120 ..
    // 8192 x 4096: 8.8 .. 9.1 -> 8.1 .. 8.6 us, x 2048: level to 0.4 ahead; at K = 7168 and 16 rows the many-rows kernel leads, 14.1 -> 13.0)
    static const bool min_m_given = getenv("LP_GEMM_THIN_ROWS_MIN_M") != nullptr;
    if (M <= 16 && N <= 8192 && K <= 4096 && !min_m_given) return false;
    // above 32 rows a workgroup pulls as many activation bytes as weight bytes, and from about a round of 256 x 256 tiles on
    // the tiled kernels, which share the activations between 256 weight rows, are ahead (us per call, this kernel -> tiles,
    // 64 rows: 65536 x 4096 63.8 -> 42.3, 98304 x 7168 150.3 -> 127.7, 129280 x 7168 200.6 -> 168.3, 57344 x 7168 113.4 ->
    // 81.1, 53248 x 7168 86.1 -> 79.9, but 49152 x 7168 72.9 -> 77.0 and 40960 x 7168 61.6 -> 69.8; 40 rows: 129280 x 7168
    // 178.0 -> 162.6, 53248 x 7168 77.0 -> 75.7).  With K <= 4096 from 24576 weight rows already (64 rows: 24576 x 4096
    // 29.4 -> 24.9, 32768 x 4096 33.2 -> 25.0, 57344 x 4096 73.6 -> 41.1, 32768 x 2048 19.4 -> 16.8, 24576 x 2048 16.9 -> 16.2,
    // but 18432 x 4096 20.1 -> 24.2; 40 rows: 24576 x 4096 26.5 -> 24.2, 57344 x 2048 36.9 -> 23.6, 98304 x 4096 85.1 -> 91.6).
    // 32 rows level at 129280 x 7168, 24 rows 153.1 -> 160.0.  LP_GEMM_THIN_ROWS_TILED_FROM_N = n (tuning aid): from n
    // weight rows whatever K.
    static const int64_t tiled_from_env = getenv("LP_GEMM_THIN_ROWS_TILED_FROM_N") ? atoll(getenv("LP_GEMM_THIN_ROWS_TILED_FROM_N")) : 0;
    const int64_t tiled_from_n = tiled_from_env > 0 ? tiled_from_env : K <= 4096 ? 24576 : 53248;
    if (M > 32 && N >= tiled_from_n) return false;
    return M >= min_m && N / 16 > min_groups;
}

// The variant that walks a long K in rounds exists from four K blocks per wave on (two rounds cover at least 57 blocks)
// and only where it needs no scratch (OK): loads and stores share one request counter and complete out of order with
// respect to each other, so a spill's store inside the run could satisfy a hand-counted wait before the request that
// wait is for has landed.  The host never asks for a long K where the variant is missing (long_k_ok, the choice of R).
#define LP_LAUNCH_LONGK(OK, LONG_KERNEL, KERNEL, ...)                                                    \
    do {                                                                                                 \
        if constexpr (PER >= 4 && (OK)) {                                                                \
            if (rounds > 1) { hipLaunchKernelGGL(LONG_KERNEL, __VA_ARGS__); break; }                     \
        }                                                                                                \
        hipLaunchKernelGGL(KERNEL, __VA_ARGS__);                                                         \
    } while (0)

template <int SDT, int PER, int R>
void launch_thin_rows_r(const void *Aq, const void *As, const void *Bq, const void *Bs, int64_t M, int64_t N, int64_t K, void *C,
                        int out_dtype, int rounds, int round_blocks, hipStream_t st)
{
    const dim3 grid((unsigned)((N + 8 * R - 1) / (8 * R))), block(64 * kThinWaves);
    if constexpr (R == 2) {
        // 16 weight rows per workgroup exist from 65 activation rows on only (up to 64 the ring kernels serve that cut)
        LP_LAUNCH_LONGK(false, (gemm_thin_rows<SDT, PER, R, 4, true>), (gemm_thin_rows<SDT, PER, R, 4>), dim3(grid.x, (unsigned)((M + 127) / 128)), block, 0, st, (const uint8_t *)Aq, As, (const uint8_t *)Bq, Bs, (int)M, N, K,
                           C, out_dtype, rounds, round_blocks);
        return;
    }
    if constexpr (R == 4) {
        // 65 .. 128 activation rows: four units of 32 per K block (R = 4 only: with more weight rows the accumulators of eight
        // row blocks no longer fit the registers, and a spill's reload would go through the request counter this kernel
        // counts by hand)
        if (M > 64) {
            LP_LAUNCH_LONGK(false, (gemm_thin_rows<SDT, PER, R, 4, true>), (gemm_thin_rows<SDT, PER, R, 4>), dim3(grid.x, (unsigned)((M + 127) / 128)), block, 0, st, (const uint8_t *)Aq, As, (const uint8_t *)Bq, Bs, (int)M, N, K,
                               C, out_dtype, rounds, round_blocks);
            return;
        }
    }
    if (M <= 32)
        LP_LAUNCH_LONGK(true, (gemm_thin_rows<SDT, PER, R, 1, true>), (gemm_thin_rows<SDT, PER, R, 1>), grid, block, 0, st, (const uint8_t *)Aq, As, (const uint8_t *)Bq, Bs, (int)M, N, K,
                           C, out_dtype, rounds, round_blocks);
    else
        LP_LAUNCH_LONGK(R <= 6, (gemm_thin_rows<SDT, PER, R, 2, true>), (gemm_thin_rows<SDT, PER, R, 2>), grid, block, 0, st, (const uint8_t *)Aq, As, (const uint8_t *)Bq, Bs, (int)M, N, K,
                           C, out_dtype, rounds, round_blocks);
}

template <int SDT, int PER>
void launch_thin_rows_per(const void *Aq, const void *As, const void *Bq, const void *Bs, int64_t M, int64_t N, int64_t K, void *C,
                          int out_dtype, int per, int r, int rounds, int round_blocks, hipStream_t st)
{
    if constexpr (PER > 1) {
        if (per < PER) return launch_thin_rows_per<SDT, PER - 1>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, per, r, rounds, round_blocks, st);
    }
    switch (r) {
    case 2: return launch_thin_rows_r<SDT, PER, 2>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, rounds, round_blocks, st);
    case 4: return launch_thin_rows_r<SDT, PER, 4>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, rounds, round_blocks, st);
    case 6: return launch_thin_rows_r<SDT, PER, 6>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, rounds, round_blocks, st);
    case 8: return launch_thin_rows_r<SDT, PER, 8>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, rounds, round_blocks, st);
    case 9: return launch_thin_rows_r<SDT, PER, 9>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, rounds, round_blocks, st);
    default: return launch_thin_rows_r<SDT, PER, 10>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, rounds, round_blocks, st);
    }
}

int launch_thin_rows(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K,
                     void *C, int out_dtype, hipStream_t st)
{
    static const int forced = getenv("LP_GEMM_THIN_ROWS") ? atoi(getenv("LP_GEMM_THIN_ROWS")) : 0;     // tuning aid: 2, 4, 6, 8, 9, 10
    int round_blocks = 0;
    const int rounds = thin_rounds(K, &round_blocks);
    const int kblocks = rounds > 1 ? round_blocks : (int)(K / 128);
    const int per = (kblocks + kThinWaves - 1) / kThinWaves;
    int best = choose_rows_r(M, N, rounds > 1, nullptr);
    if ((forced == 2 || forced == 4 || forced == 6 || forced == 8 || forced == 9 || forced == 10) && (M > 64 ? forced <= 4 : forced >= 4)) best = forced;
    if (rounds > 1 && (M > 64 || (M > 32 && best > 6)))
        return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_block: no decode kernel for K = %lld with %lld rows and %d weight rows per workgroup",
                    (long long)K, (long long)M, 8 * best);
    if (scale_dtype == LP_F32) launch_thin_rows_per<LP_F32, kThinRun>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, per, best, rounds, round_blocks, st);
    else launch_thin_rows_per<LP_E8M0, kThinRun>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, per, best, rounds, round_blocks, st);
    return check_launch("lp_gemm_fp8_block(thin, many rows)");
}

template <int SDT, int PER>
void launch_thin_per(const void *Aq, const void *As, const void *Bq, const void *Bs, int64_t M, int64_t N, int64_t K, void *C,
                     int out_dtype, int per, int kind, int rounds, int round_blocks, hipStream_t st)
{
    if constexpr (PER > 1) {
        if (per < PER) return launch_thin_per<SDT, PER - 1>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, per, kind, rounds, round_blocks, st);
    }
    const dim3 grid((unsigned)(N / 16)), block(64 * kThinWaves);
    const uint8_t *a = (const uint8_t *)Aq, *b = (const uint8_t *)Bq;
    // 49 to 64 rows: weight ring three blocks deep and activation ring three units (158 KB of LDS; with four and two,
    // 142 KB, M = 64, N = 4096, K = 7168 takes 12.9 instead of 12.75 us)
    if (M > 48) LP_LAUNCH_LONGK(true, (gemm_thin_ring2<SDT, PER, 4, 3, 3, true>), (gemm_thin_ring2<SDT, PER, 4, 3, 3>), grid, block, 0, st, a, As, b, Bs, (int)M, N, K, C, out_dtype, rounds, round_blocks);
    else if (M > 32) LP_LAUNCH_LONGK(true, (gemm_thin_ring2<SDT, PER, 3, 4, 2, true>), (gemm_thin_ring2<SDT, PER, 3>), grid, block, 0, st, a, As, b, Bs, (int)M, N, K, C, out_dtype, rounds, round_blocks);
    else if (M > 16) LP_LAUNCH_LONGK(true, (gemm_thin_ring2<SDT, PER, 2, 4, 2, true>), (gemm_thin_ring2<SDT, PER, 2>), grid, block, 0, st, a, As, b, Bs, (int)M, N, K, C, out_dtype, rounds, round_blocks);
    else if (kind == 0) hipLaunchKernelGGL((gemm_thin<SDT, PER>), grid, block, 0, st, a, As, b, Bs, (int)M, N, K, C, out_dtype);
    else if (kind == 4) LP_LAUNCH_LONGK(true, (gemm_thin_ring<SDT, PER, 4, true>), (gemm_thin_ring<SDT, PER, 4>), grid, block, 0, st, a, As, b, Bs, (int)M, N, K, C, out_dtype, rounds, round_blocks);
    else LP_LAUNCH_LONGK(true, (gemm_thin_ring<SDT, PER, 2, true>), (gemm_thin_ring<SDT, PER, 2>), grid, block, 0, st, a, As, b, Bs, (int)M, N, K, C, out_dtype, rounds, round_blocks);
}

int launch_thin(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K,
                void *C, int out_dtype, hipStream_t st)
{
    int round_blocks = 0;
    const int rounds = thin_rounds(K, &round_blocks);
    const int kblocks = rounds > 1 ? round_blocks : (int)(K / 128);
    const int per = (kblocks + kThinWaves - 1) / kThinWaves;
    // ring depth 2 (64 KB of LDS: two workgroups share a CU and one's tail overlaps the other's start) measured
    // as fast as depth 4 with one workgroup per CU at N = 4096 and faster beyond
    static const char *env = getenv("LP_GEMM_THIN_DIRECT");                      // tuning aids
    static const char *slots_env = getenv("LP_GEMM_THIN_SLOTS");
    int kind = env && rounds == 1 ? 0 : 2;              // (the kernel without rings takes no long K)
    if (!env && slots_env) kind = atoi(slots_env) == 4 ? 4 : 2;
    if (scale_dtype == LP_F32) launch_thin_per<LP_F32, kThinRun>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, per, kind, rounds, round_blocks, st);
    else launch_thin_per<LP_E8M0, kThinRun>(Aq, As, Bq, Bs, M, N, K, C, out_dtype, per, kind, rounds, round_blocks, st);
    return check_launch("lp_gemm_fp8_block(thin)");
}

}  // namespace gemm
}  // namespace lowp
