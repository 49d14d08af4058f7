// Large-tile block-scaled FP8 GEMM for gfx950 (the kernel that carries prefill-sized problems).
//
// Workgroup: 512 threads = 8 waves (4 along M x 2 along N), C tile 256(M) x TN(N)
// with TN = 128 / 192 / 256 chosen at launch to balance the last round of
// tiles over the 256 CUs.  K advances in steps of 128 = one scale block.
//
// Data movement: each step's operand tiles (256 x 128 B of activations, TN x
// 128 B of weights) are copied HBM/L2 -> LDS by global_load_lds_dwordx4, with
// no VGPR staging, into one of two stages (the copy of step k+1 overlaps the
// math of step k).  A row holds 8 chunks of 16 bytes.  The LDS serves a
// 16-byte-per-lane read at 256 bytes per clock only when every 8 consecutive
// lanes stay inside one 128-byte half of the 256-byte bank line (address bit 7
// equal) and take 8 different 16-byte slots there; rows stored in tile order
// alternate between the halves and such a read takes twice as long (measured:
// 1.83 x, SQ_LDS_BANK_CONFLICT = half of SQ_LDS_IDX_ACTIVE).  So inside every
// block of 16 tile rows the rows are stored in the order 0, 8, 1, 9, ... 7, 15
// (lds_row): the 8 rows lanes 0..7 of a fragment read address sit on even LDS
// rows, those of lanes 8..15 on odd ones, and chunk c of tile row r is stored
// in slot c ^ (r & 7).  The copies write LDS linearly (1 KB per instruction),
// so the order only decides which global row a lane of a copy fetches.
//
// Math: v_mfma_f32_16x16x128_f8f6f4 -- one instruction covers the whole 128-wide
// scale block, so every MFMA starts from a zero accumulator and its 4 results
// per lane are folded into the fp32 accumulators with 4 FMAs by
// As[m,kb] * Bs[n/128,kb].  The weight fragment is the MFMA A operand and the
// activation fragment the B operand: a lane then owns one activation row
// (lane % 16) per block, so the activation scale is one register per block
// row, and the weight scale is wave-uniform.
#include <stdlib.h>

#include "gemm_common.h"

using namespace lowp;

namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4v __attribute__((ext_vector_type(4)));

constexpr int BM = 256;             // tile rows (activations)
constexpr int KB = 128;             // bytes per row per step
constexpr int THREADS = 512;
constexpr int QUAD_DEFAULT = 0;    // the four-wave 256 x 256 loop is opt-in (LP_GEMM_QUAD=1)

#define LDS_PTR(p) ((void __attribute__((address_space(3))) *)(p))
#define GLB_PTR(p) ((const void __attribute__((address_space(1))) *)(p))

// LDS row that holds tile row r, the tile row an LDS row holds, and the slot of chunk c of tile row r
__device__ __forceinline__ int lds_row(int r) { return (r & ~15) | ((r & 7) << 1) | ((r >> 3) & 1); }
__device__ __forceinline__ int tile_row(int p) { return (p & ~15) | ((p >> 1) & 7) | ((p & 1) << 3); }
__device__ __forceinline__ int swz(int r, int chunk) { return chunk ^ (r & 7); }
// Weights stored [K, N]: a stage holds 128 contraction rows of 256 bytes; chunk c (16 columns) of row k sits in slot
// c ^ nn_swz(k).  ds_read_b64_tr_b8 takes, per 16 lanes, 8 consecutive rows of one chunk (lane pairs on its two halves):
// the low three bits spread those rows over the 8 slots of a 128-byte half, bit 5 of the row puts the four 16-lane
// groups of an instruction (rows 32 apart) alternately on the two halves (measured conflict free).
__device__ __forceinline__ int nn_swz(int k) { return (k & 7) | (((k >> 5) & 1) << 3); }

// NB = 16-column blocks per wave; TN = 2 * 16 * NB
template <int SDT, int NB>
__global__ __launch_bounds__(THREADS) void gemm_big(const uint8_t *__restrict__ Aq, const void *__restrict__ As,
                                                    const uint8_t *__restrict__ Bq, const void *__restrict__ Bs,
                                                    int64_t M, int64_t N, int64_t K, int64_t tiles_m, int64_t tiles_n,
                                                    void *__restrict__ C, int64_t ldc, int out_dtype)
{
    constexpr int TN = 32 * NB;
    constexpr int A_BYTES = BM * KB, B_BYTES = TN * KB, STAGE = A_BYTES + B_BYTES;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[2 * STAGE];

    int64_t tm, tn;
    if (!gemm::tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
    const int64_t m0 = tm * BM, n0 = tn * TN;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l16 = lane & 15, lq = lane >> 4;
    const int kblocks = (int)(K / KB);

    // ---- DMA plan: wave w, instruction i moves rows 8*(w + 8*i) .. +7 (1 KB)
    const int ld_row = lane >> 3, ld_slot = lane & 7;
    // Rows past the end of a matrix are clamped to its last row: the copies stay branch free,
    // the duplicated data only feeds accumulator rows / columns that are never stored.
    const uint8_t *a_src[BM / 64];
    const uint8_t *b_src[TN / 64];
#pragma unroll
    for (int i = 0; i < BM / 64; ++i) {
        const int row = tile_row(8 * (wave + 8 * i) + ld_row);
        const int64_t m = m0 + row < M ? m0 + row : M - 1;
        a_src[i] = Aq + m * K + swz(row, ld_slot) * 16;
    }
#pragma unroll
    for (int i = 0; i < TN / 64; ++i) {
        const int row = tile_row(8 * (wave + 8 * i) + ld_row);
        const int64_t n = n0 + row < N ? n0 + row : N - 1;
        b_src[i] = Bq + n * K + swz(row, ld_slot) * 16;
    }
    auto issue_stage = [&](int kb, int stage) {
        uint8_t *sa = smem + stage * STAGE, *sb = sa + A_BYTES;
#pragma unroll
        for (int i = 0; i < BM / 64; ++i)
            __builtin_amdgcn_global_load_lds(GLB_PTR(a_src[i] + (int64_t)kb * KB), LDS_PTR(sa + (wave + 8 * i) * 1024), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < TN / 64; ++i)
            __builtin_amdgcn_global_load_lds(GLB_PTR(b_src[i] + (int64_t)kb * KB), LDS_PTR(sb + (wave + 8 * i) * 1024), 16, 0, 0);
    };

    // ---- scales: activation rows of this lane (4 block rows), weight scale blocks of this wave
    int64_t arow[4];
    bool arow_ok[4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
        arow[mb] = m0 + wm * 64 + mb * 16 + l16;
        arow_ok[mb] = arow[mb] < M;
    }
    const int64_t wcol0 = n0 + wn * (TN / 2);                  // first weight row of this wave
    const int64_t sblk0 = wcol0 >> 7;                           // its scale block
    const int64_t sblk1 = (wcol0 + TN / 2 - 1) >> 7;            // scale block of the wave's last row
    const int64_t sblk_max = (N >> 7) - 1;
    const int split_nb = (int)((((sblk0 + 1) << 7) - wcol0) >> 4);   // first 16-col block that uses sblk1

    auto load_scales = [&](int kb, float sa[4], float sb[2]) {
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) sa[mb] = arow_ok[mb] ? gemm::scale_at<SDT>(As, arow[mb] * kblocks + kb) : 0.0f;
        sb[0] = gemm::scale_at<SDT>(Bs, (sblk0 < sblk_max ? sblk0 : sblk_max) * kblocks + kb);
        sb[1] = gemm::scale_at<SDT>(Bs, (sblk1 < sblk_max ? sblk1 : sblk_max) * kblocks + kb);
    };

    f32x4v acc[4][NB];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = f32x4v{0.0f, 0.0f, 0.0f, 0.0f};

    float sa_next[4], sb_next[2];
    issue_stage(0, 0);
    load_scales(0, sa_next, sb_next);
    __syncthreads();

    const f32x4v zero = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int kb = 0; kb < kblocks; ++kb) {
        const int stage = kb & 1;
        float sc[4][2];
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) { sc[mb][0] = sa_next[mb] * sb_next[0]; sc[mb][1] = sa_next[mb] * sb_next[1]; }
        if (kb + 1 < kblocks) {
            issue_stage(kb + 1, stage ^ 1);
            load_scales(kb + 1, sa_next, sb_next);
        }
        const uint8_t *sa = smem + stage * STAGE, *sb = sa + A_BYTES;

        // activation fragments of the wave's 4 block rows: lane reads 32 bytes (chunks 2*lq, 2*lq+1) of its row
        i32x8 af[4];
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
            const int row = wm * 64 + mb * 16 + l16;
            const u32x4 x0 = *(const u32x4 *)(sa + lds_row(row) * KB + swz(row, 2 * lq) * 16);
            const u32x4 x1 = *(const u32x4 *)(sa + lds_row(row) * KB + swz(row, 2 * lq + 1) * 16);
            af[mb] = i32x8{(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int row = wn * (TN / 2) + nb * 16 + l16;
            const u32x4 y0 = *(const u32x4 *)(sb + lds_row(row) * KB + swz(row, 2 * lq) * 16);
            const u32x4 y1 = *(const u32x4 *)(sb + lds_row(row) * KB + swz(row, 2 * lq + 1) * 16);
            const i32x8 wf = i32x8{(int)y0.x, (int)y0.y, (int)y0.z, (int)y0.w, (int)y1.x, (int)y1.y, (int)y1.z, (int)y1.w};
            const int which = nb >= split_nb ? 1 : 0;
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
                const f32x4v p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af[mb], zero, 0, 0, 0, 0, 0, 0);
                const float s = which ? sc[mb][1] : sc[mb][0];
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[mb][nb][r] = __builtin_fmaf(p[r], s, acc[mb][nb][r]);
            }
        }
        __syncthreads();      // waits for the DMA of the next stage and for every wave to leave this one
    }

    // ---- epilogue: lane owns row m = .. + l16 and, per block, columns 4*lq .. 4*lq+3
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
        if (!arow_ok[mb]) continue;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int64_t n = wcol0 + nb * 16 + 4 * lq;
            if (n >= N) continue;
            const f32x4v v = acc[mb][nb];
            if (out_dtype == LP_BF16) {
                u32x2 o = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
                *(u32x2 *)((uint16_t *)C + arow[mb] * ldc + n) = o;
            } else {
                u32x4 o = {f2u(v[0]), f2u(v[1]), f2u(v[2]), f2u(v[3])};
                *(u32x4 *)((float *)C + arow[mb] * ldc + n) = o;
            }
        }
    }
}


// ---------------------------------------------------------------------------------------------
// Hand-scheduled variant: 256 x 256 tile, fp32 scales.  Set-up and epilogue are C++, the K loop
// is the generated assembly in gemm_big_loop.inc (see gen_gemm_loop.py for the register plan).
typedef float f32x16v __attribute__((ext_vector_type(16)));

// One TM x TN tile (256 x 256 with 8 waves, or 128 x 128 with 4): activation rows m0 .. min(m0 + TM, M) - 1
// (rows at or past M are clamped on the way in and masked on the way out, so M may be the end of an
// expert's row range), weight rows n0 .. n0 + TN - 1 of the matrix at Bq / Bs.  Waves are laid out
// (TM / 64) x 2; a wave owns 64 rows x TN / 2 columns.
#define LP_ASM_CLOBBERS                                                                                                   \
    "memory", "scc", "m0", "v30", "v31", "v32", "v33", "v34", "v35", "v36", "v37", "v38", "v39", "v40", "v41", "v42", "v43",    \
        "v44", "v45", "v46", "v47", "v48", "v49", "v50", "v51", "v52", "v53", "v54", "v55", "v56", "v57", "v58", "v59",   \
        "v60", "v61", "v62", "v63", "v64", "v65", "v66", "v67", "v68", "v69", "v70", "v71", "v72", "v73", "v74", "v75",   \
        "v76", "v77", "v78", "v79", "v80", "v81", "v82", "v83", "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91",   \
        "v92", "v93", "v94", "v95", "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106",   \
        "v107", "v108", "v109", "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120",   \
        "v121", "v122", "v123", "v124", "v125", "v126", "v127", "s40", "s41", "s42", "s43", "s44", "s45", "s46", "s47",   \
        "s48", "s49", "s50", "s51", "s52", "s53", "s54", "s55", "s56", "s57", "s58", "s59", "s60", "s61", "s62", "s63",   \
        "s98", "s99"
#define LP_ASM_CLOBBERS_WIDE                                                                                              \
    "memory", "scc", "m0", "v19", "v20", "v21", "v22", "v23", "v24", "v25", "v26", "v27", "v28", "v29", "v30", "v31", "v32",  \
        "v33", "v34", "v35", "v36", "v37", "v38", "v39", "v40", "v41", "v42", "v43", "v44", "v45", "v46", "v47", "v48", "v49",   \
        "v50", "v51", "v52", "v53", "v54", "v55", "v56", "v57", "v58", "v59", "v60", "v61", "v62", "v63", "v64", "v65", "v66",   \
        "v67", "v68", "v69", "v70", "v71", "v72", "v73", "v74", "v75", "v76", "v77", "v78", "v79", "v80", "v81", "v82", "v83",   \
        "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", "v94", "v95", "v96", "v97", "v98", "v99", "v100",  \
        "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109", "v110", "v111", "s40", "s41", "s42", "s43",     \
        "s44", "s45", "s46", "s47", "s48", "s49", "s50", "s51", "s52", "s53", "s54", "s55", "s56", "s57", "s58", "s59", "s60",   \
        "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", "s72", "s73", "s74", "s75", "s76", "s77",   \
        "s78", "s79", "s80", "s81", "s82", "s83", "s84", "s85", "s86", "s87", "s88", "s98", "s99"
#define LP_ASM_CLOBBERS_QUAD                                                                                              \
    "memory", "scc", "m0", "v72", "v73", "v74", "v75", "v76", "v77", "v78", "v79", "v80", "v81", "v82", "v83", "v84",     \
        "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", "v94", "v95", "v96", "v97", "v98", "v99",          \
        "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109", "v110", "v111", "v112",           \
        "v113", "v114", "v115", "v116", "v117", "v118", "v119", "v120", "v121", "v122", "v123", "v124", "v125",           \
        "v126", "v127", "s40", "s41", "s42", "s43", "s44", "s45", "s46", "s47", "s48", "s49", "s50", "s51", "s52",        \
        "s53", "s54", "s55", "s56", "s57", "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", "a10", "a11",      \
        "a12", "a13", "a14", "a15", "a16", "a17", "a18", "a19", "a20", "a21", "a22", "a23", "a24", "a25", "a26",          \
        "a27", "a28", "a29", "a30", "a31", "a32", "a33", "a34", "a35", "a36", "a37", "a38", "a39", "a40", "a41",          \
        "a42", "a43", "a44", "a45", "a46", "a47", "a48", "a49", "a50", "a51", "a52", "a53", "a54", "a55", "a56",          \
        "a57", "a58", "a59", "a60", "a61", "a62", "a63", "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71",          \
        "a72", "a73", "a74", "a75", "a76", "a77", "a78", "a79", "a80", "a81", "a82", "a83", "a84", "a85", "a86",          \
        "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94", "a95", "a96", "a97", "a98", "a99", "a100", "a101",        \
        "a102", "a103", "a104", "a105", "a106", "a107", "a108", "a109", "a110", "a111", "a112", "a113", "a114",           \
        "a115", "a116", "a117", "a118", "a119", "a120", "a121", "a122", "a123", "a124", "a125", "a126", "a127",           \
        "a128", "a129", "a130", "a131", "a132", "a133", "a134", "a135", "a136", "a137", "a138", "a139", "a140",           \
        "a141", "a142", "a143", "a144", "a145", "a146", "a147", "a148", "a149", "a150", "a151", "a152", "a153",           \
        "a154", "a155", "a156", "a157", "a158", "a159", "a160", "a161", "a162", "a163", "a164", "a165", "a166",           \
        "a167", "a168", "a169", "a170", "a171", "a172", "a173", "a174", "a175", "a176", "a177", "a178", "a179",           \
        "a180", "a181", "a182", "a183", "a184", "a185", "a186", "a187", "a188", "a189", "a190", "a191", "a192",           \
        "a193", "a194", "a195", "a196", "a197", "a198", "a199", "a200", "a201", "a202", "a203", "a204", "a205",           \
        "a206", "a207", "a208", "a209", "a210", "a211", "a212", "a213", "a214", "a215", "a216", "a217", "a218",           \
        "a219", "a220", "a221", "a222", "a223", "a224", "a225", "a226", "a227", "a228", "a229", "a230", "a231",           \
        "a232", "a233", "a234", "a235", "a236", "a237", "a238", "a239", "a240", "a241", "a242", "a243", "a244",           \
        "a245", "a246", "a247", "a248", "a249", "a250", "a251", "a252", "a253", "a254", "a255"
#define LP_ASM_INPUTS_WIDE                                                                                                \
    [aoff0] "v"(aoff[0]), [aoff1] "v"(aoff[1]), [aoff2] "v"(aoff[2]), [aoff3] "v"(aoff[3]), [boff0] "v"(boff[0]),         \
        [soff] "v"(soff), [srd] "v"(srd), [ard0] "v"(ard0), [ard1] "v"(ard1), [brd0] "v"(brd0), [brd1] "v"(brd1),         \
        [abase] "s"(a_u), [bbase] "s"(b_u), [sbase] "s"(s_u), [bsptr] "s"(bs_u), [bsptr2] "s"(bs2_u), [m0base] "s"(m0base), \
        [trips] "s"(trips), [flags] "s"(flags), [splitnb] "s"(splitnb), [bextra] "s"(bextra), [bstride] "s"(bstride),       \
        [g4] "s"(g4), [amask0] "s"(amask[0]), [amask1] "s"(amask[1]), [amask2] "s"(amask[2]), [amask3] "s"(amask[3])
#define LP_ASM_INPUTS_NN                                                                                                  \
    [aoff0] "v"(aoff[0]), [aoff1] "v"(aoff[1]), [aoff2] "v"(aoff[2]), [aoff3] "v"(aoff[3]), [boff0] "v"(boff[0]),         \
        [boff1] "v"(boff[1]), [boff2] "v"(boff[2]), [boff3] "v"(boff[3]), [soff] "v"(soff), [srd] "v"(srd),               \
        [ard0] "v"(ard0), [ard1] "v"(ard1), [brdn0] "v"(brdn[0]), [brdn1] "v"(brdn[1]), [brdn2] "v"(brdn[2]),             \
        [brdn3] "v"(brdn[3]), [abase] "s"(a_u), [bbase] "s"(b_u), [sbase] "s"(s_u), [bsptr] "s"(bsn_u),                    \
        [m0base] "s"(m0base), [trips] "s"(trips), [flags] "s"(flags), [bsstride] "s"(bsstride), [bsbfe] "s"(bsbfe),       \
        [bstep] "s"(bstep), [amask0] "s"(amask[0]), [amask1] "s"(amask[1]), [amask2] "s"(amask[2]), [amask3] "s"(amask[3])
#define LP_ASM_INPUTS                                                                                                     \
    [aoff0] "v"(aoff[0]), [aoff1] "v"(aoff[1]), [aoff2] "v"(aoff[2]), [aoff3] "v"(aoff[3]), [boff0] "v"(boff[0]),         \
        [boff1] "v"(boff[1]), [boff2] "v"(boff[2]), [boff3] "v"(boff[3]), [soff] "v"(soff), [srd] "v"(srd),               \
        [ard0] "v"(ard0), [ard1] "v"(ard1), [brd0] "v"(brd0), [brd1] "v"(brd1), [abase] "s"(a_u), [bbase] "s"(b_u),       \
        [sbase] "s"(s_u), [bsptr] "s"(bs_u), [m0base] "s"(m0base), [trips] "s"(trips), [flags] "s"(flags),              \
        [amask0] "s"(amask[0]), [amask1] "s"(amask[1]), [amask2] "s"(amask[2]), [amask3] "s"(amask[3])

// Index arithmetic of the staged bf16 epilogue for a wave tile of 64 rows x COLS columns (COLS = 128, 96 or 64).
// A row of the staging region holds COLS bf16 plus 16 bytes of padding (rows then start 4 banks apart: the 8-byte
// writes of 16 rows spread over the banks instead of hitting the same ones).  Written per accumulator block
// (mb, nb) by lane (l16, lq): row mb * 16 + l16, columns nb * 16 + 4 lq .. + 3.  Read back in 16-byte chunks of 8
// columns: LPR lanes cover a row, 64 / LPR rows per pass.  The same formulas are restated on the host and checked to
// cover every element exactly once and to stay inside the region.
template <int COLS>
struct StagedEpilogue {
    static constexpr int PITCH = COLS * 2 + 16;
    static constexpr int WAVE_BYTES = 64 * PITCH;
    static constexpr int CHUNKS = COLS / 8;                       // 16-byte chunks per row
    static constexpr int PASSES = CHUNKS;                         // 64 rows x CHUNKS chunks, 64 chunks per pass
    __host__ __device__ static constexpr int write_offset(int mb, int nb, int l16, int lq)
    {
        return (mb * 16 + l16) * PITCH + (nb * 16 + 4 * lq) * 2;
    }
    // chunks are read back in row-major order: consecutive lanes take consecutive chunks of a row and go on with the next row
    __host__ __device__ static constexpr int read_row(int pass, int lane) { return (pass * 64 + lane) / CHUNKS; }
    __host__ __device__ static constexpr int read_chunk(int pass, int lane) { return (pass * 64 + lane) % CHUNKS; }
    __host__ __device__ static constexpr int read_offset(int row, int chunk) { return row * PITCH + chunk * 16; }
};

// The same for e4m3 results (one byte per element; the unscaled NT GEMM's fp8 output): a row of the staging region holds
// COLS bytes plus 16 of padding, a lane writes its 4 bytes of block (mb, nb), and 16-byte chunks of 16 columns are read back.
template <int COLS>
struct StagedEpilogueFp8 {
    static constexpr int PITCH = COLS + 16;
    static constexpr int WAVE_BYTES = 64 * PITCH;
    static constexpr int CHUNKS = COLS / 16;
    static constexpr int PASSES = CHUNKS;
    __host__ __device__ static constexpr int write_offset(int mb, int nb, int l16, int lq) { return (mb * 16 + l16) * PITCH + nb * 16 + 4 * lq; }
    __host__ __device__ static constexpr int read_row(int pass, int lane) { return (pass * 64 + lane) / CHUNKS; }
    __host__ __device__ static constexpr int read_chunk(int pass, int lane) { return (pass * 64 + lane) % CHUNKS; }
    __host__ __device__ static constexpr int read_offset(int row, int chunk) { return row * PITCH + chunk * 16; }
};

// WN: waves side by side along N (2, or 4 for the flat 128 x 256 tile); a wave owns 64 rows x TN / WN columns.
template <int TM, int TN, int KSUB, int NST = 2, int WN = 2>
struct AsmTile {
    static constexpr int WAVES = TM / 64 * WN, NBW = TN / WN / 16;
    static constexpr int A_BYTES = TM * KB, B_BYTES = TN * KB;                   // one K block of 128
    static constexpr int B_LDS = NST * KSUB * A_BYTES, S_LDS = NST * KSUB * (A_BYTES + B_BYTES);
    static constexpr int LOOP_BYTES = S_LDS + 2 * TM * 16;                       // NST stages of KSUB K blocks + scale groups
    static constexpr int STAGING = WAVES * StagedEpilogue<TN / WN>::WAVE_BYTES; // the waves' bf16 staging regions after the loop
    static constexpr int LDS_BYTES = LOOP_BYTES > STAGING ? LOOP_BYTES : STAGING;
};

// HWS: e8m0 scales applied by the matrix cores (v_mfma_scale_*); As / Bs then point at bytes.
// DUAL: two groups of WAVES waves work on the same tile, each on one half of K with LDS stages of its own (the loop
// itself is unchanged: both groups run the same trips and meet at the same barriers), and the second group's
// accumulators are added through LDS at the end.  For problems with about one tile per CU, where a workgroup's
// time is its chain of K steps rather than its arithmetic: the chain halves.
// NST: LDS stages (2; 3 for the flat 128 x 256 tile, whose stage in use rotates through registers; 4 for the 128 x 128
// tile with one K block per stage: three K steps in flight).
// BROW: the weights carry an e8m0 scale per row and K block ([N, K/128] bytes) instead of per 128 rows; the matrix
// instruction takes a scale per operand row anyway, so the loop only fetches them differently (hardware-scaled
// 128 x 128 loop: waves 2 and 3 copy the weight-scale dwords of a group while waves 0 and 1 copy the activations').
// STAGED: bf16 results leave through LDS, so that a store instruction writes 16 bytes per lane and whole runs of a row
// (4 rows x 256 contiguous bytes for a 128-column wave tile) instead of 16 rows x 32 bytes.  Each wave turns its own
// 64-row sub-tile in a region of its own (the stage memory, free after the loop), so only the barrier that ends the
// loop's use of that memory is needed.  With DUAL it follows the reduction, in the first K half's stage memory.
//
// Register contract of the asm statements: the loops name v30 .. v255, s40 .. s77 and m0 literally and keep their
// operands (addresses, offsets, counts) live to the end.  Accumulator outputs are therefore early-clobber ("=&"):
// without it the compiler may hand an operand the same register as an output -- the loop zeroes and accumulates into
// it and then loads from a wild offset.  m0 is on the clobber list so that no m0 set-up of the compiler's is assumed
// to survive the loop (clang warns about reserved registers on a clobber list; that is the intent here).
// check_asm_operands.py verifies both on the generated assembly at build time.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
template <int TM, int TN, int KSUB, bool HWS = false, bool DUAL = false, int NST = 2, bool BROW = false, bool STAGED = false, int WN = 2, bool NN = false,
          bool BF16 = false>
__device__ __forceinline__ void tile_asm(uint8_t *smem, const uint8_t *__restrict__ Aq, const float *__restrict__ As,
                                         const uint8_t *__restrict__ Bq, const float *__restrict__ Bs, int64_t m0, int64_t M,
                                         int64_t n0, int64_t N, int64_t K, void *__restrict__ C, int64_t ldc, int out_dtype)
{
    using T = AsmTile<TM, TN, KSUB, NST, WN>;
    constexpr int WAVES = T::WAVES, NBW = T::NBW;
    static_assert(WN == 2 || (WN == 4 && TM == 128 && TN == 256 && KSUB == 1 && !DUAL && NST == 3 && !BROW), "four waves along N: the 128 x 256 tile, three stages");
    // NN: Bq is the weight as stored for C = A W, [K, N] row-major (row pitch N), Bs its [K / 128, N / 128] scale bytes:
    // the 256-row and the flat tile with e8m0 scales (the data gradient of the grouped linear)
    static_assert(!NN || (HWS && TN == 256 && KSUB == 1 && !DUAL && !BROW && ((TM == 256 && WN == 2 && NST == 2) || (TM == 128 && WN == 4 && NST == 3))),
                  "weights stored [K, N]: hardware-scaled 256 x 256 and 128 x 256 tiles");
    static_assert(!DUAL || (TM == 128 && TN == 128), "the K split inside a workgroup is built for the 128 x 128 tile");
    static_assert(NST == 2 || (NST == 3 && WN == 4) || (NST == 4 && TM == 128 && TN == 128 && KSUB == 1 && !DUAL), "three stages: flat tile, four: 128 x 128 tile");
    static_assert(!BROW || (HWS && TM == 128 && TN == 128 && KSUB == 1 && !DUAL && NST == 2), "row-scaled weights: hardware-scaled 128 x 128 loop");
    static_assert((TM / 8 / WAVES == 4 || (WN == 4 && TM / 8 / WAVES == 2)) && (TN / 8 / WAVES == 4 || TN / 8 / WAVES == 3),
                  "copies per operand and wave");
    constexpr int NBC = TN / 8 / WAVES;                 // weight copies per wave and K block
    // The thread index is made opaque: called in a loop over tiles, everything below that depends only on it would otherwise be
    // kept in registers across the previous tile's loop, which leaves the compiler v0 .. v29, and be spilled.
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    const int lane = t & 63, wave = DUAL ? (t >> 6) & (WAVES - 1) : t >> 6;
    const int kg = DUAL ? __builtin_amdgcn_readfirstlane(t >> 6) / WAVES : 0;                 // which half of K
    const int wm = wave / WN, wn = wave % WN;
    const int l16 = lane & 15, lq = lane >> 4;
    const uint32_t kblocks = (uint32_t)(K / KB);
    const uint32_t trips = (DUAL ? kblocks / 2 : kblocks) / 4;
    constexpr int SS = HWS ? 1 : 4;                      // bytes per scale
    if (DUAL) {
        smem += kg * T::LDS_BYTES;
        Aq += (int64_t)kg * (K / 2);
        Bq += (int64_t)kg * (K / 2);
        As = (const float *)((const char *)As + (int64_t)kg * (kblocks / 2) * SS);
        Bs = (const float *)((const char *)Bs + (int64_t)kg * (kblocks / 2) * SS);
    }
    // the bases go into scalar registers: tell the compiler they are wave-uniform
    auto uniform = [](const void *p) -> uint64_t {
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)p);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uintptr_t)p >> 32));
        return ((uint64_t)hi << 32) | lo;
    };
    const bool copies_weights = BROW && wave >= TM / 64;                 // this wave stages weight scales, not activation scales
    const uint64_t a_u = uniform(Aq), b_u = uniform(Bq), s_u = uniform(copies_weights ? Bs : As);

    // DMA source offsets (bytes from the matrix base; the host guarantees they fit 32 bits)
    const int ld_row = lane >> 3, ld_slot = lane & 7;
    uint32_t aoff[4], boff[4];
    uint64_t amask[4];                                  // lanes of activation copy i whose row exists
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = tile_row(8 * (wave + WAVES * i) + ld_row);      // the tile row this lane's 16 bytes of LDS hold
        amask[i] = __ballot(m0 + row < M);
        // a lane whose row is past the end of the activations is switched off for the copy (amask): its offset only has to exist
        const int64_t m = m0 + row < M ? m0 + row : m0;
        const int64_t n = n0 + row < N ? n0 + row : N - 1;          // i = 3 is unused when there are three copies
        aoff[i] = (uint32_t)(m * K + swz(row, ld_slot) * 16);
        boff[i] = (uint32_t)(n * K + swz(row, ld_slot) * 16);
        if constexpr (NN) {
            // a copy moves 4 contraction rows of 256 bytes: lane -> row 4 (wave + WAVES i) + lane / 16 of the K step,
            // slot lane % 16, which holds chunk slot ^ nn_swz(row) of the row (columns n0 + 16 chunk ..)
            const int krow = 4 * (wave + WAVES * i) + (lane >> 4);
            boff[i] = (uint32_t)((int64_t)krow * N + n0 + (((lane & 15) ^ nn_swz(krow)) << 4));
        }
    }
    (void)NBC;
    // activation scales travel in groups of four K steps through LDS: the first TM / 64 waves copy one row per lane
    int64_t arow[4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) arow[mb] = m0 + wm * 64 + mb * 16 + l16;
    const int64_t srow = m0 + (wave % (TM / 64)) * 64 + lane;
    const int64_t wrow = n0 + (wave - TM / 64) * 64 + lane;             // weight row whose scales this lane stages (BROW)
    const uint32_t soff = copies_weights ? (uint32_t)((wrow < N ? wrow : N - 1) * kblocks * SS)
                                         : (uint32_t)((srow < M ? srow : M - 1) * kblocks * SS);
    const uint32_t copies = __builtin_amdgcn_readfirstlane(BROW || wave < TM / 64 ? 1u : 0u);
    // weight scale row(s) of this wave.  With TN / 2 = 128 or 64 columns per wave they lie in one scale block;
    // 96 columns can straddle two, and each pair of 16-column blocks is told which of the two rows it uses.
    const int64_t wcol0 = n0 + wn * (TN / WN);
    const int64_t last_blk = N >= 128 ? (N >> 7) - 1 : 0;       // never in front of the table, whatever the caller's N
    int64_t sblk = wcol0 >> 7;
    if (sblk > last_blk) sblk = last_blk;
    const uint64_t bs_u = uniform((const char *)Bs + sblk * kblocks * SS);
    int64_t sblk2 = (wcol0 + TN / WN - 1) >> 7;
    if (sblk2 > last_blk) sblk2 = last_blk;
    const uint64_t bs2_u = uniform((const char *)Bs + sblk2 * kblocks * SS);
    // pair p covers columns wcol0 + 32 p .. + 31 (within one scale block since wcol0 is a multiple of 32)
    const uint32_t sel1 = __builtin_amdgcn_readfirstlane((uint32_t)(((wcol0 + 32) >> 7) != (wcol0 >> 7)));
    const uint32_t sel2 = __builtin_amdgcn_readfirstlane((uint32_t)(((wcol0 + 64) >> 7) != (wcol0 >> 7)));
    (void)bs2_u; (void)sel1; (void)sel2;
    // 256 x 288 and 256 x 224 tiles: first 16-column block of this wave that lies in the second weight-scale block (past
    // the wave's last block when all its columns lie in one), whether this wave has the one weight copy more that the
    // first four waves have (36 or 28 groups of 8 rows over 8 waves), which group the copy moves whose group depends on
    // the wave (as group g4 + wave; 288: the fifth copy, groups 16, 17 for waves 0, 1 and 34, 35 for waves 2, 3; 224: the
    // third copy, groups 8 .. 13 for waves 0 .. 5 and 22, 23 for waves 6, 7), bytes between two groups of weight rows
    const uint32_t splitnb = __builtin_amdgcn_readfirstlane((uint32_t)(((((wcol0 >> 7) + 1) << 7) - wcol0) >> 4));
    const uint32_t bextra = __builtin_amdgcn_readfirstlane(wave < (TN / 8) % WAVES ? 1u : 0u);
    const uint32_t bstride = __builtin_amdgcn_readfirstlane((uint32_t)(8 * K));
    const uint32_t g4 = __builtin_amdgcn_readfirstlane(TN == 224 ? (wave < 6 ? 8u : 16u) : (wave < 2 ? 16u : 32u));
    // A wave none of whose 64 activation rows exist (the tail of M, or an expert's short tile) runs the loop's
    // copy-and-barrier skeleton only, in the loops generated with that second body (256-row and flat tiles).
    const uint32_t idle = __builtin_amdgcn_readfirstlane((int64_t)wm * 64 >= M - m0 ? 1u : 0u);
    // second half of the workgroup's waves: on every SIMD it shares the matrix pipe with a wave of the first half
    const uint32_t grp = __builtin_amdgcn_readfirstlane((DUAL ? (t >> 6) & (WAVES - 1) : t >> 6) >= WAVES / 2 ? 1u : 0u);
    // the wave's flags travel in one scalar operand: bit 0 copies scales, 1 idle, 2 second half of the waves, 3 first half
    // (read into the scalar register by hand: left to the compiler, the combined value can end up in a vector register,
    // which the loop's scalar instructions cannot take.  The s_nop: the compiler does not look into the statement, and
    // when the instruction it places right in front is the one that writes the vector register, v_readfirstlane reads
    // the register's old value -- seen as waves that copied no activation scales, or the wrong waves' scales.)
    const uint32_t flags_v = copies | idle << 1 | grp << 2 | (grp ^ 1u) << 3;
    uint32_t flags;
    asm volatile("s_nop 4\n\tv_readfirstlane_b32 %0, %1" : "=s"(flags) : "v"(flags_v));
    (void)splitnb; (void)bextra; (void)bstride; (void)g4;

    // LDS addresses: DMA base of this wave, fragment read addresses of this lane (stage 0).
    // Layout: activation stages, weight stages, scale groups.
    const uint32_t lds0 = (uint32_t)(uintptr_t)LDS_PTR(smem);
    const uint32_t m0base = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    const int arow_l = wm * 64 + l16, brow_l = wn * (TN / WN) + l16;
    const uint32_t ard0 = lds0 + lds_row(arow_l) * KB + swz(arow_l, 2 * lq) * 16;
    const uint32_t ard1 = lds0 + lds_row(arow_l) * KB + swz(arow_l, 2 * lq + 1) * 16;
    const uint32_t brd0 = lds0 + T::B_LDS + lds_row(brow_l) * KB + swz(brow_l, 2 * lq) * 16;
    const uint32_t brd1 = lds0 + T::B_LDS + lds_row(brow_l) * KB + swz(brow_l, 2 * lq + 1) * 16;
    // NN: fragment address per block of 16 columns: lane 16 q + s of a transposing read points at half s & 1 of chunk
    // (wn NBW + b) of contraction row 32 q + s / 2 (+ 8 per instruction of the fragment, in the offset field)
    uint32_t brdn[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (NN) {
        const int krow = 32 * lq + (l16 >> 1);
#pragma unroll
        for (int b = 0; b < NBW; ++b)
            brdn[b] = lds0 + T::B_LDS + krow * 256 + (((wn * NBW + b) ^ nn_swz(krow)) << 4) + 8 * (l16 & 1);
    }
    // NN: the wave's weight scales are column (n0 + its first column) / 128 of the [K / 128, N / 128] byte table, one row per
    // K step: the loop loads the aligned dword around each byte (rows are a multiple of 4 bytes apart, checked on the
    // host, so the byte's place in the dword is the same for every step)
    const uint64_t bsn_addr = (uint64_t)(uintptr_t)Bs + (uint64_t)(wcol0 >> 7);
    const uint64_t bsn_u = uniform((const void *)(uintptr_t)(bsn_addr & ~(uint64_t)3));
    const uint32_t bsbfe = __builtin_amdgcn_readfirstlane((uint32_t)((bsn_addr & 3) * 8) | (8u << 16));
    const uint32_t bsstride = __builtin_amdgcn_readfirstlane((uint32_t)(N >> 7));
    const uint32_t bstep = __builtin_amdgcn_readfirstlane((uint32_t)(128 * N));
    (void)bsn_u; (void)bsbfe; (void)bsstride; (void)bstep;
    // scale staging: 16 bytes per activation row (fp32, four K steps), or 4 bytes per row in 1 KB per copying wave (e8m0)
    const uint32_t srd = HWS ? lds0 + T::S_LDS + wm * 1024 + l16 * 4 : lds0 + T::S_LDS + arow_l * 16;
    // row-scaled weights: their dwords live behind the two activation halves, 1 KB per copying wave like those
    const uint32_t sdst = __builtin_amdgcn_readfirstlane((uint32_t)(T::S_LDS + (copies_weights ? 2048 : 0)));
    const uint32_t srdb = lds0 + T::S_LDS + 4096 + wn * 1024 + l16 * 4;
    (void)sdst; (void)srdb;

    f32x16v accs[NBW];
    if constexpr (TN == 288) {
        static_assert(TM == 256 && KSUB == 1 && !DUAL && NST == 2 && !BROW, "the 288-column tile exists for the 256-row kernel only");
        f32x16v acc0, acc1, acc2, acc3, acc4, acc5, acc6, acc7, acc8;
        if constexpr (HWS) {
            asm volatile(
#include "gemm_wide_hw_loop.inc"
                : "=&{v[112:127]}"(acc0), "=&{v[128:143]}"(acc1), "=&{v[144:159]}"(acc2), "=&{v[160:175]}"(acc3),
                  "=&{v[176:191]}"(acc4), "=&{v[192:207]}"(acc5), "=&{v[208:223]}"(acc6), "=&{v[224:239]}"(acc7),
                  "=&{v[240:255]}"(acc8)
                : LP_ASM_INPUTS_WIDE
                : LP_ASM_CLOBBERS_WIDE);
        } else {
            asm volatile(
#include "gemm_wide_loop.inc"
                : "=&{v[112:127]}"(acc0), "=&{v[128:143]}"(acc1), "=&{v[144:159]}"(acc2), "=&{v[160:175]}"(acc3),
                  "=&{v[176:191]}"(acc4), "=&{v[192:207]}"(acc5), "=&{v[208:223]}"(acc6), "=&{v[224:239]}"(acc7),
                  "=&{v[240:255]}"(acc8)
                : LP_ASM_INPUTS_WIDE
                : LP_ASM_CLOBBERS_WIDE);
        }
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3; accs[4] = acc4;
        accs[5] = acc5; accs[6] = acc6; accs[7] = acc7; accs[8] = acc8;
    } else if constexpr (TN == 224) {
        static_assert(TM == 256 && KSUB == 1 && !DUAL && NST == 2 && !BROW, "the 224-column tile exists for the 256-row kernel only");
        f32x16v acc0, acc1, acc2, acc3, acc4, acc5, acc6;
        if constexpr (HWS) {
            asm volatile(
#include "gemm_wide224_hw_loop.inc"
                : "=&{v[112:127]}"(acc0), "=&{v[128:143]}"(acc1), "=&{v[144:159]}"(acc2), "=&{v[160:175]}"(acc3),
                  "=&{v[176:191]}"(acc4), "=&{v[192:207]}"(acc5), "=&{v[208:223]}"(acc6)
                : LP_ASM_INPUTS_WIDE
                : LP_ASM_CLOBBERS_WIDE);
        } else {
            asm volatile(
#include "gemm_wide224_loop.inc"
                : "=&{v[112:127]}"(acc0), "=&{v[128:143]}"(acc1), "=&{v[144:159]}"(acc2), "=&{v[160:175]}"(acc3),
                  "=&{v[176:191]}"(acc4), "=&{v[192:207]}"(acc5), "=&{v[208:223]}"(acc6)
                : LP_ASM_INPUTS_WIDE
                : LP_ASM_CLOBBERS_WIDE);
        }
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3; accs[4] = acc4; accs[5] = acc5; accs[6] = acc6;
    } else if constexpr (NN && WN == 4) {
        f32x16v acc0, acc1, acc2, acc3;
        asm volatile(
#include "gemm_flat_hw_nn_loop.inc"
            : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3)
            : LP_ASM_INPUTS_NN
            : LP_ASM_CLOBBERS, "s64", "s65", "s66", "s89", "s90", "s91", "s92");
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
    } else if constexpr (NN) {
        f32x16v acc0, acc1, acc2, acc3, acc4, acc5, acc6, acc7;
        asm volatile(
#include "gemm_big_hw_nn_loop.inc"
            : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3),
              "=&{v[192:207]}"(acc4), "=&{v[208:223]}"(acc5), "=&{v[224:239]}"(acc6), "=&{v[240:255]}"(acc7)
            : LP_ASM_INPUTS_NN, [brdn4] "v"(brdn[4]), [brdn5] "v"(brdn[5]), [brdn6] "v"(brdn[6]), [brdn7] "v"(brdn[7])
            : LP_ASM_CLOBBERS, "s64", "s65", "s66");
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
        accs[4] = acc4; accs[5] = acc5; accs[6] = acc6; accs[7] = acc7;
    } else if constexpr (WN == 4) {
        // the early hand-back of this loop splits the weight copies by wave: the first four copy each wave column's first half
        f32x16v acc0, acc1, acc2, acc3;
        if constexpr (HWS) {
            asm volatile(
#include "gemm_flat_hw_loop.inc"
                : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3)
                : LP_ASM_INPUTS
                : LP_ASM_CLOBBERS, "s87", "s89", "s90", "s91", "s92");
        } else {
            asm volatile(
#include "gemm_flat_loop.inc"
                : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3)
                : LP_ASM_INPUTS
                : LP_ASM_CLOBBERS, "s87", "s89", "s90", "s91", "s92");
        }
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
    } else if constexpr (HWS && NBW == 8) {
        f32x16v acc0, acc1, acc2, acc3, acc4, acc5, acc6, acc7;
        if constexpr (BF16) {
            // bf16 operands (K counts bytes: two per value): the same loop with two bf16 matrix instructions in place of
            // each fp8 one; the scale operands are read and not used
            asm volatile(
#include "gemm_big_bf16_loop.inc"
                : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3),
                  "=&{v[192:207]}"(acc4), "=&{v[208:223]}"(acc5), "=&{v[224:239]}"(acc6), "=&{v[240:255]}"(acc7)
                : LP_ASM_INPUTS
                : LP_ASM_CLOBBERS);
        } else {
            asm volatile(
#include "gemm_big_hw_loop.inc"
                : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3),
                  "=&{v[192:207]}"(acc4), "=&{v[208:223]}"(acc5), "=&{v[224:239]}"(acc6), "=&{v[240:255]}"(acc7)
                : LP_ASM_INPUTS
                : LP_ASM_CLOBBERS);
        }
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
        accs[4] = acc4; accs[5] = acc5; accs[6] = acc6; accs[7] = acc7;
    } else if constexpr (BROW) {
        f32x16v acc0, acc1, acc2, acc3;
        asm volatile(
#include "gemm_mid_hwrow_loop.inc"
            : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3)
            : LP_ASM_INPUTS, [sdst] "s"(sdst), [srdb] "v"(srdb)
            : LP_ASM_CLOBBERS);
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
    } else if constexpr (HWS && NST == 4) {
        f32x16v acc0, acc1, acc2, acc3;
        asm volatile(
#include "gemm_mid4_hw_loop.inc"
            : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3)
            : LP_ASM_INPUTS
            : LP_ASM_CLOBBERS);
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
    } else if constexpr (NST == 4) {
        f32x16v acc0, acc1, acc2, acc3;
        asm volatile(
#include "gemm_mid4_loop.inc"
            : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3)
            : LP_ASM_INPUTS
            : LP_ASM_CLOBBERS);
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
    } else if constexpr (HWS) {
        f32x16v acc0, acc1, acc2, acc3;
        asm volatile(
#include "gemm_mid_hw_loop.inc"
            : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3)
            : LP_ASM_INPUTS
            : LP_ASM_CLOBBERS);
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
    } else if constexpr (NBW == 8) {
        f32x16v acc0, acc1, acc2, acc3, acc4, acc5, acc6, acc7;
        asm volatile(
#include "gemm_big_loop.inc"
            : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3),
              "=&{v[192:207]}"(acc4), "=&{v[208:223]}"(acc5), "=&{v[224:239]}"(acc6), "=&{v[240:255]}"(acc7)
            : LP_ASM_INPUTS
            : LP_ASM_CLOBBERS);
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
        accs[4] = acc4; accs[5] = acc5; accs[6] = acc6; accs[7] = acc7;
    } else if constexpr (NBW == 6) {
        f32x16v acc0, acc1, acc2, acc3, acc4, acc5;
        asm volatile(
#include "gemm_big192_loop.inc"
            : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3),
              "=&{v[192:207]}"(acc4), "=&{v[208:223]}"(acc5)
            : LP_ASM_INPUTS, [bsptr2] "s"(bs2_u), [sel1] "s"(sel1), [sel2] "s"(sel2)
            : LP_ASM_CLOBBERS, "v224", "v225", "v226", "v227", "v228", "v229", "v230", "v231", "s64", "s65", "s66", "s67",
              "s68", "s69", "s70", "s71", "s72", "s73", "s74", "s75", "s76", "s77");
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3; accs[4] = acc4; accs[5] = acc5;
    } else if constexpr (KSUB == 1) {
        f32x16v acc0, acc1, acc2, acc3;
        asm volatile(
#include "gemm_mid_loop.inc"
            : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3)
            : LP_ASM_INPUTS
            : LP_ASM_CLOBBERS);
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
    } else {
        f32x16v acc0, acc1, acc2, acc3;
        asm volatile(
#include "gemm_mid2_loop.inc"
            : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3)
            : LP_ASM_INPUTS
            : LP_ASM_CLOBBERS);
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
    }

    if constexpr (DUAL) {
        // second half of K: accumulators to LDS (that group's own stages, drained), first half adds and stores
        __syncthreads();
        f32x16v *dump = (f32x16v *)(smem - kg * T::LDS_BYTES + T::LDS_BYTES);          // group 1's region, seen by both
        if (kg == 1) {
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) dump[(wave * NBW + nb) * 64 + lane] = accs[nb];
        }
        __syncthreads();
        if (kg == 1) return;
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
            const f32x16v o = dump[(wave * NBW + nb) * 64 + lane];
#pragma unroll
            for (int r = 0; r < 16; ++r) accs[nb][r] += o[r];
        }
    }
    if constexpr (STAGED) {
        using E = StagedEpilogue<TN / WN>;
        static_assert(WAVES * E::WAVE_BYTES <= T::LDS_BYTES, "the waves' staging regions must fit the tile's LDS");
        if (out_dtype == LP_BF16) {
            // DUAL: only the first K half's waves are left; they stage in their own half's stage memory, which every
            // one of them left before the reduction's barriers (the reduction itself used the other half's), so no
            // barrier is needed -- and none is wanted, the other four waves have ended.
            if constexpr (!DUAL) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");    // this wave's last fragment reads
                __syncthreads();                                      // every wave is done with the stage memory
            }
            uint8_t *stage = smem + wave * E::WAVE_BYTES;
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
                for (int nb = 0; nb < NBW; ++nb) {
                    const u32x2 o = {pack_bf16(accs[nb][mb * 4], accs[nb][mb * 4 + 1]), pack_bf16(accs[nb][mb * 4 + 2], accs[nb][mb * 4 + 3])};
                    *(u32x2 *)(stage + E::write_offset(mb, nb, l16, lq)) = o;
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // a wave reads back only what it wrote: no barrier
            const int64_t row_base = m0 + wm * 64;
#pragma unroll
            for (int p = 0; p < E::PASSES; ++p) {
                const int row = E::read_row(p, lane), chunk = E::read_chunk(p, lane);
                const int64_t n = wcol0 + chunk * 8;
                if (row_base + row < M && n < N) {
                    const u32x4 v = *(const u32x4 *)(stage + E::read_offset(row, chunk));
                    // streaming hint: the result is not read again by this launch, and written this way it leaves the operand
                    // panels in the L2 (config 2 +1-2 %, the grouped launches 1-2 %, the weight gradient's 15 GB of output 3 %).
                    // Only here, where a store instruction writes whole 128-byte lines: the direct stores below write 4 to 16
                    // bytes per lane, and with the hint the unscaled 4096^3 GEMM (4-byte e4m3 stores) took 83 us instead of 55.
                    // Not for the 288- and 224-column tiles: a wave's rows are 288 or 224 bytes there and start in the middle
                    // of a 128-byte line, so neighbouring waves and tiles complete each other's lines, and a line that is
                    // pushed out half written costs the memory side a partial write (config 2 with e8m0 scales, same box:
                    // 179.6 us with plain stores, 182 - 191 with the hint; with no stores at all 173.4).
                    if constexpr (TN == 288 || TN == 224) *(u32x4 *)((uint16_t *)C + (row_base + row) * ldc + n) = v;
                    else __builtin_nontemporal_store(v, (u32x4 *)((uint16_t *)C + (row_base + row) * ldc + n));
                }
            }
            return;
        }
        if constexpr (!DUAL && (TN / WN) % 16 == 0) {
            if (out_dtype == LP_E4M3 && N % 16 == 0 && ldc % 16 == 0 && (uintptr_t)C % 16 == 0) {
                // e4m3fn results (the unscaled NT GEMM routed here) the same way: 4-byte stores per lane cost the 4096^3
                // problem a tenth of its time
                using E8 = StagedEpilogueFp8<TN / WN>;
                static_assert(WAVES * E8::WAVE_BYTES <= T::LDS_BYTES, "the waves' staging regions must fit the tile's LDS");
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __syncthreads();
                uint8_t *stage = smem + wave * E8::WAVE_BYTES;
                auto sat = [](float x) { const float c = __builtin_fminf(__builtin_fmaxf(x, -kE4M3Max), kE4M3Max); return x != x ? x : c; };
#pragma unroll
                for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
                    for (int nb = 0; nb < NBW; ++nb)
                        *(uint32_t *)(stage + E8::write_offset(mb, nb, l16, lq)) =
                            cvt4(sat(accs[nb][mb * 4]), sat(accs[nb][mb * 4 + 1]), sat(accs[nb][mb * 4 + 2]), sat(accs[nb][mb * 4 + 3]));
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                const int64_t row_base = m0 + wm * 64;
#pragma unroll
                for (int p = 0; p < E8::PASSES; ++p) {
                    const int row = E8::read_row(p, lane), chunk = E8::read_chunk(p, lane);
                    const int64_t n = wcol0 + chunk * 16;
                    if (row_base + row < M && n < N) {
                        const u32x4 v = *(const u32x4 *)(stage + E8::read_offset(row, chunk));
                        __builtin_nontemporal_store(v, (u32x4 *)((uint8_t *)C + (row_base + row) * ldc + n));
                    }
                }
                return;
            }
        }
    }
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
        if (arow[mb] >= M) continue;
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
            const int64_t n = wcol0 + nb * 16 + 4 * lq;
            if (n >= N) continue;
            const float v0 = accs[nb][mb * 4], v1 = accs[nb][mb * 4 + 1], v2 = accs[nb][mb * 4 + 2], v3 = accs[nb][mb * 4 + 3];
            if (out_dtype == LP_E4M3) {
                // e4m3fn output (the unscaled NT GEMM routed here): round to nearest even, saturate at +-448, NaN stays NaN
                auto sat = [](float x) { const float c = __builtin_fminf(__builtin_fmaxf(x, -kE4M3Max), kE4M3Max); return x != x ? x : c; };
                *(uint32_t *)((uint8_t *)C + arow[mb] * ldc + n) = cvt4(sat(v0), sat(v1), sat(v2), sat(v3));
            } else if (out_dtype == LP_BF16) {
                u32x2 o = {pack_bf16(v0, v1), pack_bf16(v2, v3)};
                *(u32x2 *)((uint16_t *)C + arow[mb] * ldc + n) = o;
            } else {
                u32x4 o = {f2u(v0), f2u(v1), f2u(v2), f2u(v3)};
                *(u32x4 *)((float *)C + arow[mb] * ldc + n) = o;
            }
        }
    }
}


// The 256 x 256 tile on four waves of 128 x 128 with the accumulators in a[0:255] (gen_gemm_quad_loop.py): e8m0 scales,
// whole tiles only (M and N multiples of 256, K of 512).  The loop statement leaves the accumulators of the wave's first
// 64 rows in v[128:255], laid out like tile_asm's (block nb of 16 columns at v[128 + 16 nb : +15], register 4 mb + r of
// lane (l16, lq) = row 16 mb + l16, column 16 nb + 4 lq + r); a second statement fetches the other 64 rows.  The compiler
// is told that the loop clobbers every accumulation register, and nothing between the two statements may use one: the
// build audit fails if the kernel's assembly names an accumulation register outside the statements.
__device__ __forceinline__ void tile_quad(uint8_t *smem, const uint8_t *__restrict__ Aq, const uint8_t *__restrict__ As,
                                          const uint8_t *__restrict__ Bq, const uint8_t *__restrict__ Bs, int64_t m0, int64_t n0,
                                          int64_t M, int64_t N, int64_t K, void *__restrict__ C, int64_t ldc, int out_dtype)
{
    constexpr int WAVES = 4, A_BYTES = 256 * KB, B_LDS = 2 * A_BYTES, S_LDS = 4 * A_BYTES;
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l16 = lane & 15, lq = lane >> 4;
    const uint32_t kblocks = (uint32_t)(K / KB);
    const uint32_t trips = kblocks / 4;
    auto uniform = [](const void *p) -> uint64_t {
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)p);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uintptr_t)p >> 32));
        return ((uint64_t)hi << 32) | lo;
    };
    const int64_t wcol0 = n0 + wn * 128;
    const uint64_t a_u = uniform(Aq), b_u = uniform(Bq), s_u = uniform(As), bs_u = uniform(Bs + (wcol0 >> 7) * kblocks);
    // copy i of this wave moves the 8 LDS rows 8 (wave + 4 i) ..: lane -> row lane / 8 of them, 16-byte slot lane % 8
    const int ld_row = lane >> 3, ld_slot = lane & 7;
    uint32_t aoff[8], boff[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int row = tile_row(8 * (wave + WAVES * i) + ld_row);
        aoff[i] = (uint32_t)((m0 + row) * K + swz(row, ld_slot) * 16);
        boff[i] = (uint32_t)((n0 + row) * K + swz(row, ld_slot) * 16);
    }
    // scale bytes of a group of four K steps: each wave copies the dwords of 64 activation rows (one per lane) and its own
    // weight-scale dword into every lane's slot
    const uint32_t soff = (uint32_t)((m0 + wave * 64 + lane) * kblocks);
    uint32_t zero = 0;
    asm volatile("" : "+v"(zero));
    const uint32_t lds0 = (uint32_t)(uintptr_t)LDS_PTR(smem);
    const uint32_t m0base = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    const uint32_t s0base = __builtin_amdgcn_readfirstlane(lds0 + S_LDS + wave * 256);
    const int arow_l = wm * 128 + l16, brow_l = wn * 128 + l16;
    const uint32_t ard0 = lds0 + lds_row(arow_l) * KB + swz(arow_l, 2 * lq) * 16;
    const uint32_t ard1 = lds0 + lds_row(arow_l) * KB + swz(arow_l, 2 * lq + 1) * 16;
    const uint32_t brd0 = lds0 + B_LDS + lds_row(brow_l) * KB + swz(brow_l, 2 * lq) * 16;
    const uint32_t brd1 = lds0 + B_LDS + lds_row(brow_l) * KB + swz(brow_l, 2 * lq + 1) * 16;
    const uint32_t srd = lds0 + S_LDS + arow_l * 4;
    const uint32_t wsrd = lds0 + S_LDS + 1024 + wave * 256 + lane * 4;

    f32x16v accs[8];
    {
        f32x16v acc0, acc1, acc2, acc3, acc4, acc5, acc6, acc7;
        asm volatile(
#include "gemm_quad_hw_loop.inc"
            : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3),
              "=&{v[192:207]}"(acc4), "=&{v[208:223]}"(acc5), "=&{v[224:239]}"(acc6), "=&{v[240:255]}"(acc7)
            : [aoff0] "v"(aoff[0]), [aoff1] "v"(aoff[1]), [aoff2] "v"(aoff[2]), [aoff3] "v"(aoff[3]), [aoff4] "v"(aoff[4]),
              [aoff5] "v"(aoff[5]), [aoff6] "v"(aoff[6]), [aoff7] "v"(aoff[7]), [boff0] "v"(boff[0]), [boff1] "v"(boff[1]),
              [boff2] "v"(boff[2]), [boff3] "v"(boff[3]), [boff4] "v"(boff[4]), [boff5] "v"(boff[5]), [boff6] "v"(boff[6]),
              [boff7] "v"(boff[7]), [soff] "v"(soff), [zero] "v"(zero), [srd] "v"(srd), [wsrd] "v"(wsrd), [ard0] "v"(ard0),
              [ard1] "v"(ard1), [brd0] "v"(brd0), [brd1] "v"(brd1), [abase] "s"(a_u), [bbase] "s"(b_u), [sbase] "s"(s_u),
              [bsptr] "s"(bs_u), [m0base] "s"(m0base), [s0base] "s"(s0base), [trips] "s"(trips)
            : LP_ASM_CLOBBERS_QUAD);
        accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
        accs[4] = acc4; accs[5] = acc5; accs[6] = acc6; accs[7] = acc7;
    }
    using E = StagedEpilogue<128>;
    static_assert(WAVES * E::WAVE_BYTES <= S_LDS, "the waves' staging regions must fit the stage memory");
    __syncthreads();                                      // every wave is done with the stage memory
    uint8_t *stage = smem + wave * E::WAVE_BYTES;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        if (half == 1) {
            f32x16v acc0, acc1, acc2, acc3, acc4, acc5, acc6, acc7;
            asm volatile(
#include "gemm_quad_tail_loop.inc"
                : "=&{v[128:143]}"(acc0), "=&{v[144:159]}"(acc1), "=&{v[160:175]}"(acc2), "=&{v[176:191]}"(acc3),
                  "=&{v[192:207]}"(acc4), "=&{v[208:223]}"(acc5), "=&{v[224:239]}"(acc6), "=&{v[240:255]}"(acc7)
                :
                : "memory");
            accs[0] = acc0; accs[1] = acc1; accs[2] = acc2; accs[3] = acc3;
            accs[4] = acc4; accs[5] = acc5; accs[6] = acc6; accs[7] = acc7;
        }
        const int64_t row_base = m0 + wm * 128 + half * 64;
        if (out_dtype == LP_BF16) {
            // through LDS, so that a store instruction writes whole 128-byte lines (see tile_asm); a wave reads back only
            // what it wrote, in a region of its own
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
                for (int nb = 0; nb < 8; ++nb) {
                    const u32x2 o = {pack_bf16(accs[nb][mb * 4], accs[nb][mb * 4 + 1]), pack_bf16(accs[nb][mb * 4 + 2], accs[nb][mb * 4 + 3])};
                    *(u32x2 *)(stage + E::write_offset(mb, nb, l16, lq)) = o;
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int p = 0; p < E::PASSES; ++p) {
                const int row = E::read_row(p, lane), chunk = E::read_chunk(p, lane);
                const u32x4 v = *(const u32x4 *)(stage + E::read_offset(row, chunk));
                __builtin_nontemporal_store(v, (u32x4 *)((uint16_t *)C + (row_base + row) * ldc + wcol0 + chunk * 8));
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the other half's staging writes follow
            continue;
        }
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
            const int64_t row = row_base + mb * 16 + l16;
#pragma unroll
            for (int nb = 0; nb < 8; ++nb) {
                const int64_t n = wcol0 + nb * 16 + 4 * lq;
                const float v0 = accs[nb][mb * 4], v1 = accs[nb][mb * 4 + 1], v2 = accs[nb][mb * 4 + 2], v3 = accs[nb][mb * 4 + 3];
                if (out_dtype == LP_E4M3) {
                    auto sat = [](float x) { const float c = __builtin_fminf(__builtin_fmaxf(x, -kE4M3Max), kE4M3Max); return x != x ? x : c; };
                    *(uint32_t *)((uint8_t *)C + row * ldc + n) = cvt4(sat(v0), sat(v1), sat(v2), sat(v3));
                } else {
                    u32x4 o = {f2u(v0), f2u(v1), f2u(v2), f2u(v3)};
                    *(u32x4 *)((float *)C + row * ldc + n) = o;
                }
            }
        }
    }
    (void)M; (void)N;
}

#pragma clang diagnostic pop

template <int TM, int TN, int KSUB, bool HWS = false, int NST = 2>
__global__ __launch_bounds__(TM * 2) void gemm_asm(const uint8_t *__restrict__ Aq, const float *__restrict__ As,
                                                   const uint8_t *__restrict__ Bq, const float *__restrict__ Bs, int64_t M,
                                                   int64_t N, int64_t K, int64_t tiles_m, int64_t tiles_n,
                                                   void *__restrict__ C, int64_t ldc, int out_dtype)
{
    __shared__ __attribute__((aligned(1024))) uint8_t smem[AsmTile<TM, TN, KSUB, NST>::LDS_BYTES];
    int64_t tm, tn;
    if (!gemm::tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
    tile_asm<TM, TN, KSUB, HWS, false, NST, false, true>(smem, Aq, As, Bq, Bs, tm * TM, M, tn * TN, N, K, C, ldc, out_dtype);
}

// The unscaled bf16 NT GEMM on the 256 x 256 loop (tile_asm with BF16): row_bytes = 2 K, every scale byte 2^0.
__global__ __launch_bounds__(512) void gemm_asm_bf16(const uint8_t *__restrict__ A, const float *__restrict__ ones,
                                                     const uint8_t *__restrict__ B, int64_t M, int64_t N, int64_t row_bytes,
                                                     int64_t tiles_m, int64_t tiles_n, void *__restrict__ C, int64_t ldc, int out_dtype)
{
    __shared__ __attribute__((aligned(1024))) uint8_t smem[AsmTile<256, 256, 1>::LDS_BYTES];
    int64_t tm, tn;
    if (!gemm::tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
    tile_asm<256, 256, 1, true, false, 2, false, true, 2, false, true>(smem, A, ones, B, ones, tm * 256, M, tn * 256, N, row_bytes, C, ldc, out_dtype);
}

// 256 x 288 tiles: N = 18432 is 64 of them, so a 2048-row problem is 512 tiles, exactly two rounds on 256 CUs.
// 256 x 224 tiles: N = 7168 is 32 of them, so 4096 rows are 512 tiles where 256 x 256 tiles make 448 (1.75 rounds).
template <bool HWS, int TN = 288>
__global__ __launch_bounds__(512) void gemm_asm_wide(const uint8_t *__restrict__ Aq, const float *__restrict__ As,
                                                     const uint8_t *__restrict__ Bq, const float *__restrict__ Bs, int64_t M,
                                                     int64_t N, int64_t K, int64_t tiles_m, int64_t tiles_n,
                                                     void *__restrict__ C, int64_t ldc, int out_dtype)
{
    __shared__ __attribute__((aligned(1024))) uint8_t smem[AsmTile<256, TN, 1>::LDS_BYTES];
    int64_t tm, tn;
    if (!gemm::tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
    tile_asm<256, TN, 1, HWS, false, 2, false, true>(smem, Aq, As, Bq, Bs, tm * 256, M, tn * TN, N, K, C, ldc, out_dtype);
}

// 256 x 256 tiles on four waves with the accumulators in the accumulation registers (tile_quad): e8m0 scales, whole tiles.
__global__ __launch_bounds__(256) void gemm_asm_quad(const uint8_t *__restrict__ Aq, const uint8_t *__restrict__ As,
                                                     const uint8_t *__restrict__ Bq, const uint8_t *__restrict__ Bs, int64_t M,
                                                     int64_t N, int64_t K, int64_t tiles_m, int64_t tiles_n,
                                                     void *__restrict__ C, int64_t ldc, int out_dtype)
{
    __shared__ __attribute__((aligned(1024))) uint8_t smem[4 * 256 * KB + 4096];
    int64_t tm, tn;
    if (!gemm::tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
    tile_quad(smem, Aq, As, Bq, Bs, tm * 256, tn * 256, M, N, K, C, ldc, out_dtype);
}

// 128 x 128 tile with the K split inside the workgroup (see tile_asm): 8 waves, two sets of LDS stages.
template <int KSUB, bool HWS>
__global__ __launch_bounds__(512) void gemm_asm_dual(const uint8_t *__restrict__ Aq, const float *__restrict__ As,
                                                     const uint8_t *__restrict__ Bq, const float *__restrict__ Bs, int64_t M,
                                                     int64_t N, int64_t K, int64_t tiles_m, int64_t tiles_n,
                                                     void *__restrict__ C, int64_t ldc, int out_dtype)
{
    __shared__ __attribute__((aligned(1024))) uint8_t smem[2 * AsmTile<128, 128, KSUB>::LDS_BYTES];
    int64_t tm, tn;
    if (!gemm::tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
    tile_asm<128, 128, KSUB, HWS, true, 2, false, true>(smem, Aq, As, Bq, Bs, tm * 128, M, tn * 128, N, K, C, ldc, out_dtype);
}

// One launch for a problem split by columns: 256 x 256 tiles on weight rows [0, n_big) and K-split 128 x 128 tiles on the
// rest (what gemm_asm<256, 256, 1> followed by gemm_asm_dual would do in two launches).  The big tiles come first in the
// grid; a CU that has finished its last big tile goes on with the small ones, so the launch gap and the uneven end
// of the big tiles' last round are not waited for.  grid_big is a multiple of 8, so both parts keep their XCD mapping.
template <bool HWS>
__global__ __launch_bounds__(512) void gemm_asm_mixed(const uint8_t *__restrict__ Aq, const float *__restrict__ As,
                                                      const uint8_t *__restrict__ Bq, const float *__restrict__ Bs, int64_t M,
                                                      int64_t N, int64_t K, int64_t n_big, int64_t grid_big, void *__restrict__ C,
                                                      int64_t ldc, int out_dtype)
{
    constexpr int LDS_BIG = AsmTile<256, 256, 1>::LDS_BYTES, LDS_DUAL = 2 * AsmTile<128, 128, 1>::LDS_BYTES;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[LDS_BIG > LDS_DUAL ? LDS_BIG : LDS_DUAL];
    int64_t tm, tn;
    if ((int64_t)blockIdx.x < grid_big) {
        if (!gemm::tile_coords(blockIdx.x, (M + 255) / 256, n_big / 256, tm, tn)) return;
        tile_asm<256, 256, 1, HWS, false, 2, false, true>(smem, Aq, As, Bq, Bs, tm * 256, M, tn * 256, n_big, K, C, ldc, out_dtype);
    } else {
        const int64_t n_small = N - n_big;
        if (!gemm::tile_coords(blockIdx.x - grid_big, (M + 127) / 128, n_small / 128, tm, tn)) return;
        const char *bs = (const char *)Bs + (n_big / 128) * (K / KB) * (HWS ? 1 : 4);
        char *c = (char *)C + n_big * (out_dtype == LP_BF16 ? 2 : 4);
        tile_asm<128, 128, 1, HWS, true, 2, false, true>(smem, Aq, As, Bq + n_big * K, (const float *)bs, tm * 128, M, tn * 128,
                                                         n_small, K, c, ldc, out_dtype);
    }
}

// 128 x 128 tiles, e8m0 scales per row and K block on both operands (the weight-gradient GEMM of the grouped linear).
__global__ __launch_bounds__(256) void gemm_asm_rowscale(const uint8_t *__restrict__ Aq, const float *__restrict__ As,
                                                         const uint8_t *__restrict__ Bq, const float *__restrict__ Bs, int64_t M,
                                                         int64_t N, int64_t K, int64_t tiles_m, int64_t tiles_n,
                                                         void *__restrict__ C, int64_t ldc, int out_dtype)
{
    __shared__ __attribute__((aligned(1024))) uint8_t smem[AsmTile<128, 128, 1>::LDS_BYTES + 4096];
    int64_t tm, tn;
    if (!gemm::tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
    tile_asm<128, 128, 1, true, false, 2, true, true>(smem, Aq, As, Bq, Bs, tm * 128, M, tn * 128, N, K, C, ldc, out_dtype);
}

// The same for a list of problems that share M and N and differ in K (the weight gradients of the experts of a grouped
// linear): entry g of `groups` = {output slot, K blocks of 128, K blocks of all problems before it in the operand
// buffers, unused}.  Problem g reads Aq + M * 128 * before (its [M, K_g] codes), As + M * before, the same for B with
// N, and writes C + slot * M * N.  per_group workgroups (a multiple of 256) belong to each entry.
__global__ __launch_bounds__(256) void gemm_asm_rowscale_grouped(const uint8_t *__restrict__ Aq, const float *__restrict__ As,
                                                                 const uint8_t *__restrict__ Bq, const float *__restrict__ Bs,
                                                                 const int32_t *__restrict__ groups, int64_t M, int64_t N,
                                                                 int64_t tiles_m, int64_t tiles_n, int64_t per_group,
                                                                 void *__restrict__ C, int out_dtype, int max_k_blocks)
{
    __shared__ __attribute__((aligned(1024))) uint8_t smem[AsmTile<128, 128, 1>::LDS_BYTES + 4096];
    const int64_t g = blockIdx.x / per_group, local = blockIdx.x - g * per_group;
    int64_t tm, tn;
    if (!gemm::tile_coords(local, tiles_m, tiles_n, tm, tn)) return;
    const int64_t slot = groups[4 * g], kb = groups[4 * g + 1], before = groups[4 * g + 2];
    // an entry that breaks the caller's promise writes nothing: more K blocks than max_k_blocks (on which the host checked
    // that the operands fit 32-bit offsets), a count that is not a multiple of four (the loop works in groups of four
    // K blocks and would silently drop the rest), a negative slot or offset
    if (kb <= 0 || kb > max_k_blocks || (kb & 3) || slot < 0 || before < 0) return;
    char *c = (char *)C + slot * M * N * (out_dtype == LP_BF16 ? 2 : 4);
    tile_asm<128, 128, 1, true, false, 2, true, true>(smem, Aq + M * 128 * before, (const float *)((const char *)As + M * before),
                                                      Bq + N * 128 * before, (const float *)((const char *)Bs + N * before), tm * 128, M,
                                                      tn * 128, N, kb * 128, c, N, out_dtype);
}

// Grouped variant: expert e owns rows m_offsets[e] .. m_offsets[e+1]-1 and the weight matrix e of Bq / Bs.
// The grid is sized from an upper bound on the number of row tiles; each workgroup finds its expert with a
// block-wide scan over the per-expert tile counts.  PART selects which rows of every expert a launch covers:
//   0  all rows, in tiles of TM (the last tile of an expert may be partly empty)
//   1  only the full 256-row tiles (TM = 256)
//   2  what PART 1 leaves, i.e. the last M_e % 256 rows, in tiles of TM
// Launching 1 with 256 x 256 tiles and then 2 with 128 x 128 tiles keeps the large tiles full and bounds the
// padding of an expert by 127 rows.
template <int TM, int TN, int KSUB, int PART, bool HWS = false>
__global__ __launch_bounds__(TM * 2) void gemm_asm_grouped(const uint8_t *__restrict__ Aq, const float *__restrict__ As,
                                                           const uint8_t *__restrict__ Bq, const float *__restrict__ Bs,
                                                           const int32_t *__restrict__ m_offsets, int E, int64_t M_total,
                                                           int64_t N, int64_t K, int64_t max_mtiles, int64_t tiles_n,
                                                           void *__restrict__ C, int out_dtype)
{
    constexpr int NT = TM * 2;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[AsmTile<TM, TN, KSUB>::LDS_BYTES];
    __shared__ int wave_total[NT / 64];
    __shared__ int found_e, found_first;
    int64_t gmt, tn;
    const bool in_range = gemm::tile_coords(blockIdx.x, max_mtiles, tiles_n, gmt, tn, true, gridDim.x);
    const int t = threadIdx.x;
    if (t == 0) found_e = -1;
    auto tiles_of = [](int rows) -> int {
        if (PART == 1) return rows / TM;
        if (PART == 2) rows %= 256;
        return (rows + TM - 1) / TM;
    };
    // Which expert owns row tile gmt: a prefix sum over the experts' tile counts, NT experts at a time -- inside a
    // wave by shuffles, across the waves through their totals (two barriers per NT experts).
    int base = 0;
    for (int e0 = 0; e0 < E; e0 += NT) {
        const int e = e0 + t;
        int64_t unused;
        const int cnt = e < E ? tiles_of(gemm::expert_rows(m_offsets, e, M_total, unused)) : 0;
        int incl = cnt;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int up = __shfl_up(incl, off);
            if ((t & 63) >= off) incl += up;
        }
        if ((t & 63) == 63) wave_total[t >> 6] = incl;
        __syncthreads();                                       // also orders found_e = -1 before the write below
        int before = base, all = 0;
#pragma unroll
        for (int w = 0; w < NT / 64; ++w) {
            const int v = wave_total[w];
            if (w < (t >> 6)) before += v;
            all += v;
        }
        incl += before;
        if (in_range && e < E && gmt >= incl - cnt && gmt < incl) { found_e = e; found_first = incl - cnt; }
        base += all;
        __syncthreads();
    }
    if (!in_range || found_e < 0) return;
    const int e = found_e;
    int64_t row_begin;
    const int64_t row_end = gemm::expert_rows(m_offsets, e, M_total, row_begin) + row_begin;
    const int64_t first = PART == 2 ? row_begin + (row_end - row_begin) / 256 * 256 : row_begin;
    const int64_t kblocks = K / KB;
    const float *bs_e = (const float *)((const char *)Bs + (int64_t)e * (N / 128) * kblocks * (HWS ? 1 : 4));
    tile_asm<TM, TN, KSUB, HWS, false, 2, false, true>(smem, Aq, As, Bq + (int64_t)e * N * K, bs_e, first + (gmt - found_first) * TM, row_end,
                                tn * TN, N, K, C, N, out_dtype);
}

// Grouped problem in ONE launch with two tile heights.  Every 256 rows of an expert, and a remainder of more than 128
// rows, go to a 256 x 256 tile (class "big"); a remainder of 1 .. 128 rows goes to a 128 x 256 tile (class "small": eight
// waves as 2 x 4, half the activation rows per step for the same 256 weight rows).  What a tile costs a CU is mostly the
// bytes it pulls through the L2 -> LDS copies, and an expert with few rows is a stream of its weights: the flat tile
// moves 48 KB per K step and 256 weight rows where two 128 x 128 tiles move 64 KB.
// The tile list is built on the device from m_offsets (at most 512 experts): one scan gives every thread the two class
// totals and the running tile counts of its expert, from which the workgroup finds its class, its tile and the expert
// that owns it.  Within every XCD's sequence of workgroup ids the two classes are dealt in the ratio of their sizes
// (1 big : ps small), and each class keeps the 8(M) x 4(N) blocks of neighbouring tiles per XCD that let operand panels
// be re-used out of one L2.
constexpr int kMixedMaxExperts = 512;

// NN: expert e's weight is stored [K, N] (the layer's own [out, in] weight read for the data gradient dX = dY W: K = out
// features = the contraction, N = in features = the columns of C), its scale bytes [K / 128, N / 128].
template <bool HWS, bool NN = false>
__global__ __launch_bounds__(512) void gemm_asm_grouped_mixed(const uint8_t *__restrict__ Aq, const float *__restrict__ As,
                                                              const uint8_t *__restrict__ Bq, const float *__restrict__ Bs,
                                                              const int32_t *__restrict__ m_offsets, int E, int64_t M_total,
                                                              int64_t N, int64_t K, void *__restrict__ C, int out_dtype, int small_first)
{
    constexpr int LDS_BIG = AsmTile<256, 256, 1>::LDS_BYTES, LDS_FLAT = AsmTile<128, 256, 1, 3, 4>::LDS_BYTES;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[LDS_BIG > LDS_FLAT ? LDS_BIG : LDS_FLAT];
    __shared__ int wave_big[8], wave_small[8];
    // row tiles of the experts up to and including e, per class (what a workgroup searches for its tile's expert)
    __shared__ int upto_big[kMixedMaxExperts], upto_small[kMixedMaxExperts];
    constexpr int kTable = 256;
    __shared__ int4 table[kTable];                      // this workgroup's next tiles
    const int t = threadIdx.x, lane = t & 63, wv = t >> 6;
    int tot_big = 0, tot_small = 0;
    {
        // thread t's expert: rows, tiles of both classes, running counts over the experts before it
        int64_t begin = 0;
        const int rows = t < E ? gemm::expert_rows(m_offsets, t, M_total, begin) : 0;
        const int rem = rows & 255;
        const int nb = (rows >> 8) + (rem > 128 ? 1 : 0), ns = rem > 0 && rem <= 128 ? 1 : 0;
        int ib = nb, is = ns;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int ub = __shfl_up(ib, off), us = __shfl_up(is, off);
            if (lane >= off) { ib += ub; is += us; }
        }
        if (lane == 63) { wave_big[wv] = ib; wave_small[wv] = is; }
        __syncthreads();
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            const int vb = wave_big[w], vs = wave_small[w];
            if (w < wv) { ib += vb; is += vs; }
            tot_big += vb;
            tot_small += vs;
        }
        upto_big[t] = ib;
        upto_small[t] = is;
    }
    tot_big = __builtin_amdgcn_readfirstlane(tot_big);
    tot_small = __builtin_amdgcn_readfirstlane(tot_small);
    // ---- which class and which tile of it this workgroup takes (32-bit arithmetic: the grid is below 2^31, and 64-bit
    // divisions by run-time values would cost this prologue about a microsecond per workgroup)
    const uint32_t tiles_n = (uint32_t)(N >> 8);
    auto padded_slots = [](uint32_t tiles) -> uint32_t {                   // workgroups per XCD for that many tiles
        const uint32_t chunks = (tiles + gemm::CHUNK - 1) / gemm::CHUNK;
        return ((chunks + 7) / 8) * gemm::CHUNK;
    };
    const uint32_t slots_big = padded_slots((uint32_t)tot_big * tiles_n), slots_small = padded_slots((uint32_t)tot_small * tiles_n);
    // A workgroup takes slots blockIdx.x, blockIdx.x + gridDim.x, ...: with one workgroup per CU (grid = number of CUs, a
    // multiple of 8, so a workgroup stays on its XCD's share of the slots) the scan above is paid once per CU instead of
    // once per tile; with a grid of all slots the loop below runs once.  The workgroup's tiles are looked up kTable slots at a
    // time, one slot per thread, and listed in LDS: between two tiles only a table entry is read (a workgroup has its CU to
    // itself, so whatever happens between two K loops is time the matrix cores stand still).
    __syncthreads();                                    // the running counts are written
    const uint32_t slots = slots_big + slots_small;
    const uint64_t all_slots = (uint64_t)slots * 8;     // below 2^31
    const int64_t kblocks = K / KB;
    for (uint64_t first = blockIdx.x; first < all_slots; first += (uint64_t)kTable * gridDim.x) {
        __syncthreads();                                // every thread has read the previous batch's last entry
        if (t < kTable) {
            const uint64_t slot64 = first + (uint64_t)t * gridDim.x;
            int4 entry = {-1, 0, 0, 0};                 // expert (-1: no tile; bit 30: 256-row tile), first row, end of the expert's rows, first column
            if (slot64 < all_slots) {
                const uint32_t slot = (uint32_t)slot64;
                const uint32_t xcd = slot & 7, sidx = slot >> 3;
                bool big;
                uint32_t idx;
                if (small_first > 0) {
                    // XCDs below small_first work through their small tiles first and then their big ones, the others the
                    // other way round: every XCD has the same share of both classes, and at any time some XCDs stream weights
                    // while the others compute, each class with an L2 to itself
                    if (xcd < (uint32_t)small_first) { big = sidx >= slots_small; idx = big ? sidx - slots_small : sidx; }
                    else { big = sidx < slots_big; idx = big ? sidx : sidx - slots_big; }
                } else {
                    // the classes dealt alternately in the ratio of their sizes (1 big : ps small)
                    uint32_t ps = slots_big > 0 ? (slots_small + slots_big / 2) / slots_big : 1;
                    if (ps < 1) ps = 1;
                    const uint32_t period = 1 + ps;
                    const uint32_t rounds = slots_big < slots_small / ps ? slots_big : slots_small / ps;      // periods in which both classes have tiles
                    if (sidx < rounds * period) {
                        const uint32_t q = sidx / period, rr = sidx - q * period;
                        big = rr == 0;
                        idx = big ? q : q * ps + (rr - 1);
                    } else {
                        const uint32_t w = sidx - rounds * period, left_big = slots_big - rounds;
                        big = w < left_big;
                        idx = big ? rounds + w : rounds * ps + (w - left_big);
                    }
                }
                // Tiles of a class are numbered expert by expert (expert e owns tiles_n numbers per row tile) and an XCD takes
                // 32 consecutive numbers at a time, so the tiles it runs together belong to one expert, or to neighbours.
                const uint32_t lin = ((idx / gemm::CHUNK) * 8 + xcd) * gemm::CHUNK + idx % gemm::CHUNK;
                if (lin < (uint32_t)(big ? tot_big : tot_small) * tiles_n) {
                    const int gmt = (int)(lin / tiles_n);
                    // the expert that owns row tile gmt of the class: the first whose running count exceeds gmt
                    const int *upto = big ? upto_big : upto_small;
                    int e = 0;
                    for (int span = kMixedMaxExperts / 2; span > 0; span >>= 1)
                        if (upto[e + span - 1] <= gmt) e += span;
                    if (e < E) {
                        const int before = e > 0 ? upto[e - 1] : 0, cnt = upto[e] - before;
                        int64_t row_begin;
                        const int rows = gemm::expert_rows(m_offsets, e, M_total, row_begin);
                        // Inside the expert: groups of 8 row tiles (the last may be short), in a group blocks of gn column
                        // tiles with the row tile running fastest, gn such that a block is about 32 tiles: the 32 tiles an XCD
                        // runs together share gm activation panels and gn weight panels of one expert (one row tile: its
                        // activations and the whole weight matrix once).
                        const uint32_t in_e = lin - (uint32_t)before * tiles_n, per_group = gemm::GROUP_M * tiles_n;
                        const uint32_t grp = in_e / per_group, in_grp = in_e - grp * per_group;
                        const uint32_t left = (uint32_t)cnt - grp * gemm::GROUP_M;
                        const uint32_t gm = left < gemm::GROUP_M ? left : gemm::GROUP_M;
                        const uint32_t gn = gemm::CHUNK / gm;
                        const uint32_t per_nblock = gm * gn;
                        const uint32_t nblk = in_grp / per_nblock, in_blk = in_grp - nblk * per_nblock;
                        const uint32_t local = grp * gemm::GROUP_M + in_blk % gm, tn = nblk * gn + in_blk / gm;
                        entry.x = e | (big ? 1 << 30 : 0);
                        entry.y = (int)(row_begin + (big ? (int64_t)local * 256 : (int64_t)(rows >> 8) * 256));     // M_total < 2^31
                        entry.z = (int)(row_begin + rows);
                        entry.w = (int)(tn * 256);
                    }
                }
            }
            table[t] = entry;
        }
        __syncthreads();
        for (int i = 0; i < kTable; ++i) {
            if (first + (uint64_t)i * gridDim.x >= all_slots) break;
            const int4 entry = table[i];
            const int ex = __builtin_amdgcn_readfirstlane(entry.x);
            if (ex < 0) continue;
            const int e = ex & 0xFFFF;
            const int64_t m0 = __builtin_amdgcn_readfirstlane(entry.y), row_end = __builtin_amdgcn_readfirstlane(entry.z);
            const int64_t n0 = __builtin_amdgcn_readfirstlane(entry.w);
            const float *bs_e = (const float *)((const char *)Bs + (int64_t)e * (N / 128) * kblocks * (HWS ? 1 : 4));
            const uint8_t *bq_e = Bq + (int64_t)e * N * K;
            __syncthreads();                            // every wave is done with the previous tile's use of the stage memory
            if (ex >> 30)
                tile_asm<256, 256, 1, HWS, false, 2, false, true, 2, NN>(smem, Aq, As, bq_e, bs_e, m0, row_end, n0, N, K, C, N, out_dtype);
            else
                tile_asm<128, 256, 1, HWS, false, 3, false, true, 4, NN>(smem, Aq, As, bq_e, bs_e, m0, row_end, n0, N, K, C, N, out_dtype);
        }
    }
}

template <int SDT, int NB>
int launch_nb(const void *Aq, const void *As, const void *Bq, const void *Bs, int64_t M, int64_t N, int64_t K, void *C,
              int64_t ldc, int out_dtype, hipStream_t st)
{
    const int64_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + 32 * NB - 1) / (32 * NB);
    const int64_t grid = gemm::padded_grid(tiles_m, tiles_n);
    if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_block: problem too large");
    hipLaunchKernelGGL((gemm_big<SDT, NB>), dim3((unsigned)grid), dim3(THREADS), 0, st, (const uint8_t *)Aq, As,
                       (const uint8_t *)Bq, Bs, M, N, K, tiles_m, tiles_n, C, ldc, out_dtype);
    return check_launch("lp_gemm_fp8_block(big)");
}

}  // namespace

namespace lowp {
namespace gemm {

// The hand-scheduled loop addresses operands with 32-bit offsets and moves scales in 16-byte groups
// of four K steps.
static bool asm_shape_ok(const void *As, const void *Bs, int64_t M, int64_t N, int64_t K, int scale_dtype = LP_F32)
{
    const uintptr_t align = scale_dtype == LP_E8M0 ? 3 : 15;          // one group of four scales per access
    return K % 512 == 0 && (((uintptr_t)As | (uintptr_t)Bs) & align) == 0 && M * K < 0xFFFFFFFFll && N * K < 0xFFFFFFFFll &&
           M * (K / 128) * 4 < 0xFFFFFFFFll;
}

// Picks the tile width whose last round of tiles wastes the fewest CU slots.
int choose_big_tn(int64_t M, int64_t N)
{
    const int64_t tiles_m = (M + BM - 1) / BM;
    int best = 256;
    double best_cost = 1e30;
    for (int tn : {256, 192, 128}) {
        const int64_t tiles = tiles_m * ((N + tn - 1) / tn);
        const int64_t rounds = (tiles + 255) / 256;
        // time ~ rounds * (work per tile); narrower tiles pay more operand traffic per flop
        const double cost = (double)rounds * tn * (tn == 256 ? 1.0 : tn == 192 ? 1.04 : 1.10);
        if (cost < best_cost) { best_cost = cost; best = tn; }
    }
    return best;
}

// Whole 256 x 256 tiles only: the four-wave loop copies and stores without masks.  LP_GEMM_QUAD = 0 / 1 (tuning aid).
static bool quad_ok(int64_t M, int64_t N)
{
    static const int knob = getenv("LP_GEMM_QUAD") ? atoi(getenv("LP_GEMM_QUAD")) : QUAD_DEFAULT;
    return knob != 0 && M % 256 == 0 && N % 256 == 0;
}

int launch_big(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N,
               int64_t K, void *C, int64_t ldc, int out_dtype, int tn, hipStream_t st)
{
#define GO(SDT)                                                                                         \
    do {                                                                                                \
        if (tn == 256) return launch_nb<SDT, 8>(Aq, As, Bq, Bs, M, N, K, C, ldc, out_dtype, st);             \
        if (tn == 192) return launch_nb<SDT, 6>(Aq, As, Bq, Bs, M, N, K, C, ldc, out_dtype, st);             \
        return launch_nb<SDT, 4>(Aq, As, Bq, Bs, M, N, K, C, ldc, out_dtype, st);                            \
    } while (0)
    static const bool no_asm = getenv("LP_GEMM_NO_ASM") != nullptr;       // tuning / test aid
    if (!no_asm && scale_dtype == LP_E8M0 && tn == 256 && asm_shape_ok(As, Bs, M, N, K, LP_E8M0)) {
        // e8m0 scales: the matrix cores apply them (no fold, accumulation in place)
        const int64_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + 255) / 256;
        const int64_t grid = gemm::padded_grid(tiles_m, tiles_n);
        if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_block: problem too large");
        if (quad_ok(M, N)) {
            hipLaunchKernelGGL(gemm_asm_quad, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq, (const uint8_t *)As,
                               (const uint8_t *)Bq, (const uint8_t *)Bs, M, N, K, tiles_m, tiles_n, C, ldc, out_dtype);
            return check_launch("lp_gemm_fp8_block(asm e8m0, four waves)");
        }
        hipLaunchKernelGGL((gemm_asm<256, 256, 1, true>), dim3((unsigned)grid), dim3(THREADS), 0, st, (const uint8_t *)Aq,
                           (const float *)As, (const uint8_t *)Bq, (const float *)Bs, M, N, K, tiles_m, tiles_n, C, ldc,
                           out_dtype);
        return check_launch("lp_gemm_fp8_block(asm e8m0)");
    }
    if (!no_asm && scale_dtype == LP_F32 && (tn == 256 || tn == 192) && asm_shape_ok(As, Bs, M, N, K)) {
        const int64_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + tn - 1) / tn;
        const int64_t grid = gemm::padded_grid(tiles_m, tiles_n);
        if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_block: problem too large");
        if (tn == 256)
            hipLaunchKernelGGL((gemm_asm<256, 256, 1>), dim3((unsigned)grid), dim3(THREADS), 0, st, (const uint8_t *)Aq,
                               (const float *)As, (const uint8_t *)Bq, (const float *)Bs, M, N, K, tiles_m, tiles_n, C, ldc,
                               out_dtype);
        else
            hipLaunchKernelGGL((gemm_asm<256, 192, 1>), dim3((unsigned)grid), dim3(THREADS), 0, st, (const uint8_t *)Aq,
                               (const float *)As, (const uint8_t *)Bq, (const float *)Bs, M, N, K, tiles_m, tiles_n, C, ldc,
                               out_dtype);
        return check_launch("lp_gemm_fp8_block(asm)");
    }
    if (scale_dtype == LP_F32) GO(LP_F32);
    GO(LP_E8M0);
#undef GO
}

// Unscaled fp8 NT GEMM on the hardware-scaled 256 x 256 loop with every scale byte 0x7F (2^0): `ones` holds at least
// max(M, N / 128) * K / 128 such bytes.  out_dtype may be LP_E4M3 here (see tile_asm's last store loop).  bf16: the operands
// are bf16 and K is the number of bytes of an operand row (two per value).
int launch_nt_unit_scales(const void *A, const void *B, const void *ones, int64_t M, int64_t N, int64_t K, void *C, int out_dtype,
                          hipStream_t st, bool bf16)
{
    const int64_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + 255) / 256;
    const int64_t grid = gemm::padded_grid(tiles_m, tiles_n);
    if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_nt: problem too large");
    if (bf16) {
        // K = bytes per operand row here
        hipLaunchKernelGGL(gemm_asm_bf16, dim3((unsigned)grid), dim3(THREADS), 0, st, (const uint8_t *)A, (const float *)ones,
                           (const uint8_t *)B, M, N, K, tiles_m, tiles_n, C, N, out_dtype);
        return check_launch("lp_gemm_nt(asm, bf16)");
    }
    if (quad_ok(M, N)) {
        hipLaunchKernelGGL(gemm_asm_quad, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)A, (const uint8_t *)ones,
                           (const uint8_t *)B, (const uint8_t *)ones, M, N, K, tiles_m, tiles_n, C, N, out_dtype);
        return check_launch("lp_gemm_nt(asm, unit scales, four waves)");
    }
    hipLaunchKernelGGL((gemm_asm<256, 256, 1, true>), dim3((unsigned)grid), dim3(THREADS), 0, st, (const uint8_t *)A, (const float *)ones,
                       (const uint8_t *)B, (const float *)ones, M, N, K, tiles_m, tiles_n, C, N, out_dtype);
    return check_launch("lp_gemm_nt(asm, unit scales)");
}

bool nt_unit_scales_ok(const void *ones, int64_t M, int64_t N, int64_t K)
{
    static const bool no_asm = getenv("LP_GEMM_NO_ASM") != nullptr;
    return !no_asm && asm_shape_ok(ones, ones, M, N, K, LP_E8M0);
}

// 256 x 288 or 256 x 224 tiles when they divide N and fill the last round of tiles better than 256 x 256 tiles would
// (of the two, the one that fills it better; 288 when they tie); false when the shape does not fit (the caller goes on
// with the other kernels).  LP_GEMM_WIDE = 0 switches the route off, 288 or 224 forces that width where it divides N.
bool launch_wide(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K,
                 void *C, int64_t ldc, int out_dtype, hipStream_t st, int *rc)
{
    static const int knob = getenv("LP_GEMM_WIDE") ? atoi(getenv("LP_GEMM_WIDE")) : -1;             // tuning aid
    static const bool off = getenv("LP_GEMM_NO_ASM") != nullptr || knob == 0;
    if (off || (scale_dtype != LP_F32 && scale_dtype != LP_E8M0) || !asm_shape_ok(As, Bs, M, N, K, scale_dtype)) return false;
    const int64_t tiles_m = (M + 255) / 256, big = tiles_m * ((N + 255) / 256);
    // fraction of CU slots used over whole rounds of 256 tiles
    auto fill = [](int64_t tiles) { return (double)tiles / (double)((tiles + 255) / 256 * 256); };
    int width = 0;
    for (int w : {288, 224}) {
        if (N % w) continue;
        if (knob == w) { width = w; break; }
        if (knob > 0) continue;
        const double f = fill(tiles_m * (N / w));
        if (f >= 0.9 && f > fill(big) + 0.05 && (!width || f > fill(tiles_m * (N / width)))) width = w;
    }
    if (!width) return false;
    const int64_t tiles_n = N / width, grid = gemm::padded_grid(tiles_m, tiles_n);
    if (grid > 0x7FFFFFFF) return false;
    auto go = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(512), 0, st, (const uint8_t *)Aq, (const float *)As, (const uint8_t *)Bq,
                           (const float *)Bs, M, N, K, tiles_m, tiles_n, C, ldc, out_dtype);
    };
    if (width == 288) scale_dtype == LP_E8M0 ? go(gemm_asm_wide<true, 288>) : go(gemm_asm_wide<false, 288>);
    else scale_dtype == LP_E8M0 ? go(gemm_asm_wide<true, 224>) : go(gemm_asm_wide<false, 224>);
    *rc = check_launch(width == 288 ? "lp_gemm_fp8_block(asm 256x288)" : "lp_gemm_fp8_block(asm 256x224)");
    return true;
}

// Columns [0, n_big) on 256 x 256 tiles and [n_big, N) on K-split 128 x 128 tiles in one launch; false when the shape does
// not fit both loops (the caller then launches the two kernels one after the other).
bool launch_mixed(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K,
                  int64_t n_big, void *C, int64_t ldc, int out_dtype, hipStream_t st, int *rc)
{
    static const bool off = getenv("LP_GEMM_NO_ASM") != nullptr || getenv("LP_GEMM_NO_MID") != nullptr ||
                            (getenv("LP_GEMM_MIXED") && atoi(getenv("LP_GEMM_MIXED")) == 0);
    const int64_t n_small = N - n_big;
    if (off || (scale_dtype != LP_F32 && scale_dtype != LP_E8M0) || n_big <= 0 || n_small <= 0 || n_big % 256 || n_small % 128 ||
        K % 1024 || !asm_shape_ok(As, Bs, M, N, K, scale_dtype))
        return false;
    const int64_t small_tiles = ((M + 127) / 128) * (n_small / 128);
    if (small_tiles > 256) return false;                               // the K split pays up to one tile per CU
    const int64_t grid_big = gemm::padded_grid((M + 255) / 256, n_big / 256);
    const int64_t grid = grid_big + gemm::padded_grid((M + 127) / 128, n_small / 128);
    if (grid > 0x7FFFFFFF) return false;
    if (scale_dtype == LP_E8M0)
        hipLaunchKernelGGL((gemm_asm_mixed<true>), dim3((unsigned)grid), dim3(512), 0, st, (const uint8_t *)Aq, (const float *)As,
                           (const uint8_t *)Bq, (const float *)Bs, M, N, K, n_big, grid_big, C, ldc, out_dtype);
    else
        hipLaunchKernelGGL((gemm_asm_mixed<false>), dim3((unsigned)grid), dim3(512), 0, st, (const uint8_t *)Aq, (const float *)As,
                           (const uint8_t *)Bq, (const float *)Bs, M, N, K, n_big, grid_big, C, ldc, out_dtype);
    *rc = check_launch("lp_gemm_fp8_block(asm mixed)");
    return true;
}

// 128 x 128 tiles on the hand-scheduled loop: two workgroups share a CU, so one computes while the other waits.
bool mid_asm_ok(const void *As, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K)
{
    static const bool no_asm = getenv("LP_GEMM_NO_ASM") != nullptr || getenv("LP_GEMM_NO_MID") != nullptr;
    return !no_asm && (scale_dtype == LP_F32 || scale_dtype == LP_E8M0) && asm_shape_ok(As, Bs, M, N, K, scale_dtype);
}

int launch_mid_asm(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype, int64_t M, int64_t N,
                   int64_t K, void *C, int64_t ldc, int out_dtype, hipStream_t st)
{
    const int64_t tiles_m = (M + 127) / 128, tiles_n = (N + 127) / 128;
    const int64_t grid = gemm::padded_grid(tiles_m, tiles_n);
    if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_block: problem too large");
    // At most one tile per CU: split K inside the workgroup (needs whole scale groups of 512 in each half).  With
    // more tiles than CUs the 512-thread workgroups would need a second round where 256-thread ones share the CUs
    // (288 tiles at K = 7168: 90 us with the split against 60 without).
    static const char *dual_env = getenv("LP_GEMM_MID_DUAL");        // tuning aid: 0 / 1 forces it off / on
    // (fp32 scales only: the hardware-scaled loop has no folds to share out and is 3 - 12 % faster without the split --
    // 512 x 7168 x 2048 11.2 against 12.8 us, 384 x 4096 x 7168 28.2 against 29.1 -- where the fp32-scaled one gains 15 %)
    const bool dual = K % 1024 == 0 && (dual_env ? atoi(dual_env) != 0 : tiles_m * tiles_n <= 256 && scale_dtype == LP_F32);
    static const char *deep_env = getenv("LP_GEMM_MID_STAGES");      // tuning aid: 4 forces the four-stage loop, 2 forbids it
    const bool four = deep_env ? atoi(deep_env) == 4 : false;
    if (four) {
        if (scale_dtype == LP_E8M0)
            hipLaunchKernelGGL((gemm_asm<128, 128, 1, true, 4>), dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq,
                               (const float *)As, (const uint8_t *)Bq, (const float *)Bs, M, N, K, tiles_m, tiles_n, C, ldc,
                               out_dtype);
        else
            hipLaunchKernelGGL((gemm_asm<128, 128, 1, false, 4>), dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq,
                               (const float *)As, (const uint8_t *)Bq, (const float *)Bs, M, N, K, tiles_m, tiles_n, C, ldc,
                               out_dtype);
        return check_launch("lp_gemm_fp8_block(asm128 four stages)");
    }
    if (dual) {
        if (scale_dtype == LP_E8M0)
            hipLaunchKernelGGL((gemm_asm_dual<1, true>), dim3((unsigned)grid), dim3(512), 0, st, (const uint8_t *)Aq,
                               (const float *)As, (const uint8_t *)Bq, (const float *)Bs, M, N, K, tiles_m, tiles_n, C, ldc,
                               out_dtype);
        else
            hipLaunchKernelGGL((gemm_asm_dual<1, false>), dim3((unsigned)grid), dim3(512), 0, st, (const uint8_t *)Aq,
                               (const float *)As, (const uint8_t *)Bq, (const float *)Bs, M, N, K, tiles_m, tiles_n, C, ldc,
                               out_dtype);
        return check_launch("lp_gemm_fp8_block(asm128 dual)");
    }
    if (scale_dtype == LP_E8M0) {
        hipLaunchKernelGGL((gemm_asm<128, 128, 1, true>), dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq,
                           (const float *)As, (const uint8_t *)Bq, (const float *)Bs, M, N, K, tiles_m, tiles_n, C, ldc,
                           out_dtype);
        return check_launch("lp_gemm_fp8_block(asm128 e8m0)");
    }
    // With two K blocks per stage a workgroup keeps twice the bytes in flight but owns the CU's LDS alone:
    // better while there is at most about one tile per CU, worse when two workgroups could share a CU.
    static const char *force = getenv("LP_GEMM_MID_KSUB");           // tuning aid
    const bool deep = force ? atoi(force) == 2 : tiles_m * tiles_n <= 256;
    if (deep)
        hipLaunchKernelGGL((gemm_asm<128, 128, 2>), dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq,
                           (const float *)As, (const uint8_t *)Bq, (const float *)Bs, M, N, K, tiles_m, tiles_n, C, ldc,
                           out_dtype);
    else
        hipLaunchKernelGGL((gemm_asm<128, 128, 1>), dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq,
                           (const float *)As, (const uint8_t *)Bq, (const float *)Bs, M, N, K, tiles_m, tiles_n, C, ldc,
                           out_dtype);
    return check_launch("lp_gemm_fp8_block(asm128)");
}

// Row-scaled weights on the hardware-scaled loop: e8m0 scales, K in whole groups of four blocks, 32-bit operand offsets.
bool rowscale_asm_ok(const void *As, const void *Bs, int scale_dtype, int64_t M, int64_t N, int64_t K)
{
    static const bool no_asm = getenv("LP_GEMM_NO_ASM") != nullptr;
    return !no_asm && scale_dtype == LP_E8M0 && K % 512 == 0 && (uintptr_t)As % 4 == 0 && (uintptr_t)Bs % 4 == 0 &&
           M * K < 0xFFFFFFFFLL && N * K < 0xFFFFFFFFLL;
}

int launch_rowscale_asm(const void *Aq, const void *As, const void *Bq, const void *Bs, int64_t M, int64_t N, int64_t K, void *C,
                        int out_dtype, hipStream_t st)
{
    const int64_t tiles_m = (M + 127) / 128, tiles_n = N / 128;
    const int64_t grid = gemm::padded_grid(tiles_m, tiles_n);
    if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_rowscale: problem too large");
    hipLaunchKernelGGL(gemm_asm_rowscale, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq, (const float *)As,
                       (const uint8_t *)Bq, (const float *)Bs, M, N, K, tiles_m, tiles_n, C, N, out_dtype);
    return check_launch("lp_gemm_fp8_rowscale(asm)");
}

int launch_rowscale_grouped_asm(const void *Aq, const void *As, const void *Bq, const void *Bs, const int32_t *groups, int G, int max_k_blocks, int64_t M,
                                int64_t N, void *C, int out_dtype, hipStream_t st)
{
    const int64_t tiles_m = (M + 127) / 128, tiles_n = N / 128;
    const int64_t per_group = gemm::padded_grid(tiles_m, tiles_n), grid = per_group * G;
    if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_rowscale_grouped: problem too large");
    hipLaunchKernelGGL(gemm_asm_rowscale_grouped, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq, (const float *)As,
                       (const uint8_t *)Bq, (const float *)Bs, groups, M, N, tiles_m, tiles_n, per_group, C, out_dtype, max_k_blocks);
    return check_launch("lp_gemm_fp8_rowscale_grouped(asm)");
}

// Grouped problems on the hand-scheduled kernel: fp32 scales, N a multiple of 256, offsets that fit 32 bits.
bool big_grouped_ok(const void *As, const void *Bs, int scale_dtype, int64_t M_total, int64_t N, int64_t K)
{
    static const bool no_asm = getenv("LP_GEMM_NO_ASM") != nullptr;
    return !no_asm && (scale_dtype == LP_F32 || scale_dtype == LP_E8M0) && N % 256 == 0 &&
           asm_shape_ok(As, Bs, M_total, N, K, scale_dtype);
}

// CUs of the current device (0 if it cannot be asked); asked once per device
static int compute_units()
{
    static int cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
        cached[dev] = n > 0 ? n : -1;
    }
    return cached[dev] > 0 ? cached[dev] : 0;
}

// The data gradient of the grouped linear on the stored weights (no transposed copy): e8m0 scales, N a multiple of 256,
// K of 512, the scale table's rows a multiple of 4 bytes apart and 4-byte aligned, at most kMixedMaxExperts experts.
bool grouped_nn_ok(const void *As, const void *Bs, int scale_dtype, int E, int64_t M_total, int64_t N, int64_t K)
{
    return scale_dtype == LP_E8M0 && E <= kMixedMaxExperts && N % 256 == 0 && (N / 128) % 4 == 0 && ((uintptr_t)Bs & 3) == 0 &&
           asm_shape_ok(As, Bs, M_total, N, K, LP_E8M0);
}

int launch_grouped_nn(const void *Aq, const void *As, const void *Bq, const void *Bs, const int32_t *m_offsets, int E,
                      int64_t M_total, int64_t N, int64_t K, void *C, int out_dtype, hipStream_t st)
{
    int64_t grid = padded_grid(M_total / 256 + E, N / 256) + 2 * 8 * CHUNK;
    if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_grouped_nn: problem too large");
    const int cus = compute_units();
    if (cus >= 8 && grid > cus) grid = cus / 8 * 8;            // one workgroup per CU walks the tile slots, as in the forward launch
    hipLaunchKernelGGL((gemm_asm_grouped_mixed<true, true>), dim3((unsigned)grid), dim3(512), 0, st, (const uint8_t *)Aq,
                       (const float *)As, (const uint8_t *)Bq, (const float *)Bs, m_offsets, E, M_total, N, K, C, out_dtype, 4);
    return check_launch("lp_gemm_fp8_grouped_nn");
}

int launch_big_grouped(const void *Aq, const void *As, const void *Bq, const void *Bs, int scale_dtype,
                       const int32_t *m_offsets, int E, int64_t M_total, int64_t N, int64_t K, void *C, int out_dtype,
                       hipStream_t st)
{
    static const char *force = getenv("LP_GEMM_GROUPED_MODE");          // tuning aid: 0 = 128 tiles, 1 = 256 + 128 in two launches, 2 = one mixed launch
    const int mode = force ? atoi(force) : -1;
    // One launch with both tile heights when the experts are not all tiny and few (see many_flat_tiles below), whatever
    // the K: its workgroups own a CU alone, so what a tile spends before and after its K loop is not hidden behind a
    // second workgroup, and still it is ahead of the 128 x 128 kernel down to K = 512 (config 4's rows per expert, N =
    // 4096, fp32 scales: K = 512 0.29 against 0.36 ms, 1024 0.48 / 0.54, 1536 0.63 / 0.71, 2048 (down) 1.29 / 1.40).
    // An expert has at most one small tile, and M_e / 256 big ones plus one when more than 128 rows are left over.
    // The launch needs work for every CU: at least one 256-row tile's worth per CU, counting an expert as half a tile on
    // top of its rows (the host sees the row total, not the split).  Below that the 128 x 128 kernel, whose workgroups
    // start at once and share CUs in pairs, is up to twice as fast (8 experts of 256 rows, N = 2048, K = 512: 8.3 against
    // 17.8 us; 16 experts, N = 4096, K = 1536: 37.4 against 32.9 the other way).  Decode-sized batches pass the same test
    // with their flat tiles alone: 256 experts of 1 .. 127 rows, gate_up shape, 1.10 - 1.30 ms against 1.26 - 1.49 on the
    // 128 x 128 kernel (three LDS stages of streamed weights against two); 8 such experts stay there, 45 against 72 us.
    const bool enough_tiles = (M_total / 256 + E / 2) * (N / 256) >= 256;
    if (mode == 2 || (mode < 0 && E <= kMixedMaxExperts && enough_tiles)) {
        // an expert with r rows has r / 256 tiles plus one when rows are left over, big or small: M_total / 256 + E row
        // tiles at most over both classes, each class rounded up to whole groups of 8 x 32 workgroups
        int64_t grid = padded_grid(M_total / 256 + E, N / 256) + 2 * 8 * CHUNK;
        if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_grouped: problem too large");
        if (E <= kMixedMaxExperts) {
            // one workgroup per CU that works through every grid-th slot (a workgroup owns its CU: the tiles' LDS)
            // (LP_GEMM_GROUPED_PERSIST, read at every call so that a test can change it: 0 = one workgroup per slot, n >= 8 =
            // that many workgroups, e.g. few enough that each walks more slots than one table holds)
            const char *persist_env = getenv("LP_GEMM_GROUPED_PERSIST");
            const int forced = persist_env ? atoi(persist_env) : -1;
            const int cus = forced == 0 ? 0 : (forced >= 8 ? forced : compute_units());
            if (cus >= 8 && grid > cus) grid = cus / 8 * 8;
            static const char *order_env = getenv("LP_GEMM_GROUPED_ORDER");     // tuning aid: XCDs that take their small tiles first (0: classes dealt alternately)
            const int small_first = order_env ? atoi(order_env) : 4;
            if (scale_dtype == LP_E8M0)
                hipLaunchKernelGGL((gemm_asm_grouped_mixed<true>), dim3((unsigned)grid), dim3(512), 0, st, (const uint8_t *)Aq,
                                   (const float *)As, (const uint8_t *)Bq, (const float *)Bs, m_offsets, E, M_total, N, K, C, out_dtype, small_first);
            else
                hipLaunchKernelGGL((gemm_asm_grouped_mixed<false>), dim3((unsigned)grid), dim3(512), 0, st, (const uint8_t *)Aq,
                                   (const float *)As, (const uint8_t *)Bq, (const float *)Bs, m_offsets, E, M_total, N, K, C, out_dtype, small_first);
            return check_launch("lp_gemm_fp8_grouped(asm mixed heights)");
        }
    }
    if (scale_dtype == LP_E8M0) {
        // e8m0 scales: 128 x 128 tiles on the kernel whose matrix instructions apply the scales
        const int64_t mtiles = M_total / 128 + E;
        const int64_t grid = padded_grid(mtiles, N / 128);
        if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_grouped: problem too large");
        hipLaunchKernelGGL((gemm_asm_grouped<128, 128, 1, 0, true>), dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq,
                           (const float *)As, (const uint8_t *)Bq, (const float *)Bs, m_offsets, E, M_total, N, K, mtiles, N / 128, C,
                           out_dtype);
        return check_launch("lp_gemm_fp8_grouped(asm 128 e8m0)");
    }
    // Few rows per expert on average: the weights of most experts are read for one or two row tiles, so the launch
    // is as much a weight stream as a GEMM.  128 x 128 tiles (two workgroups per CU, tiles taken from both ends
    // of the expert list) let streaming tiles and compute-bound tiles overlap and bound the padding per expert
    // by 127 rows.  With many rows per expert the 256 x 256 kernel takes the full 256-row tiles and the
    // 128 x 128 kernel what is left.
    const bool split = mode >= 0 ? mode == 1 : M_total >= (int64_t)E * 1024;
    if (split) {
        const int64_t big_mtiles = M_total / 256;
        const int64_t grid = padded_grid(big_mtiles, N / 256);
        if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_grouped: problem too large");
        hipLaunchKernelGGL((gemm_asm_grouped<256, 256, 1, 1>), dim3((unsigned)grid), dim3(512), 0, st, (const uint8_t *)Aq,
                           (const float *)As, (const uint8_t *)Bq, (const float *)Bs, m_offsets, E, M_total, N, K, big_mtiles, N / 256,
                           C, out_dtype);
        const int rc = check_launch("lp_gemm_fp8_grouped(asm 256)");
        if (rc) return rc;
        int64_t rest_mtiles = 2 * (int64_t)E;
        if (rest_mtiles > M_total / 128 + E) rest_mtiles = M_total / 128 + E;
        const int64_t grid2 = padded_grid(rest_mtiles, N / 128);
        if (grid2 > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_grouped: problem too large");
        hipLaunchKernelGGL((gemm_asm_grouped<128, 128, 1, 2>), dim3((unsigned)grid2), dim3(256), 0, st, (const uint8_t *)Aq,
                           (const float *)As, (const uint8_t *)Bq, (const float *)Bs, m_offsets, E, M_total, N, K, rest_mtiles, N / 128,
                           C, out_dtype);
        return check_launch("lp_gemm_fp8_grouped(asm 128)");
    }
    const int64_t mtiles = M_total / 128 + E;
    const int64_t grid = padded_grid(mtiles, N / 128);
    if (grid > 0x7FFFFFFF) return fail(LP_ERR_UNSUPPORTED, "lp_gemm_fp8_grouped: problem too large");
    hipLaunchKernelGGL((gemm_asm_grouped<128, 128, 1, 0>), dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t *)Aq,
                       (const float *)As, (const uint8_t *)Bq, (const float *)Bs, m_offsets, E, M_total, N, K, mtiles, N / 128, C,
                       out_dtype);
    return check_launch("lp_gemm_fp8_grouped(asm 128)");
}

}  // namespace gemm
}  // namespace lowp
