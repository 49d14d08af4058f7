// DeepSeek-V4 style expert conversion for gfx950: packed e2m1 codes with one
// e8m0 scale per 1 x 32 block -> e4m3fn codes with one scale per 128 x 128 tile.
//
//   fp4_rebase : lossless re-basing; outer scale = (largest e8m0 of the tile)/64,
//                element = table(code) * 2^(sb - S + 6), cast without clamp.
//   fp4_amax   : the bf16 value table(code) * 2^(sb-127) is formed in registers
//                (exact), then quantised like a 128 x 128 bf16 tile
//                (scale from amax); the bf16 tensor is written only on request.
//
// One workgroup (256 or 512 threads) owns a 128-row x 256-column "super tile" (two scale
// tiles side by side) so that every row segment it touches is a full 128-byte
// line of packed input and 256 bytes of output.  Lane l of a 32-lane half wave
// owns 4 packed bytes (8 elements); lanes 0-15 belong to the left tile, 16-31
// to the right one.  The packed tile lives in 16 (8) VGPRs per lane, so HBM is
// read exactly once.
#include "lowp_device.h"

using namespace lowp;

namespace {

// Threads per workgroup (NT, a template parameter of everything below): 32 lanes cover a row of the super tile, so
// a pass covers NT / 32 rows and a lane makes 128 / (NT / 32) passes.  Measured on config 5: the re-basing kernel
// is 3-5 % faster with 512 threads than with 256, the fused kernel is indifferent (its per-tile set-up weighs
// more when a lane has fewer passes; with 1024 threads both lose 10-20 %).
constexpr int kRebaseThreads = 512;
constexpr int kAmaxThreads = 256;

// Maxima over the two 128 x 128 tiles of the super tile: every lane gets its own tile's and the other tile's,
// from one barrier.  The 16 lanes of a DPP row all belong to one tile and the rows of a wave alternate between
// the tiles, so a wave reduces to one value per tile (DPP within rows, one cross-lane exchange between rows r and
// r + 2), the workgroup's waves meet in `lds`, and a second DPP reduction over one entry per lane finishes.
// The caller must put a barrier before it uses `lds` again.
template <int NT>
__device__ __forceinline__ void tile_max_both_u32(uint32_t m, uint32_t (*lds)[16], int t, uint32_t &own, uint32_t &other)
{
    m = row16_max_u32(m);
    const uint32_t o = (uint32_t)__shfl_xor((int)m, 32);
    m = o > m ? o : m;
    const int half = (t >> 4) & 1;
    if ((t & 47) == 0) lds[half][t >> 6] = m;          // lanes 0 and 16 of every wave
    __syncthreads();
    const int e = t & 15;
    const uint32_t a = e < NT / 64 ? lds[half][e] : 0u, b = e < NT / 64 ? lds[half ^ 1][e] : 0u;
    own = row16_max_u32(a);
    other = row16_max_u32(b);
}

// Max over the lane's own tile; leaves `lds` free for the next use.
template <int NT>
__device__ __forceinline__ uint32_t tile_max_u32(uint32_t m, uint32_t (*lds)[16], int t)
{
    uint32_t own, other;
    tile_max_both_u32<NT>(m, lds, t, own, other);
    __syncthreads();
    return own;
}

struct Geometry {
    int64_t row0;        // first row of this lane in pass 0
    int64_t colb;        // byte column of this lane's 4 packed bytes
    int64_t scol;        // scale column of this lane
    int64_t tile;        // index of this lane's tile in the [rows/128, cols/128] grid
    bool active;         // lane's tile exists (odd number of tiles per row)
};

__device__ __forceinline__ Geometry geometry(int64_t super, int64_t supers_c, int64_t cols, int t)
{
    Geometry g;
    // the launchers keep the number of super tiles below 2^31: a 32-bit division instead of the
    // ~150 scalar instructions of a 64-bit one
    const int64_t sr = (uint32_t)super / (uint32_t)supers_c, sc = super - sr * supers_c;
    const int lane32 = t & 31;
    const int64_t col = sc * 256 + lane32 * 8;      // logical column of the lane's first element
    g.row0 = sr * 128 + (t >> 5);
    g.colb = col >> 1;
    g.scol = col >> 5;
    g.active = col < cols;
    g.tile = sr * (cols >> 7) + (col >> 7);
    return g;
}

// XCD-aware workgroup order: hardware deals consecutive workgroup ids to the 8
// XCDs in turn; remapping gives each XCD a contiguous run of super tiles so
// that neighbours sharing scale cache lines sit behind the same L2.
__device__ __forceinline__ int64_t xcd_remap(int64_t b, int64_t per_xcd) { return (b & 7) * per_xcd + (b >> 3); }

template <int NT>
__global__ __launch_bounds__(NT) void fp4_rebase(const uint8_t *__restrict__ packed, const uint8_t *__restrict__ scale,
                                                  int64_t cols, int64_t supers_c, int64_t n_supers, int64_t per_xcd,
                                                  uint8_t *__restrict__ q, void *__restrict__ scale_out, int scale_dtype)
{
    constexpr int kRowsPerPass = NT / 32, kPasses = 128 / kRowsPerPass;
    __shared__ uint32_t lds[2][16];
    const int64_t super = xcd_remap(blockIdx.x, per_xcd);
    if (super >= n_supers) return;
    const int t = threadIdx.x;
    const Geometry g = geometry(super, supers_c, cols, t);
    const int64_t pcols = cols >> 1, scols = cols >> 5;

    uint32_t w[kPasses];
    uint32_t sb[kPasses];
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
        const int64_t r = g.row0 + p * kRowsPerPass;
        if (g.active) {
            w[p] = __builtin_nontemporal_load((const uint32_t *)(packed + r * pcols + g.colb));
            sb[p] = scale[r * scols + g.scol];
        } else {
            w[p] = 0; sb[p] = 0;
        }
    }
    uint32_t S = 0;
#pragma unroll
    for (int p = 0; p < kPasses; ++p) S = sb[p] > S ? sb[p] : S;
    S = tile_max_u32<NT>(S, lds, t);

    const bool nan_tile = S == 0xFFu;
    if (g.active && (t & 15) == 0 && (t >> 5) == 0) {
        // outer = 2^(S-127) / 64 rounded to e8m0: byte max(S-6, 0); 0xFF stays NaN
        uint32_t ob = nan_tile ? 0xFFu : (S > 6u ? S - 6u : 0u);
        if (scale_dtype == LP_E8M0) ((uint8_t *)scale_out)[g.tile] = (uint8_t)ob;
        else ((float *)scale_out)[g.tile] = e8m0_to_f32(ob);
    }
    if (!g.active) return;

#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
        const int64_t r = g.row0 + p * kRowsPerPass;
        u32x2 out;
        if (!nan_tile) {
            // offset = 2^(sb - S + 6); below 2^-30 every product rounds to (signed) zero anyway
            int d = (int)sb[p] - (int)S + 6;
            d = d < -30 ? -30 : d;
            const float off = u2f((uint32_t)(127 + d) << 23);
            float v[8];
            fp4_decode8(fp4_pos_zero(w[p]), v);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] *= off;
            out.x = cvt4(v[0], v[1], v[2], v[3]);
            out.y = cvt4(v[4], v[5], v[6], v[7]);
        } else {
            out.x = 0x7F7F7F7Fu; out.y = 0x7F7F7F7Fu;
        }
        __builtin_nontemporal_store(out, (u32x2 *)(q + r * cols + (g.colb << 1)));
    }
}

// ---------------------------------------------------------------- fused amax

template <int MODE, bool WRITE_BF16, int NT>
__global__ __launch_bounds__(NT) void fp4_amax(const uint8_t *__restrict__ packed, const uint8_t *__restrict__ scale,
                                                int64_t cols, int64_t supers_c, int64_t n_supers, int64_t per_xcd,
                                                float amax_floor, int zero_rule, uint8_t *__restrict__ q,
                                                void *__restrict__ scale_out, int scale_dtype, uint16_t *__restrict__ bf16_out)
{
    constexpr int kRowsPerPass = NT / 32, kPasses = 128 / kRowsPerPass;
    __shared__ uint32_t lds[2][16];
    const int64_t super = xcd_remap(blockIdx.x, per_xcd);
    if (super >= n_supers) return;
    const int t = threadIdx.x;
    const Geometry g = geometry(super, supers_c, cols, t);
    const int64_t pcols = cols >> 1, scols = cols >> 5;

    // Lanes of a half that lies past the last tile (odd tile count per row) read the left half's
    // columns instead, so the loads need no branches; their results are never stored.
    const int64_t ld_colb = g.active ? g.colb : g.colb - 64, ld_scol = g.active ? g.scol : g.scol - 4;
    uint32_t w[kPasses];
    uint32_t sb[kPasses];
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
        const int64_t r = g.row0 + p * kRowsPerPass;
        w[p] = fp4_pos_zero(__builtin_nontemporal_load((const uint32_t *)(packed + r * pcols + ld_colb)));
        sb[p] = scale[r * scols + ld_scol];
    }

    // amax of |table(code)| * 2^(sb-127).  The product is exact in fp32 (and
    // in bf16) for scale bytes 2..252; any other byte sends the whole super
    // tile down the literal slow path.
    uint32_t mbits = 0;
    uint32_t edge = 0;
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
        float v[8];
        fp4_decode8(w[p], v);
        float m = fmaxf(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))),
                        fmaxf(fmaxf(fabsf(v[4]), fabsf(v[5])), fmaxf(fabsf(v[6]), fabsf(v[7]))));
        uint32_t prod = f2u(m * u2f(sb[p] << 23));
        mbits = prod > mbits ? prod : mbits;
        edge |= (sb[p] < 2u || sb[p] > 252u) ? 1u : 0u;
    }
    // Every thread of the workgroup must take the same number of barriers, so both slow decisions
    // (edge scale bytes, tile scale outside the fast range) are made for the super tile as a whole -- by
    // every lane for both tiles, from one reduction: an edge byte travels as the key 0xFFFFFFFF (products
    // are finite positive floats, so that pattern is free), and the scale of the other tile is derived
    // redundantly instead of being voted on.
    uint32_t key, key_other;
    tile_max_both_u32<NT>(edge ? 0xFFFFFFFFu : mbits, lds, t, key, key_other);
    bool slow_tile = key == 0xFFFFFFFFu || key_other == 0xFFFFFFFFu;
    BlockScale bs;
    // Each element is +-{0, .5, 1, 2, 4} * 2^e (even codes and 0.5) or +-{1, 2, 4} * 1.5 * 2^e (codes
    // 1.5, 3, 6), so its quotient by the tile scale is a power-of-two multiple of one of two numbers,
    // c1 = RN(1/s) and c3 = RN(1.5/s) (resp. f and RN(1.5 f) in the multiply form): two correctly
    // rounded constants per tile replace one division per element, and power-of-two scaling keeps
    // them correctly rounded.
    float c1 = 1.0f, c3 = 1.5f;
    if (!slow_tile) {
        auto out_of_range = [&](const BlockScale &b) -> bool {
            if (MODE == LP_SCALE_POW2) return b.exp2 < -100 || b.exp2 > 100;
            if (MODE == LP_SCALE_DIV) return !b.fast;
            return !(b.div >= 0x1p-100f && b.div <= 0x1p100f);
        };
        bs = derive_scale<MODE>(u2f(key), amax_floor, zero_rule);
        slow_tile = out_of_range(bs) || out_of_range(derive_scale<MODE>(u2f(key_other), amax_floor, zero_rule));
        if (MODE == LP_SCALE_POW2) {
            c1 = ldexpf(1.0f, -bs.exp2);
            c3 = ldexpf(1.5f, -bs.exp2);
        } else if (MODE == LP_SCALE_DIV) {
            c1 = bs.recip;
            c3 = 1.5f / bs.div;
        } else {
            c1 = bs.div;
            c3 = 1.5f * bs.div;
        }
    }

    if (!slow_tile) {
        if (g.active && (t & 15) == 0 && (t >> 5) == 0) store_scale(scale_out, scale_dtype, g.tile, bs.stored);
        if (!g.active) return;
        // All 8 elements of a pass share one scale byte sb, so their codes are eight numbers per pass:
        //   magnitude 0 .5 1 1.5 2 3 4 6  ->  e4m3(0, t1/2, t1, t3, 2 t1, 2 t3, 4 t1, 4 t3),  t = c * 2^(sb-127).
        // Four conversions build that table in two registers and byte permutes look the nibbles up: no
        // decode, no multiply per element (a conversion costs about 3 plain VALU instructions, measured).
        // The factors are formed by adding to the exponent field.  c1 and c3 are normal here (exponent
        // field cf, c3's at most cf + 1), so t1/2 .. 4 t3 are normal floats for sb in [129 - cf, 378 - cf],
        // and clamping sb to that range changes no result: a non-zero block has 2^(sb-127) <= 2 amax,
        // i.e. sb <= 264 - cf, so above the range every element is zero (and zero maps to table entry 0);
        // below it every quotient is under 2^-120 in magnitude and becomes a signed zero with the clamped
        // factor as with the true one.
        const uint32_t c1b = f2u(c1), c3b = f2u(c3);
        const int cf = (int)(c1b >> 23);
        const int sb_lo = 129 - cf, sb_hi = 378 - cf;
        const uint32_t c1adj = c1b - (127u << 23), c3adj = c3b - (127u << 23);
#pragma unroll
        for (int p = 0; p < kPasses; ++p) {
            const int64_t r = g.row0 + p * kRowsPerPass;
            int sbe = (int)sb[p];
            sbe = sbe < sb_lo ? sb_lo : (sbe > sb_hi ? sb_hi : sbe);
            const uint32_t t1 = c1adj + ((uint32_t)sbe << 23), t3 = c3adj + ((uint32_t)sbe << 23);
            const uint32_t tab_lo = cvt4(0.0f, u2f(t1 - (1u << 23)), u2f(t1), u2f(t3));
            const uint32_t tab_hi = cvt4(u2f(t1 + (1u << 23)), u2f(t3 + (1u << 23)), u2f(t1 + (2u << 23)), u2f(t3 + (2u << 23)));
            uint32_t wp = w[p];
            asm volatile("" : "+v"(wp));                       // keep the packed word, not values derived before the barrier
            // even elements sit in the low nibbles of the four bytes, odd elements in the high nibbles
            uint32_t ce = __builtin_amdgcn_perm(tab_hi, tab_lo, wp & 0x07070707u);
            uint32_t co = __builtin_amdgcn_perm(tab_hi, tab_lo, (wp >> 4) & 0x07070707u);
            ce |= (wp & 0x08080808u) << 4;                     // signs (zero magnitudes carry none, see fp4_pos_zero)
            co |= wp & 0x80808080u;
            u32x2 out = {__builtin_amdgcn_perm(co, ce, 0x05010400u), __builtin_amdgcn_perm(co, ce, 0x07030602u)};
            __builtin_nontemporal_store(out, (u32x2 *)(q + r * cols + (g.colb << 1)));
            if (WRITE_BF16) {
                const float s = u2f(sb[p] << 23);            // sb in 2..252: a normal power of two
                float b[8];
                fp4_decode8(wp, b);
                u32x4 o = {pack_bf16(b[0] * s, b[1] * s), pack_bf16(b[2] * s, b[3] * s), pack_bf16(b[4] * s, b[5] * s),
                           pack_bf16(b[6] * s, b[7] * s)};
                __builtin_nontemporal_store(o, (u32x4 *)(bf16_out + r * cols + (g.colb << 1)));
            }
        }
        return;
    }

    __syncthreads();                                          // the reduction below writes `lds` again
    // Slow tile: scale bytes at the edge of the e8m0 range (bf16 rounding,
    // overflow to inf, NaN).  Literal arithmetic with software casts; inputs
    // are read again from memory so that the fast path keeps its registers.
    uint32_t m2 = 0;
    if (g.active) {
        for (int p = 0; p < kPasses; ++p) {
            const int64_t r = g.row0 + p * kRowsPerPass;
            const uint32_t wp = fp4_pos_zero(*(const uint32_t *)(packed + r * pcols + g.colb));
            const float s = e8m0_to_f32(scale[r * scols + g.scol]);
            for (int j = 0; j < 8; ++j) {
                float b = bf16_bits_to_f32(sw_f32_to_bf16(sw_e2m1_to_f32((wp >> (4 * j)) & 0xFu, false) * s));
                uint32_t a = f2u(b) & 0x7FFFFFFFu;
                m2 = a > m2 ? a : m2;
            }
        }
    }
    m2 = tile_max_u32<NT>(m2, lds, t);
    const bool has_nan = m2 > 0x7F800000u;
    const float amax = u2f(has_nan ? 0x7FC00000u : m2);
    bs = derive_scale<MODE>(amax, amax_floor, zero_rule);
    if (has_nan && MODE == LP_SCALE_DIV) { bs.div = amax; bs.stored = amax; }
    if (g.active && (t & 15) == 0 && (t >> 5) == 0) store_scale(scale_out, scale_dtype, g.tile, bs.stored);
    if (!g.active) return;
    for (int p = 0; p < kPasses; ++p) {
        const int64_t r = g.row0 + p * kRowsPerPass;
        const uint32_t wp = fp4_pos_zero(*(const uint32_t *)(packed + r * pcols + g.colb));
        const float s = e8m0_to_f32(scale[r * scols + g.scol]);
        uint32_t o0 = 0, o1 = 0, h0 = 0, h1 = 0, h2 = 0, h3 = 0;
        for (int j = 0; j < 8; ++j) {
            uint32_t hb = sw_f32_to_bf16(sw_e2m1_to_f32((wp >> (4 * j)) & 0xFu, false) * s);
            uint32_t c = quant_slow<MODE>(bf16_bits_to_f32(hb), bs);
            uint32_t hs = hb << (16 * (j & 1)), cs = c << (8 * (j & 3));
            if (j < 4) o0 |= cs; else o1 |= cs;
            if (j < 2) h0 |= hs; else if (j < 4) h1 |= hs; else if (j < 6) h2 |= hs; else h3 |= hs;
        }
        if (bf16_out) {
            u32x4 ob = {h0, h1, h2, h3};
            *(u32x4 *)(bf16_out + r * cols + (g.colb << 1)) = ob;
        }
        u32x2 out = {o0, o1};
        *(u32x2 *)(q + r * cols + (g.colb << 1)) = out;
    }
}

int check_fp4_args(const char *name, const void *packed, const void *scale, int64_t rows, int64_t cols, const void *q_out,
                   const void *scale_out)
{
    LP_REQUIRE(rows >= 0 && cols >= 0, "%s: bad shape", name);
    LP_REQUIRE(rows % 128 == 0 && cols % 128 == 0, "%s: shape (%lld, %lld) must be a multiple of 128 x 128", name,
               (long long)rows, (long long)cols);
    if (rows == 0 || cols == 0) return 1;
    LP_REQUIRE(packed && scale && q_out && scale_out, "%s: null pointer", name);
    LP_REQUIRE((uintptr_t)packed % 4 == 0 && (uintptr_t)q_out % 8 == 0, "%s: buffers must be 8-byte aligned", name);
    return LP_OK;
}

}  // namespace

extern "C" int lp_fp4_to_fp8_rebase(const void *packed, const void *scale, int64_t rows, int64_t cols, void *q_out,
                                    void *scale_out, int scale_dtype, lp_stream_t stream)
{
    LP_REQUIRE(scale_dtype == LP_E8M0 || scale_dtype == LP_F32, "lp_fp4_to_fp8_rebase: scale_dtype must be LP_E8M0 or LP_F32");
    int rc = check_fp4_args("lp_fp4_to_fp8_rebase", packed, scale, rows, cols, q_out, scale_out);
    if (rc) return rc > 0 ? LP_OK : rc;
    const int64_t supers_c = (cols + 255) / 256, n_supers = (rows / 128) * supers_c;
    const int64_t per_xcd = (n_supers + 7) / 8;
    LP_REQUIRE(per_xcd * 8 <= 0x7FFFFFFF, "lp_fp4_to_fp8_rebase: too many tiles");
    hipLaunchKernelGGL(fp4_rebase<kRebaseThreads>, dim3((unsigned)(per_xcd * 8)), dim3(kRebaseThreads), 0, (hipStream_t)stream, (const uint8_t *)packed,
                       (const uint8_t *)scale, cols, supers_c, n_supers, per_xcd, (uint8_t *)q_out, scale_out, scale_dtype);
    return check_launch("lp_fp4_to_fp8_rebase");
}

extern "C" int lp_fp4_to_fp8_amax(const void *packed, const void *scale, int64_t rows, int64_t cols, int scale_mode,
                                  float amax_floor, int zero_rule, void *q_out, void *scale_out, int scale_dtype,
                                  void *bf16_out, lp_stream_t stream)
{
    LP_REQUIRE(is_scale_dtype(scale_dtype), "lp_fp4_to_fp8_amax: bad scale_dtype %d", scale_dtype);
    LP_REQUIRE(scale_mode >= LP_SCALE_POW2 && scale_mode <= LP_SCALE_MUL, "lp_fp4_to_fp8_amax: bad scale_mode");
    LP_REQUIRE(zero_rule >= LP_ZERO_NONE && zero_rule <= LP_ZERO_SCALE_TO_ONE, "lp_fp4_to_fp8_amax: bad zero_rule");
    LP_REQUIRE(amax_floor >= 0.0f, "lp_fp4_to_fp8_amax: amax_floor must be >= 0");
    int rc = check_fp4_args("lp_fp4_to_fp8_amax", packed, scale, rows, cols, q_out, scale_out);
    if (rc) return rc > 0 ? LP_OK : rc;
    LP_REQUIRE(!bf16_out || (uintptr_t)bf16_out % 16 == 0, "lp_fp4_to_fp8_amax: bf16_out must be 16-byte aligned");
    const int64_t supers_c = (cols + 255) / 256, n_supers = (rows / 128) * supers_c;
    const int64_t per_xcd = (n_supers + 7) / 8;
    LP_REQUIRE(per_xcd * 8 <= 0x7FFFFFFF, "lp_fp4_to_fp8_amax: too many tiles");
    dim3 grid((unsigned)(per_xcd * 8)), block(kAmaxThreads);
    hipStream_t st = (hipStream_t)stream;
#define LAUNCH(MODE)                                                                                                   \
    do {                                                                                                               \
        if (bf16_out)                                                                                                  \
            hipLaunchKernelGGL((fp4_amax<MODE, true, kAmaxThreads>), grid, block, 0, st, (const uint8_t *)packed, (const uint8_t *)scale, \
                               cols, supers_c, n_supers, per_xcd, amax_floor, zero_rule, (uint8_t *)q_out, scale_out,   \
                               scale_dtype, (uint16_t *)bf16_out);                                                      \
        else                                                                                                           \
            hipLaunchKernelGGL((fp4_amax<MODE, false, kAmaxThreads>), grid, block, 0, st, (const uint8_t *)packed, (const uint8_t *)scale, \
                               cols, supers_c, n_supers, per_xcd, amax_floor, zero_rule, (uint8_t *)q_out, scale_out,   \
                               scale_dtype, (uint16_t *)bf16_out);                                                      \
    } while (0)
    if (scale_mode == LP_SCALE_POW2) LAUNCH(LP_SCALE_POW2);
    else if (scale_mode == LP_SCALE_DIV) LAUNCH(LP_SCALE_DIV);
    else LAUNCH(LP_SCALE_MUL);
#undef LAUNCH
    return check_launch("lp_fp4_to_fp8_amax");
}
