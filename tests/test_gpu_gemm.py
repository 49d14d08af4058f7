"""GPU parity of the block-scaled FP8 GEMMs against fp32 dequant-then-matmul.

Bars: max relative error <= 2e-2 (relative to the largest |reference| entry) and cosine
>= 0.9999, plus the reference's own bars: avg_abs < 1e-2 * scale, calc_diff < 1e-5
(tests/test_gfused/test_my_gemm_fp8.py:239-243), cos > 0.999 and max_err < 1.0
(tests/test_gpatch_v4/test_deep_gemm_grouped_gemm_fp8.py:118-119).
"""
import pytest
import torch

from oracle import torch_ref as T
from tests import _inputs as I

pytestmark = pytest.mark.gpu

E4M3, E8M0 = torch.float8_e4m3fn, torch.float8_e8m0fnu


def say(*a):
    print("[case]", *a, flush=True)


@pytest.fixture(scope="module")
def G():
    import gcore_lowp
    return gcore_lowp


def calc_diff(x, y):
    x, y = x.double(), y.double()
    return float(1 - 2 * (x * y).sum() / (x * x + y * y).sum())


def check(out, ref, what):
    out, ref = out.float().cpu(), ref.float().cpu()
    assert torch.isfinite(out).all(), what
    denom = ref.abs().max().item()
    max_rel = ((out - ref).abs().max().item()) / max(denom, 1e-30)
    cos = torch.nn.functional.cosine_similarity(out.flatten().double(), ref.flatten().double(), dim=0).item()
    cd = calc_diff(out, ref)
    print(f"    {what}: max_rel={max_rel:.3e} cos={cos:.7f} calc_diff={cd:.3e}", flush=True)
    assert max_rel <= 2e-2, (what, max_rel)
    assert cos >= 0.9999, (what, cos)
    assert cd < 1e-5, (what, cd)


def quantized_problem(M, N, K, seed, pow2=False):
    x = I.act_like(M, K, seed)
    w = I.weight_like(N, K, seed + 1, outliers=False)
    if pow2:
        xq, xs = T.quant_fp8_e4m3_scale_e8m0(x, (1, 128))
        wq, ws = T.quant_fp8_e4m3_scale_e8m0(w, (128, 128))
    else:
        xq, xs = T.quant_block_fp32_scale(x, (1, 128))
        wq, ws = T.quant_block_fp32_scale(w, (128, 128))
    return xq, xs, wq, ws


def ref_gemm(xq, xs, wq, ws):
    # fp32 dequant then matmul, on the GPU for speed (fp32 accumulate, no TF32 on ROCm)
    a = T.dequant_act_f32(xq.cuda(), xs.float().cuda())
    b = T.dequant_weight_f32(wq.cuda(), ws.float().cuda())
    return (a.double() @ b.double().T).float() if a.numel() * b.shape[0] < 2 ** 27 else a @ b.T


DENSE_SHAPES = [
    (128, 128, 128), (128, 256, 256), (256, 128, 512), (64, 4096, 7168), (1, 128, 128), (7, 256, 384),
    (200, 384, 1024), (512, 1024, 2048), (2048, 4096, 7168), (128, 4096, 4096), (1024, 4096, 1024),
    (333, 640, 896),
    # prefill-sized: 256-row kernel (hand-scheduled loop), ragged M / N tails, and the column split
    # between the 256 x 256 and the 128 x 128 kernel (576 tiles on 256 CUs)
    (333, 8320, 512), (200, 16384, 256), (2048, 4224, 384), (256, 32768, 128), (1000, 9216, 640),
    (2048, 18432, 512), (4096, 4096, 1024), (1024, 16384, 1536), (32, 128, 7168), (48, 16384, 2048), (64, 2048, 7168),
    # N = 18432 = 64 x 288: the 256 x 288 tile kernel (512 tiles for 2048 rows, two full rounds), ragged M
    (2048, 18432, 1024), (1900, 18432, 2048),
    # the column split in one launch (256 x 256 tiles, then K-split 128 x 128 tiles): K a multiple of 1024, ragged M
    (3000, 12800, 1024), (2048, 9472, 1024), (1900, 9472, 2048),
    # at most 16 rows: one workgroup per 16 weight rows over the whole of K (ragged K-block runs, M < 16, one K block)
    (16, 4096, 7168), (1, 4096, 7168), (5, 3072, 2048), (16, 7168, 2560), (13, 18432, 128), (16, 3200, 6528),
    # 17 to 64 rows: the same cut with separate rings for weights and activations (2, 3, 4 row groups)
    (17, 4096, 7168), (32, 3072, 1024), (40, 3200, 6528), (48, 4096, 896), (50, 3072, 4096), (64, 18432, 2048),
    # 65 to 128 rows against at most 8192 weight rows: the many-rows decode kernel with four activation units per K block
    # (ragged last unit, one K block, a last workgroup past the end of N, 8192 / 8320 either side of its limit)
    (65, 4096, 7168), (128, 4096, 4096), (100, 3072, 1024), (96, 7168, 2048), (127, 6144, 128), (128, 8192, 896), (128, 8320, 512),
    (97, 3200, 640),
    # the same cuts with fewer workgroups than CUs (few weight rows): 16 rows per workgroup up to 64 activation rows and, from 65,
    # on the many-rows kernel (its narrowest cut); one group of 16 rows, a ragged last K-block run, one K block
    (64, 512, 7168), (33, 128, 1024), (8, 256, 4096), (1, 128, 128), (20, 1024, 6528), (128, 512, 7168), (65, 2048, 2048), (100, 128, 1024),
    (128, 1024, 128), (90, 384, 6528),
    # more than 128 rows in slices of 128 on that kernel (all workgroups in one round): a ragged last slice, a last slice of
    # one row, the largest row count, 16- and 32-row workgroups; and shapes just outside the rule (two rounds, K = 512)
    (129, 256, 1024), (256, 2048, 4096), (300, 1024, 7168), (512, 2048, 4096), (384, 2560, 2048), (1000, 128, 1024), (1024, 1024, 1152),
    (513, 2048, 1024), (256, 4096, 512), (8192, 128, 1024), (5000, 128, 2048), (2048, 512, 4096), (1300, 768, 3072), (2049, 256, 4096),
    # K beyond 7168 on the decode kernels: the workgroup walks K in rounds (two rounds of 29 blocks with a ragged last run, eight
    # rounds, every kernel of the family), and shapes the rule leaves to the tiled kernels
    (1, 4096, 14336), (16, 7168, 8192), (64, 5120, 7296), (40, 6144, 9216), (128, 7168, 8192), (8, 4096, 57344), (8, 256, 14336), (13, 18432, 8192),
    (64, 8192, 14336), (33, 7168, 18432), (48, 4096, 8192), (100, 3072, 9216),
    # ... beyond 8192 weight rows: up to 32 rows every cut, above only cuts of at most 48 rows that fill their rounds of workgroups
    (24, 12288, 8192), (40, 12288, 9216), (20, 18432, 8192), (48, 18432, 8192),
    # 9 .. 16 rows either side of the hand-over between the 16-row ring kernel and the many-rows kernel
    (12, 7168, 4096), (16, 8192, 2048), (9, 5120, 4096), (16, 8320, 4096), (12, 8192, 4224),
    # 33 .. 64 rows either side of the weight-row count from which the tiled kernels take them
    (48, 24576, 2048), (48, 24448, 2048), (32, 24576, 2048),
]


@pytest.mark.parametrize("shape", DENSE_SHAPES, ids=lambda s: "M%d_N%d_K%d" % s)
@pytest.mark.parametrize("pow2", [False, True], ids=["f32scale", "e8m0scale"])
def test_gemm_dense(G, shape, pow2):
    M, N, K = shape
    xq, xs, wq, ws = quantized_problem(M, N, K, seed=M + N + K, pow2=pow2)
    say("gemm dense", shape, "pow2" if pow2 else "f32")
    out = G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda())
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (M, N)
    check(out, ref_gemm(xq, xs, wq, ws), f"dense {shape}")


@pytest.mark.parametrize("shape", [(2048, 2048, 7168), (300, 2048, 1024), (129, 1280, 2560), (1000, 4096, 512), (513, 18432, 1024),
                                   (2048, 18432, 512), (777, 4224, 1536), (257, 19200, 512), (64, 24576, 1536), (16, 4096, 2048),
                                   (2048, 18432, 1024), (1900, 18432, 2048), (3000, 12800, 1024), (2048, 9472, 1024),
                                   (128, 4096, 4096), (70, 7168, 2048)],
                         ids=lambda s: "M%d_N%d_K%d" % s)
@pytest.mark.parametrize("pow2", [False, True], ids=["f32scale", "e8m0scale"])
def test_gemm_bf16_output_is_the_rounded_fp32_output(G, shape, pow2):
    """Every kernel rounds the same fp32 accumulators whichever way the result leaves (directly or as whole row runs
    through LDS): the bf16 output equals the fp32 output rounded to nearest-even, element for element, and rows or
    columns outside the problem are not written.  Shapes cover the K split inside a workgroup (<= 256 tiles), the
    256-row kernels with ragged M and N, the single-launch column split and the decode kernels."""
    M, N, K = shape
    xq, xs, wq, ws = quantized_problem(M, N, K, seed=M + N + K + 7, pow2=pow2)
    say("gemm bf16 vs fp32 output", shape, "pow2" if pow2 else "f32")
    args = (xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda())
    wide = G.gemm_fp8_block_scaling_impl(*args, out_dtype=torch.float32)
    narrow = G.gemm_fp8_block_scaling_impl(*args)
    assert narrow.dtype == torch.bfloat16 and wide.dtype == torch.float32
    assert torch.equal(narrow, wide.to(torch.bfloat16)), (narrow.float() - wide).abs().max().item()


def test_gemm_small_exact_vs_c_oracle(G, corc):
    """Small case against the double-precision scalar oracle, fp32 output: catches scale indexing
    (As[i, kb], Bs[j // 128, kb]) with distinct scales per block."""
    torch.manual_seed(0)
    M, N, K = 70, 256, 384
    aq = (torch.randn(M, K) * 40).to(E4M3)
    bq = (torch.randn(N, K) * 40).to(E4M3)
    a_s = torch.rand(M, K // 128) * 2 + 0.25
    b_s = torch.rand(N // 128, K // 128) * 2 + 0.25
    say("gemm small vs C oracle")
    out = G.gemm_fp8_block_scaling_impl(aq.cuda(), a_s.cuda(), bq.cuda(), b_s.cuda(), out_dtype=torch.float32)
    want = torch.from_numpy(corc.gemm_fp8_block(aq.view(torch.uint8).numpy(), a_s.numpy(),
                                                bq.view(torch.uint8).numpy(), b_s.numpy()))
    # fp32 accumulation over 384 products of magnitude up to 448^2 against a double-precision sum
    assert (out.cpu() - want).abs().max().item() <= want.abs().max().item() * 3e-5


def test_gemm_cpu_inputs_round_trip(G):
    xq, xs, wq, ws = quantized_problem(64, 128, 256, 3)
    say("gemm CPU inputs")
    out = G.gemm_fp8_block_scaling_impl(xq, xs, wq, ws)
    assert not out.is_cuda
    check(out, ref_gemm(xq, xs, wq, ws), "cpu-in")


def _grouped_problem(E, N, K, m_splits, seed):
    M = sum(m_splits)
    x = I.act_like(max(M, 1), K, seed)[:M]
    g = torch.Generator().manual_seed(seed + 1)
    w = (torch.randn(E, N, K, generator=g) * 0.02).to(torch.bfloat16)
    xq, xs = T.quant_block_fp32_scale(x, (1, 128), amax_floor=None, zero_scale_to_one=True)
    wq, ws = T.quant_block_fp32_scale(w, (128, 128), amax_floor=None, zero_scale_to_one=True)
    return xq, xs, wq, ws


GROUPED = [
    (8, 256, 512, [256] * 8),
    (16, 512, 1024, [128] * 16),
    (4, 2048, 7168, [256] * 4),
    (6, 256, 256, [0, 5, 130, 0, 257, 1]),
    (5, 128, 384, [0, 0, 0, 0, 0]),
    (3, 384, 512, [300, 0, 77]),
    (300, 128, 128, [i % 7 for i in range(300)]),
    # decode-sized batch: many experts of a few rows each and enough flat tiles for the launch with two tile heights
    (64, 2048, 2048, [i % 5 for i in range(64)]),
    # many rows per expert: 256-row tiles on the hand-scheduled kernel (ragged experts, empty experts)
    (8, 512, 512, [700, 0, 300, 1, 255, 256, 257, 600]),
    (16, 768, 1024, [513, 0, 0, 90, 1024, 17, 256, 300, 2, 511, 128, 129, 64, 1, 700, 333]),
    (3, 256, 384, [2048, 1, 515]),
    (4, 256, 512, [300, 0, 255, 513]),
    (6, 512, 1024, [128, 129, 256, 257, 1, 640]),
    (5, 256, 1536, [0, 0, 7, 0, 0]),
    # long K: one launch with 256 x 256 tiles for whole 256 rows (and left-overs above 128) and 128 x 256 tiles for the rest
    (6, 512, 4096, [128, 129, 256, 257, 1, 640]),
    (8, 256, 4096, [700, 0, 300, 1, 255, 256, 257, 600]),
    (5, 768, 5120, [3, 1100, 0, 127, 385]),
]


@pytest.mark.parametrize("case", GROUPED, ids=lambda c: "E%d_N%d_K%d" % c[:3])
def test_gemm_grouped(G, case):
    E, N, K, m_splits = case
    xq, xs, wq, ws = _grouped_problem(E, N, K, m_splits, seed=E + N)
    M = sum(m_splits)
    say("gemm grouped", E, N, K, "M=", M)
    offs = torch.zeros(E + 1, dtype=torch.int32)
    offs[1:] = torch.cumsum(torch.tensor(m_splits), 0)
    out = G.grouped_gemm_fp8(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), offs.cuda())
    assert tuple(out.shape) == (M, N) and out.dtype == torch.bfloat16
    if M == 0:
        return
    ref = T.grouped_gemm_fp8_ref(xq, xs, wq, ws, m_splits)
    check(out, ref, f"grouped {case[:3]}")
    assert (out.float().cpu() - ref).abs().max().item() < 1.0
    # whichever way the results leave the kernel (directly, or as row runs through LDS): the same rounded accumulators
    wide = G.grouped_gemm_fp8(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), offs.cuda(), out_dtype=torch.float32)
    assert wide.dtype == torch.float32 and torch.equal(out, wide.to(torch.bfloat16))
    say("deepgemm-style call")
    m_indices = torch.repeat_interleave(torch.arange(E), torch.tensor(m_splits)).to(torch.int32)
    out2 = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    G.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((xq.cuda(), xs.cuda()), (wq.cuda(), ws.cuda()), out2, m_indices.cuda())
    assert torch.equal(out2, out)


@pytest.mark.parametrize("case", [(8, 512, 512, [700, 0, 300, 1, 255, 256, 257, 600]), (4, 256, 1024, [300, 0, 255, 513]),
                                  (3, 384, 512, [300, 0, 77]), (6, 512, 4096, [128, 129, 256, 257, 1, 640]),
                                  (5, 768, 5120, [3, 1100, 0, 127, 385])], ids=lambda c: "E%d_N%d_K%d" % c[:3])
def test_gemm_grouped_e8m0_scales(G, case):
    """power-of-two scales on both operands: the kernels whose matrix instructions apply the scales"""
    E, N, K, m_splits = case
    M = sum(m_splits)
    say("gemm grouped e8m0", E, N, K, "M=", M)
    x = I.act_like(M, K, E + N)
    w = (torch.randn(E, N, K, generator=torch.Generator().manual_seed(E)) * 0.02).to(torch.bfloat16)
    xq, xs = T.quant_fp8_e4m3_scale_e8m0(x, (1, 128))
    wq, ws = T.quant_fp8_e4m3_scale_e8m0(w, (128, 128))
    offs = torch.zeros(E + 1, dtype=torch.int32)
    offs[1:] = torch.cumsum(torch.tensor(m_splits), 0)
    out = G.grouped_gemm_fp8(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), offs.cuda())
    ref = T.grouped_gemm_fp8_ref(xq, xs.float(), wq, ws.float(), m_splits)
    check(out, ref, f"grouped e8m0 {case[:3]}")


def test_gemm_grouped_same_bits_however_the_slots_are_dealt(G, monkeypatch):
    """The mixed-height grouped kernel lets one workgroup per CU walk its share of the tile slots, looking them up 256 at
    a time.  With 8 workgroups each walks more than one table's worth (two look-up batches); with one workgroup per
    slot nothing is walked.  All three launches must give the same bits, and the reference's result."""
    E, N, K = 96, 2048, 2048
    m_splits = [300 + (i * 37) % 500 if i % 11 else 0 for i in range(E)]
    xq, xs, wq, ws = _grouped_problem(E, N, K, m_splits, seed=5)
    M = sum(m_splits)
    offs = torch.zeros(E + 1, dtype=torch.int32)
    offs[1:] = torch.cumsum(torch.tensor(m_splits), 0)
    args = (xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), offs.cuda())
    say("gemm grouped, slot walk", E, N, K, "M=", M)
    monkeypatch.delenv("LP_GEMM_GROUPED_PERSIST", raising=False)
    out = G.grouped_gemm_fp8(*args)
    ref = T.grouped_gemm_fp8_ref(xq, xs, wq, ws, m_splits)
    check(out, ref, "grouped, one workgroup per CU")
    for grid in ("8", "0"):
        say("LP_GEMM_GROUPED_PERSIST =", grid)
        monkeypatch.setenv("LP_GEMM_GROUPED_PERSIST", grid)
        assert torch.equal(G.grouped_gemm_fp8(*args), out), grid


@pytest.mark.parametrize("K", [512, 4096], ids=["128-row-tiles", "mixed-heights"])
def test_gemm_grouped_survives_a_bad_offset_table(G, K):
    """Offsets that decrease or run past the rows are made harmless inside the kernels (both ends clamped to the row
    count, a decreasing pair = an expert without rows): the call returns, experts with a sane range get their result,
    nothing outside `out` is written (the guard rows behind it keep their fill)."""
    E, N, M = 4, 256, 800
    xq, xs, wq, ws = _grouped_problem(E, N, K, [M], seed=77)
    offs = torch.tensor([0, 300, 200, 900, 5000], dtype=torch.int32)       # expert 1 "ends" before it begins, 2 and 3 overrun
    buf = torch.full((M + 64, N), 7.0, dtype=torch.bfloat16, device="cuda")
    say("gemm grouped with a bad offset table, K =", K)
    G.grouped_gemm_fp8(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), offs.cuda(), out=buf[:M])
    torch.cuda.synchronize()
    assert (buf[M:] == 7.0).all()
    # expert 0 owns rows 0 .. 299 and the clamped expert 2 rows 200 .. 799: outside the overlap each row has one owner
    ref0 = T.grouped_gemm_fp8_ref(xq[:200], xs[:200], wq[:1], ws[:1], [200])
    check(buf[:200], ref0, "expert 0 beside bad offsets")
    ref2 = T.grouped_gemm_fp8_ref(xq[300:800], xs[300:800], wq[2:3], ws[2:3], [500])
    check(buf[300:800], ref2, "expert 2 clamped to the rows that exist")


def test_grouped_linear_module(G):
    E, N, K = 4, 256, 512
    m_splits = [100, 0, 31, 200]
    x = I.act_like(sum(m_splits), K, 5).cuda()
    w = (torch.randn(E, N, K, generator=torch.Generator().manual_seed(6)) * 0.02).to(torch.bfloat16).cuda()
    say("MyTeGroupedLinearFp8 bf16 weights")
    lin = G.MyTeGroupedLinearFp8(E)
    out = lin(x, w, m_splits)
    ref = torch.cat([x[sum(m_splits[:e]):sum(m_splits[:e + 1])].float() @ w[e].float().T for e in range(E)])
    rel = (out.float() - ref).norm() / ref.norm()
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (sum(m_splits), N) and rel.item() < 0.05
    say("MyTeGroupedLinearFp8 pre-quantised weights")
    wq, ws = G.quant_fp8_e4m3_scale_e8m0(w)
    out2 = lin(x, (wq, ws), m_splits)
    assert torch.equal(out2, out)


# ---------------------------------------------------------------------------------------------
# unscaled NT GEMM (gemm_impl): shapes and tolerance of the reference's test_gemm_fp8
NT_SHAPES = [(128, 4096, 2048), (512, 1024, 4096), (2048, 4096, 1024), (4096, 4096, 4096), (200, 1280, 4096),
             (1000, 16384, 512), (1, 16, 128), (77, 4112, 256),
             # enough tiles for the hand-scheduled loop with unit scales: a ragged last column block, and fewer columns
             # than one weight-scale block (which must stay on the compiler-scheduled kernel)
             (4096, 4112, 512), (51200, 48, 512)]


@pytest.mark.parametrize("shape", NT_SHAPES, ids=lambda s: "M%d_N%d_K%d" % s)
@pytest.mark.parametrize("kind", ["fp8", "bf16"])
def test_gemm_impl(G, shape, kind):
    say("gemm_impl", shape, kind)
    M, N, K = shape
    g = torch.Generator().manual_seed(M + N + K)
    dt = torch.float8_e4m3fn if kind == "fp8" else torch.bfloat16
    a = torch.randn(M, K, generator=g).to(dt)
    b = torch.randn(N, K, generator=g).to(dt)
    ref = a.float().cuda() @ b.float().cuda().T
    for out_dtype in ([torch.float8_e4m3fn, torch.bfloat16] if kind == "fp8" else [torch.bfloat16, torch.float32]):
        c = G.gemm_impl(a.cuda(), b.cuda(), 128, 128, 64, dtype=dt, out_dtype=out_dtype)
        assert c.dtype == out_dtype and tuple(c.shape) == (M, N)
        want = ref.clamp(-448, 448).to(out_dtype) if out_dtype == torch.float8_e4m3fn else ref.to(out_dtype)
        assert calc_diff(c.float(), want.float()) < 1e-3       # the reference's own bar (test_my_gemm_fp8.py:131)
        if out_dtype != torch.float8_e4m3fn:
            err = (c.float() - ref).abs().max() / ref.abs().max()
            assert err < (1e-2 if out_dtype == torch.bfloat16 else 1e-5), err
        else:
            # fp32 accumulation order differs from the library matmul: allow results one code apart
            ci, wi = c.view(torch.uint8).int(), want.view(torch.uint8).int()
            assert ((ci - wi).abs() <= 1).float().mean() > 0.9999


def test_gemm_impl_compile_and_profiler(G):
    """gemm_impl.compile(...).get_profiler().do_bench() as the reference's benchmark drives it
    (tests/test_gfused/test_my_gemm_fp8.py:141-163): a callable fixed to one shape, and a positive latency."""
    say("gemm_impl.compile / do_bench")
    k = G.gemm_impl.compile(M=256, N=256, K=512, dtype=torch.float8_e4m3fn, out_dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(5)
    a = torch.randint(-3, 4, (256, 512), generator=g).float().to(torch.float8_e4m3fn).cuda()
    b = torch.randint(-3, 4, (256, 512), generator=g).float().to(torch.float8_e4m3fn).cuda()
    c = k(a, b)
    assert torch.equal(c.float(), (a.float() @ b.float().T).to(torch.bfloat16).float())        # small integers: exact
    ms = k.get_profiler().do_bench(warmup=1, rep=2)
    assert ms > 0.0
    with pytest.raises(AssertionError):
        k(a[:128], b)


def test_gemm_impl_errors_and_cpu_inputs(G):
    a = torch.randn(64, 256).to(torch.bfloat16)
    b = torch.randn(32, 256).to(torch.bfloat16)
    c = G.gemm_impl(a, b)                     # CPU in -> CPU out, like every wrapper
    assert c.device.type == "cpu"
    assert calc_diff(c.float(), a.float() @ b.float().T) < 1e-4
    with pytest.raises(TypeError):
        G.gemm_impl(a.half(), b.half(), dtype=torch.float16)
    with pytest.raises(Exception):
        G.gemm_impl(a[:, :100].contiguous(), b[:, :100].contiguous())      # K not a multiple of 64


# ---------------------------------------------------------------------------------------------
# backward of the grouped linear (gpatch_v4/models/deepseek_v4/fp8.py:285-343)
def test_quant_colwise_t_matches_oracle(G):
    say("quant_fp8_colwise_t")
    m_splits = [300, 0, 128, 1, 77, 513]
    x = I.act_like(sum(m_splits), 384, 21)
    x[5, 7] = 0.0
    # columns of the first block whose maxima sit on, just above and just below 448 * 2^k (where the scale exponent
    # steps), an all-zero column, maxima below the smallest normal float and near the largest
    edge = [3584.0, 3600.0, 3568.0, 0.0, 2.0 ** -130, 1.75 * 2.0 ** -126, 1.7578125 * 2.0 ** -126, 3.0e38,
            448.0 * 2.0 ** -20, 450.0 * 2.0 ** -20, 2.0 ** -133]
    for c, v in enumerate(edge):
        x[:128, c] *= 2.0 ** -140 if v < 1e-30 else min(1.0, abs(v) * 0.01)
        if v == 0.0:
            x[:128, c] = 0.0
        else:
            x[(7 * c + 3) % 128, c] = -v if c % 2 else v
    offs = torch.zeros(len(m_splits) + 1, dtype=torch.int32)
    offs[1:] = torch.cumsum(torch.tensor(m_splits), 0)
    for dt in (torch.bfloat16, torch.float32):
        xin = x.to(dt)
        q, s, nblk = G.quant_fp8_colwise_t(xin.cuda(), offs.cuda(), m_splits, pad_rows=128)
        want = T.quant_colwise_t(xin, m_splits)
        assert nblk == [3, 0, 1, 1, 1, 5]
        done = 0
        for e, (wq, ws) in enumerate(want):
            p = nblk[e] * 128
            got_q = q[384 * done * 128:384 * (done * 128 + p)].view(384, p).cpu()
            got_s = s.view(torch.uint8)[384 * done:384 * (done + nblk[e])].view(384, nblk[e]).cpu()
            assert torch.equal(got_q, wq.view(torch.uint8)), (dt, e)
            assert torch.equal(got_s, ws.view(torch.uint8)), (dt, e)
            done += nblk[e]
    # padding to 512 rows: the same codes and scales, followed by blocks of zero codes with scale 1
    q5, s5, nblk5 = G.quant_fp8_colwise_t(x.to(torch.bfloat16).cuda(), offs.cuda(), m_splits, pad_rows=512)
    assert nblk5 == [4, 0, 4, 4, 4, 8]
    want = T.quant_colwise_t(x.to(torch.bfloat16), m_splits)
    done = 0
    for e, (wq, ws) in enumerate(want):
        p5, nb = nblk5[e] * 128, wq.shape[1] // 128
        got_q = q5[384 * done * 128:384 * (done * 128 + p5)].view(384, p5).cpu()
        got_s = s5.view(torch.uint8)[384 * done:384 * (done + nblk5[e])].view(384, nblk5[e]).cpu()
        if p5:
            assert torch.equal(got_q[:, :nb * 128], wq.view(torch.uint8)) and not got_q[:, nb * 128:].any()
            assert torch.equal(got_s[:, :nb], ws.view(torch.uint8)) and bool((got_s[:, nb:] == 127).all())
        done += nblk5[e]
    # mixed padding: experts of at most 256 rows to multiples of 128, the others to multiples of 512
    import gcore_lowp._abi as _A
    qm, sm_, nblkm = G.quant_fp8_colwise_t(x.to(torch.bfloat16).cuda(), offs.cuda(), m_splits, pad_rows=_A.PAD_MIXED)
    assert nblkm == [4, 0, 1, 1, 1, 8]
    done = 0
    for e, (wq, ws) in enumerate(want):
        pm, nb = nblkm[e] * 128, wq.shape[1] // 128
        got_q = qm[384 * done * 128:384 * (done * 128 + pm)].view(384, pm).cpu()
        got_s = sm_.view(torch.uint8)[384 * done:384 * (done + nblkm[e])].view(384, nblkm[e]).cpu()
        if pm:
            assert torch.equal(got_q[:, :nb * 128], wq.view(torch.uint8)) and not got_q[:, nb * 128:].any(), e
            assert torch.equal(got_s[:, :nb], ws.view(torch.uint8)) and bool((got_s[:, nb:] == 127).all()), e
        done += nblkm[e]


@pytest.mark.parametrize("shape", [(128, 128, 128), (512, 384, 256), (256, 384, 128), (4096, 7168, 256), (300, 256, 1024), (4096, 7168, 384), (128, 128, 512),
                                   (1000, 640, 2048), (4096, 7168, 1024), (77, 128, 1536)],
                         ids=lambda s: "M%d_N%d_K%d" % s)
def test_gemm_rowscale(G, shape):
    M, N, K = shape
    say("gemm rowscale", shape)
    a = I.act_like(M, K, 3)
    b = I.act_like(N, K, 4) * 0.05
    aq, a_s = T.quant_fp8_e4m3_scale_e8m0(a, (1, 128))
    bq, b_s = T.quant_fp8_e4m3_scale_e8m0(b, (1, 128))
    ref = (T.dequant_act_f32(aq.cuda(), a_s.float().cuda()) @ T.dequant_act_f32(bq.cuda(), b_s.float().cuda()).T)
    outs = {}
    for dt in (torch.float32, torch.bfloat16):           # bf16 leaves through the LDS-staged epilogue
        out = torch.full((M, N), float("nan"), dtype=dt, device="cuda")
        G.gemm_fp8_rowscale(aq.view(torch.uint8).cuda(), a_s.view(torch.uint8).cuda(), bq.view(torch.uint8).cuda(),
                            b_s.view(torch.uint8).cuda(), M, N, K, out)
        check(out, ref, f"rowscale {shape} {dt}")
        outs[dt] = out
    assert torch.equal(outs[torch.bfloat16], outs[torch.float32].to(torch.bfloat16)), "bf16 output is the rounded fp32 output"


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_gemm_rowscale_grouped_equals_per_problem_launches(G, out_dtype):
    """The grouped launches (one per kind of problem: K a multiple of 512, one K block, two K blocks, the rest) write what
    one lp_gemm_fp8_rowscale launch per problem writes, bit for bit: same kernels, same order of summation.  K blocks per
    problem cover multiples of 4, one and two blocks (the kernel without a K loop), other counts and an empty problem,
    which is zero-filled."""
    M, N = 256, 384
    k_blocks = [4, 1, 0, 8, 3, 12, 0, 5, 2, 1, 2]
    say("gemm rowscale grouped", (M, N), k_blocks, out_dtype)
    total = sum(k_blocks)
    a = I.act_like(M, total * 128, 21)
    b = I.act_like(N, total * 128, 22) * 0.05
    aq, a_s = T.quant_fp8_e4m3_scale_e8m0(a, (1, 128))
    bq, b_s = T.quant_fp8_e4m3_scale_e8m0(b, (1, 128))
    # problem e's operands stored as [M, K_e] / [N, K_e] one after the other
    cut = lambda t, w: torch.cat([t[:, w * sum(k_blocks[:e]):w * sum(k_blocks[:e + 1])].contiguous().view(torch.uint8).flatten()
                                  for e in range(len(k_blocks))]).cuda()
    aqf, asf, bqf, bsf = cut(aq, 128), cut(a_s, 1), cut(bq, 128), cut(b_s, 1)
    out = torch.full((len(k_blocks), M, N), float("nan"), dtype=out_dtype, device="cuda")
    G.gemm_fp8_rowscale_grouped(aqf, asf, bqf, bsf, k_blocks, M, N, out)
    before = 0
    for e, kb in enumerate(k_blocks):
        if kb == 0:
            assert not out[e].any()
            continue
        one = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
        G.gemm_fp8_rowscale(aqf[M * 128 * before:], asf[M * before:], bqf[N * 128 * before:], bsf[N * before:], M, N, kb * 128, one)
        assert torch.equal(out[e], one), (e, kb)
        sl = slice(before * 128, (before + kb) * 128)
        ref = T.dequant_act_f32(aq[:, sl].cuda(), a_s[:, before:before + kb].float().cuda()) @ \
            T.dequant_act_f32(bq[:, sl].cuda(), b_s[:, before:before + kb].float().cuda()).T
        check(out[e], ref, f"rowscale grouped problem {e} kb={kb}")
        before += kb
    # A table that breaks the caller's promises: an entry with more K blocks than max_k_blocks, one whose count is not a
    # multiple of the promised 4, a negative slot.  The table is device memory, so the host cannot refuse it: such an entry
    # must compute and write nothing (its output keeps its contents), and the entries beside it are served as usual.
    from gcore_lowp import _abi as A
    table = torch.tensor([[0, 4, 0, 0], [1, 16, 0, 0], [2, 3, 4, 0], [-1, 4, 0, 0], [3, 8, 5, 0]], dtype=torch.int32, device="cuda")
    out2 = torch.full((4, M, N), 7.0, dtype=out_dtype, device="cuda")
    A.check(A.lib().lp_gemm_fp8_rowscale_grouped(aqf.data_ptr(), asf.data_ptr(), bqf.data_ptr(), bsf.data_ptr(), A.E8M0, table.data_ptr(), 5, 8, 4,
                                                 M, N, out2.data_ptr(), A.BF16 if out_dtype == torch.bfloat16 else A.F32, A.stream_ptr()))
    torch.cuda.synchronize()
    assert torch.equal(out2[0], out[0])                      # problem 0: 4 blocks from block 0
    assert bool((out2[1] == 7).all()) and bool((out2[2] == 7).all())           # 16 > max_k_blocks; 3 is not a multiple of 4
    assert torch.equal(out2[3], out[3])                      # problem 3: 8 blocks behind the 5 of problems 0 .. 2
    # the same for the kernel of one-block problems: an entry of another size, or with a negative slot, writes nothing
    table = torch.tensor([[0, 1, 4, 0], [1, 2, 25, 0], [-1, 1, 4, 0], [2, 1, 35, 0]], dtype=torch.int32, device="cuda")
    out3 = torch.full((3, M, N), 7.0, dtype=out_dtype, device="cuda")
    A.check(A.lib().lp_gemm_fp8_rowscale_grouped(aqf.data_ptr(), asf.data_ptr(), bqf.data_ptr(), bsf.data_ptr(), A.E8M0, table.data_ptr(), 4, 1, 1,
                                                 M, N, out3.data_ptr(), A.BF16 if out_dtype == torch.bfloat16 else A.F32, A.stream_ptr()))
    torch.cuda.synchronize()
    assert torch.equal(out3[0], out[1]) and bool((out3[1] == 7).all()) and torch.equal(out3[2], out[9])


@pytest.mark.parametrize("case", [([300, 0, 128, 1, 77, 513], 512, 512), ([2048, 16, 700], 1024, 2048), ([64, 64, 64, 64], 2048, 512),
                                  ([1000, 5, 0, 260, 129], 512, 4096)],
                         ids=lambda c: "E%d_N%d_K%d" % (len(c[0]), c[1], c[2]))
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_gemm_grouped_nn_equals_transposed_weights(G, case, out_dtype):
    """The data gradient's GEMM on the stored weights, out_e = x_e W_e with W [E, K, N] (layout NN,
    gpatch_v4/models/deepseek_v4/fp8.py:301-313): the kernel that turns the weight operand on its way out of LDS gives the
    bits of the NT kernel on a transposed copy of the weights (same products, same order of accumulation), and both are
    the fp32 dequantise-then-matmul within the GEMM tolerance."""
    m_splits, N, K = case
    E, M = len(m_splits), sum(m_splits)
    say("grouped NN", m_splits, N, K, out_dtype)
    g = torch.Generator().manual_seed(N + K + M)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(E, K, N, generator=g) * 0.05).to(torch.bfloat16).cuda()
    xq, xs = G.quant_fp8_e4m3_scale_e8m0(x, (1, 128))
    wq, ws = G.quant_fp8_e4m3_scale_e8m0(w, (128, 128))
    offs = torch.zeros(E + 1, dtype=torch.int32)
    offs[1:] = torch.cumsum(torch.tensor(m_splits), 0)
    out = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    G.grouped_gemm_fp8_nn(xq, xs, wq, ws, offs.cuda(), out=out)
    wt = wq.view(torch.uint8).transpose(1, 2).contiguous().view(torch.float8_e4m3fn)
    wst = ws.view(torch.uint8).transpose(1, 2).contiguous().view(torch.float8_e8m0fnu)
    want = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    G.grouped_gemm_fp8(xq, xs, wt, wst, offs.cuda(), out=want)
    assert torch.equal(out.view(torch.int16 if out_dtype == torch.bfloat16 else torch.int32),
                       want.view(torch.int16 if out_dtype == torch.bfloat16 else torch.int32))
    xd = T.dequant_act_f32(xq, xs.float())
    off = 0
    for e, m in enumerate(m_splits):
        if m:
            wd = T.dequant_weight_f32(wq[e], ws[e].float())
            check(out[off:off + m], xd[off:off + m] @ wd, f"grouped NN expert {e}")
        off += m
    # a shape the kernel does not take (N not a multiple of 512) goes through the transposed copy inside the wrapper
    if N == 512:
        w2 = w[:, :, :384].contiguous()
        wq2, ws2 = G.quant_fp8_e4m3_scale_e8m0(w2, (128, 128))
        got = G.grouped_gemm_fp8_nn(xq, xs, wq2, ws2, offs.cuda(), out_dtype=out_dtype, total_rows=M)
        off = 0
        for e, m in enumerate(m_splits):
            if m:
                check(got[off:off + m], xd[off:off + m] @ T.dequant_weight_f32(wq2[e], ws2[e].float()), f"grouped NN fallback expert {e}")
            off += m


@pytest.mark.parametrize("m_splits", [[8192, 16, 2048, 256], [32, 1, 2000, 323], [100, 0, 31, 200], [2048, 1024, 0, 4096]],
                         ids=["even", "uneven", "empty", "pad512"])
def test_grouped_linear_backward(G, m_splits):
    """tests/test_gfused/test_te_gemm_fp8.py:543-585: forward, input gradient and weight gradient within 5 % (norm)
    of per-expert bf16 matmuls; TransformerEngine itself is not available, so its bit-exact comparison (:475-503)
    has no counterpart here."""
    E, H_IN, H_OUT = len(m_splits), 256, 512
    say("grouped linear fwd+bwd", m_splits)
    torch.manual_seed(11)
    x = torch.randn(sum(m_splits), H_IN, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    w = torch.randn(E, H_OUT, H_IN, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    xr, wr = x.detach().clone().requires_grad_(True), w.detach().clone().requires_grad_(True)
    outs, off = [], 0
    for i, m in enumerate(m_splits):
        outs.append(xr[off:off + m] @ wr[i].T)
        off += m
    ref = torch.cat(outs)
    g = torch.randn_like(ref)
    ref.backward(g)
    lin = G.MyTeGroupedLinearFp8(E)
    out = lin(x, w, m_splits)
    out.backward(g)
    rel = lambda a, b: ((a.float() - b.float()).norm() / b.float().norm()).item()
    assert out.shape == ref.shape and rel(out, ref) < 0.05
    assert x.grad.shape == x.shape and rel(x.grad, xr.grad) < 0.05
    assert w.grad.shape == w.shape and rel(w.grad, wr.grad) < 0.05
    assert torch.isfinite(out).all() and torch.isfinite(x.grad).all() and torch.isfinite(w.grad).all()
    for e, m in enumerate(m_splits):
        if m == 0:
            assert not w.grad[e].any()
    # exact identities of the construction: dgrad = quantised dY times the dequantised weight, in fp32
    from gcore_lowp.eager_quant_kernels import quant_fp8_e4m3_scale_e8m0
    wq, ws = quant_fp8_e4m3_scale_e8m0(w.detach(), block_size=(128, 128))
    gq, gs = quant_fp8_e4m3_scale_e8m0(g, block_size=(1, 128))
    wd = T.dequant_weight_f32(wq.view(E * H_OUT, H_IN), ws.float().view(-1, H_IN // 128)).view(E, H_OUT, H_IN)
    gd = T.dequant_act_f32(gq, gs.float())
    off = 0
    for e, m in enumerate(m_splits):
        if m:
            check(x.grad[off:off + m], gd[off:off + m] @ wd[e], f"dgrad expert {e}")
        off += m
    # pre-quantised weights give the same forward and input gradient (:587-612)
    x2 = x.detach().clone().requires_grad_(True)
    out2 = lin(x2, (wq, ws), m_splits)
    out2.backward(g)
    assert torch.equal(out2, out) and torch.equal(x2.grad, x.grad)


def test_gemm_skinny_pair_opt_in():
    """The K-split weight-streaming kernel pair is no longer chosen by default; LP_GEMM_SKINNY=1 selects it (the
    switch is read once per process, hence the child process).  Decode shapes with caller workspace, against the
    fp32 dequantise-then-matmul reference, to the path's tolerance."""
    import os
    import subprocess
    import sys
    say("gemm skinny pair (LP_GEMM_SKINNY=1, child process)")
    code = r'''
import sys, torch
import gcore_lowp as G
torch.manual_seed(3)
for (M, N, K) in ((8, 2048, 7168), (33, 4096, 14336), (64, 1536, 3584), (16, 4096, 7168)):
    a = torch.randn(M, K, device="cuda"); b = torch.randn(N, K, device="cuda") * 0.02
    aq, as_ = G.quant_1d(a); bq, bs = G.quant_2d(b)
    print("[case] skinny", M, N, K, flush=True)
    c = G.gemm_fp8_block_scaling_impl(aq, as_, bq, bs)
    ref = (aq.float() * as_.repeat_interleave(128, 1)) @ (bq.float() * bs.repeat_interleave(128, 0).repeat_interleave(128, 1)).t()
    err = (c.float() - ref).abs().max().item() / ref.abs().max().item()
    cos = torch.nn.functional.cosine_similarity(c.float().flatten(), ref.flatten(), dim=0).item()
    assert err <= 2e-2 and cos >= 0.9999, (M, N, K, err, cos)
print("ok")
'''
    env = dict(os.environ, LP_GEMM_SKINNY="1", PYTHONPATH=os.pathsep.join(p for p in sys.path if p))
    env.pop("LP_GEMM_NO_SKINNY", None)
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=200)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), (r.stdout[-1500:], r.stderr[-1500:])


def test_gemm_column_split_one_launch_equals_two_launches(G):
    """The single-launch column split (256 x 256 tiles, then K-split 128 x 128 tiles) gives bit for bit what the two
    launches it replaces give; LP_GEMM_MIXED=0 restores those (the switch is read once per process, hence the child
    process, which prints a digest of every output)."""
    import hashlib
    import os
    import subprocess
    import sys
    say("gemm column split: one launch against two (LP_GEMM_MIXED=0 in a child process)")
    shapes = ((2048, 9472, 1024), (1900, 9472, 2048))          # 296 tiles of 256 x 256: one round and 40 left over

    def digests():
        out = []
        for (M, N, K) in shapes:
            for pow2 in (False, True):
                xq, xs, wq, ws = quantized_problem(M, N, K, seed=M + K, pow2=pow2)
                c = G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda())
                out.append(hashlib.md5(c.view(torch.int16).cpu().numpy().tobytes()).hexdigest())
        return out

    code = (
        "import sys, hashlib, torch\n"
        "import gcore_lowp as G\n"
        "sys.path.insert(0, %r)\n"
        "from tests import test_gpu_gemm as t\n"
        "for (M, N, K) in %r:\n"
        "    for pow2 in (False, True):\n"
        "        xq, xs, wq, ws = t.quantized_problem(M, N, K, seed=M + K, pow2=pow2)\n"
        "        print('[case] two launches', M, N, K, pow2, flush=True)\n"
        "        c = G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda())\n"
        "        print('md5', hashlib.md5(c.view(torch.int16).cpu().numpy().tobytes()).hexdigest(), flush=True)\n"
    ) % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))), shapes)
    env = dict(os.environ, LP_GEMM_MIXED="0", PYTHONPATH=os.pathsep.join(p for p in sys.path if p))
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, (r.stdout[-1500:], r.stderr[-1500:])
    theirs = [l.split()[1] for l in r.stdout.splitlines() if l.startswith("md5 ")]
    assert len(theirs) == 2 * len(shapes) and theirs == digests(), (theirs, r.stdout[-800:])


@pytest.mark.parametrize("width,shapes", [(288, ((2048, 4608, 512), (1000, 13824, 512), (333, 27648, 1024))),
                                          (224, ((2048, 3584, 512), (1000, 10752, 512), (333, 21504, 1024)))])
def test_gemm_wide_tile_forced_on_other_shapes(G, width, shapes):
    """The 256 x 288 and 256 x 224 tile kernels are chosen by themselves only where they fill whole rounds of CUs;
    LP_GEMM_WIDE=288 or 224 (read once per process, hence the child) sends every prefill-sized problem whose N is a
    multiple of that width to it: few tile columns, ragged M, tile origins at every offset inside a weight-scale block
    (wave columns that straddle two blocks and, for 224, wave columns inside one), both scale types; with
    power-of-two scales the result must equal the default kernels' bit for bit (same order of summation)."""
    import hashlib
    import os
    import subprocess
    import sys
    say(f"gemm 256 x {width} tiles forced (LP_GEMM_WIDE={width} in a child process)")
    mine = []
    for (M, N, K) in shapes:
        xq, xs, wq, ws = quantized_problem(M, N, K, seed=M + K, pow2=True)
        c = G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda())
        mine.append(hashlib.md5(c.view(torch.int16).cpu().numpy().tobytes()).hexdigest())
    code = (
        "import sys, hashlib, torch\n"
        "import gcore_lowp as G\n"
        "sys.path.insert(0, %r)\n"
        "from tests import test_gpu_gemm as t\n"
        "for (M, N, K) in %r:\n"
        "    for pow2 in (False, True):\n"
        "        xq, xs, wq, ws = t.quantized_problem(M, N, K, seed=M + K, pow2=pow2)\n"
        "        print('[case] wide tiles', M, N, K, pow2, flush=True)\n"
        "        c = G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda())\n"
        "        wide = G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), out_dtype=torch.float32)\n"
        "        assert torch.equal(c, wide.to(torch.bfloat16))\n"
        "        t.check(c, t.ref_gemm(xq, xs, wq, ws), 'forced wide %%s' %% ((M, N, K),))\n"
        "        if pow2:\n"
        "            print('md5', hashlib.md5(c.view(torch.int16).cpu().numpy().tobytes()).hexdigest(), flush=True)\n"
    ) % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))), shapes)
    env = dict(os.environ, LP_GEMM_WIDE=str(width), PYTHONPATH=os.pathsep.join(p for p in sys.path if p))
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, (r.stdout[-1500:], r.stderr[-1500:])
    theirs = [l.split()[1] for l in r.stdout.splitlines() if l.startswith("md5 ")]
    assert theirs == mine, (theirs, mine, r.stdout[-800:])



def test_gemm_four_wave_loop_equals_the_eight_wave_loop(G):
    """The opt-in 256 x 256 loop on four waves with the accumulators in the accumulation registers (LP_GEMM_QUAD=1, read
    once per process, hence the child): e8m0 problems of whole tiles must give the default kernel's bits (same order of
    summation), bf16 output must be the rounded fp32 output, and the unscaled NT route through it is checked against
    an fp32 matmul for all three output types."""
    import hashlib
    import os
    import subprocess
    import sys
    say("gemm four-wave loop (LP_GEMM_QUAD=1 in a child process)")
    shapes = ((4096, 4096, 512), (2048, 8192, 1024), (2560, 5120, 1536), (4096, 7168, 2048))
    mine = []
    for (M, N, K) in shapes:
        xq, xs, wq, ws = quantized_problem(M, N, K, seed=M + K, pow2=True)
        c = G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda())
        mine.append(hashlib.md5(c.view(torch.int16).cpu().numpy().tobytes()).hexdigest())
    code = (
        "import sys, hashlib, torch\n"
        "import gcore_lowp as G\n"
        "sys.path.insert(0, %r)\n"
        "from tests import test_gpu_gemm as t\n"
        "for (M, N, K) in %r:\n"
        "    xq, xs, wq, ws = t.quantized_problem(M, N, K, seed=M + K, pow2=True)\n"
        "    print('[case] four waves', M, N, K, flush=True)\n"
        "    c = G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda())\n"
        "    wide = G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), out_dtype=torch.float32)\n"
        "    assert torch.equal(c, wide.to(torch.bfloat16))\n"
        "    t.check(c, t.ref_gemm(xq, xs, wq, ws), 'four waves %%s' %% ((M, N, K),))\n"
        "    print('md5', hashlib.md5(c.view(torch.int16).cpu().numpy().tobytes()).hexdigest(), flush=True)\n"
        "g = torch.Generator(device='cuda').manual_seed(5)\n"
        "a = torch.randn(4096, 1024, generator=g, device='cuda').to(torch.float8_e4m3fn)\n"
        "b = torch.randn(4096, 1024, generator=g, device='cuda').to(torch.float8_e4m3fn)\n"
        "ref = a.float() @ b.float().T\n"
        "for od, tol in ((torch.bfloat16, 8e-3), (torch.float32, 1e-4), (torch.float8_e4m3fn, 7e-2)):\n"
        "    print('[case] four waves, unscaled NT', od, flush=True)\n"
        "    c = G.gemm_impl(a, b, dtype=torch.float8_e4m3fn, out_dtype=od)\n"
        "    r = ref.clamp(-448, 448) if od == torch.float8_e4m3fn else ref\n"
        "    err = (c.float() - r).abs().max().item() / r.abs().max().item()\n"
        "    assert err < tol, (od, err)\n"
    ) % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))), shapes)
    env = dict(os.environ, LP_GEMM_QUAD="1", LP_GEMM_WIDE="0", PYTHONPATH=os.pathsep.join(p for p in sys.path if p))
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, (r.stdout[-1500:], r.stderr[-1500:])
    theirs = [l.split()[1] for l in r.stdout.splitlines() if l.startswith("md5 ")]
    assert theirs == mine, (theirs, mine, r.stdout[-800:])


@pytest.mark.parametrize("shape", [(64, 18432, 7168), (17, 18432, 1024), (16, 18432, 7168), (9, 8192, 1024), (33, 16384, 2048), (48, 12288, 896), (64, 8320, 512), (64, 6144, 7168), (20, 7168, 2048),
                                   (40, 18560, 3584), (64, 36864, 1536)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("pow2", [False, True], ids=["f32scale", "e8m0scale"])
def test_gemm_decode_rows_against_many_weight_rows(G, shape, pow2):
    """9 .. 64 activation rows against more than 4096 weight rows: the kernel that gives a workgroup 8 R weight rows
    (R = 4 .. 10, chosen from N), so rows per workgroup that are not a multiple of 16 (R = 9), a last workgroup with
    rows missing (18560 = 257 x 72 + 56), runs of 1 .. 7 K blocks per wave including a last wave with fewer (896 = 7
    blocks over 8 waves), blocks of 16 rows that straddle two weight-scale blocks."""
    M, N, K = shape
    xq, xs, wq, ws = quantized_problem(M, N, K, seed=M + N + K, pow2=pow2)
    say("decode rows", shape, "e8m0" if pow2 else "f32")
    c = G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda())
    wide = G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), out_dtype=torch.float32)
    assert torch.equal(c, wide.to(torch.bfloat16))
    check(c, ref_gemm(xq, xs, wq, ws), f"decode rows {shape}")
    assert torch.equal(c, G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda()))
