"""GPU parity at the exact shapes the benchmark times (the other GPU tests reach the same kernels at reduced
sizes): the prefill GEMM 2048 x 18432 x 7168 with both scale types, the whole 256-expert grouped problem with the
benchmark's row histogram plus an appended expert without rows, and the whole-layer FP4 conversions.

Operands are produced on the GPU by the library's own quantisers, which the small-size tests pin bit for bit against
the CPU oracles; the GEMM reference is an fp32 dequantise-then-matmul on the GPU (tests/test_gfused/test_my_gemm_fp8.py:
217-243, tests/test_gpatch_v4/test_deep_gemm_grouped_gemm_fp8.py:75-135).  Bars: max relative error <= 2e-2 of the
largest |reference| entry, cosine >= 0.9999, calc_diff < 1e-5."""
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


def _randn(rows, cols, std, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.empty(rows, cols, dtype=torch.bfloat16, device="cuda")
    for r in range(0, rows, 16384):
        x[r:r + 16384].normal_(0.0, std, generator=g)
    return x


def _bars(out, ref, what):
    out, ref = out.float(), ref.float()
    assert torch.isfinite(out).all(), what
    denom = max(ref.abs().max().item(), 1e-30)
    max_rel = (out - ref).abs().max().item() / denom
    o, r = out.flatten().double(), ref.flatten().double()
    cos = (torch.dot(o, r) / (o.norm() * r.norm()).clamp(min=1e-300)).item()
    cd = float(1 - 2 * torch.dot(o, r) / (torch.dot(o, o) + torch.dot(r, r)).clamp(min=1e-300))
    assert max_rel <= 2e-2 and cos >= 0.9999 and cd < 1e-5, (what, max_rel, cos, cd)
    return max_rel, cos


def _f32(s):
    """Scales as fp32; e8m0 bytes are decoded from their bits (2^(b - 127); the quantisers never emit byte 0 or 255 here)."""
    if s.dtype == E8M0:
        return (s.view(torch.uint8).to(torch.int32) << 23).view(torch.float32)
    return s.float()


def _dequant_w(wq, ws):
    return wq.float() * _f32(ws).repeat_interleave(128, 0).repeat_interleave(128, 1)


def _dequant_a(xq, xs):
    return xq.float() * _f32(xs).repeat_interleave(128, 1)


@pytest.mark.parametrize("shape", [(2048, 18432, 7168), (4096, 7168, 18432)], ids=["config2", "deepK"])
@pytest.mark.parametrize("pow2", [False, True], ids=["f32scale", "e8m0scale"])
def test_prefill_gemm_at_benchmark_shape(G, pow2, shape):
    M, N, K = shape
    x, w = _randn(M, K, 1.0, 11), _randn(N, K, 0.02, 12)
    if pow2:
        xq, xs = G.quant_fp8_e4m3_scale_e8m0(x, (1, 128))
        wq, ws = G.quant_fp8_e4m3_scale_e8m0(w, (128, 128))
    else:
        xq, xs = G.quant_1d(x)
        wq, ws = G.quant_2d(w)
    del x, w
    say("prefill gemm", (M, N, K), "e8m0" if pow2 else "f32")
    out = G.gemm_fp8_block_scaling_impl(xq, xs, wq, ws)
    wide = G.gemm_fp8_block_scaling_impl(xq, xs, wq, ws, out_dtype=torch.float32)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (M, N)
    ref = _dequant_a(xq, xs) @ _dequant_w(wq, ws).T
    max_rel, cos = _bars(out, ref, "prefill gemm")
    print(f"    max_rel={max_rel:.3e} cos={cos:.7f}", flush=True)
    assert torch.equal(out, wide.to(torch.bfloat16))
    # a second call gives the same bits (no race between the tiles of one launch)
    assert torch.equal(out, G.gemm_fp8_block_scaling_impl(xq, xs, wq, ws))


@pytest.mark.parametrize("pow2", [False, True], ids=["f32scale", "e8m0scale"])
def test_gemm_at_the_reference_benchmarks_largest_shape(G, pow2):
    """8096 x 129280 x 4096 (tests/test_gfused/test_my_gemm_fp8.py:280: a vocabulary projection; 8096 rows end inside a
    256-row tile, 2.1 GB of bf16 output): checked slab by slab of 16160 weight rows against fp32 dequantise-then-matmul."""
    M, N, K = 8096, 129280, 4096
    x, w = _randn(M, K, 1.0, 21), _randn(N, K, 0.02, 22)
    if pow2:
        xq, xs = G.quant_fp8_e4m3_scale_e8m0(x, (1, 128))
        wq, ws = G.quant_fp8_e4m3_scale_e8m0(w, (128, 128))
    else:
        xq, xs = G.quant_1d(x)
        wq, ws = G.quant_2d(w)
    del x, w
    say("largest reference benchmark shape", (M, N, K), "e8m0" if pow2 else "f32")
    out = G.gemm_fp8_block_scaling_impl(xq, xs, wq, ws)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (M, N)
    a = _dequant_a(xq, xs)
    slab = 16160                                           # 126.25 x 128 rows: slab borders inside scale blocks and tiles
    for n0 in range(0, N, slab):
        n1 = min(n0 + slab, N)
        lo, hi = n0 // 128 * 128, (n1 + 127) // 128 * 128
        wd = _dequant_w(wq[lo:hi], ws[lo // 128:hi // 128])[n0 - lo:n1 - lo]
        _bars(out[:, n0:n1], a @ wd.T, f"slab {n0}")
        del wd


@pytest.mark.parametrize("pow2", [False, True], ids=["f32scale", "e8m0scale"])
def test_decode_rows_against_the_vocabulary_projection(G, pow2):
    """1 ... 64 rows x 129280 x 7168: the same vocabulary weight as a decode step sees it (8080 workgroups of 16 weight rows
    on the ring kernel up to 8 rows, rounds of 256 workgroups on the many-rows kernel up to 32, the tiled kernels above), one weight quantised once,
    checked slab by slab against fp32 dequantise-then-matmul."""
    N, K = 129280, 7168
    w = _randn(N, K, 0.02, 32)
    wq, ws = G.quant_fp8_e4m3_scale_e8m0(w, (128, 128)) if pow2 else G.quant_2d(w)
    del w
    for M in (1, 7, 16, 24, 40, 64):
        x = _randn(M, K, 1.0, 40 + M)
        xq, xs = G.quant_fp8_e4m3_scale_e8m0(x, (1, 128)) if pow2 else G.quant_1d(x)
        say("decode rows x vocabulary projection", (M, N, K), "e8m0" if pow2 else "f32")
        out = G.gemm_fp8_block_scaling_impl(xq, xs, wq, ws)
        assert out.dtype == torch.bfloat16 and tuple(out.shape) == (M, N)
        a = _dequant_a(xq, xs)
        slab = 16160
        for n0 in range(0, N, slab):
            n1 = min(n0 + slab, N)
            lo, hi = n0 // 128 * 128, (n1 + 127) // 128 * 128
            wd = _dequant_w(wq[lo:hi], ws[lo // 128:hi // 128])[n0 - lo:n1 - lo]
            _bars(out[:, n0:n1], a @ wd.T, f"M {M} slab {n0}")
            del wd


@pytest.mark.parametrize("proj,N,K", [("gate_up", 4096, 7168), ("down", 7168, 2048)])
@pytest.mark.parametrize("pow2", [False, True], ids=["f32scale", "e8m0scale"])
def test_grouped_gemm_at_benchmark_shape(G, proj, N, K, pow2):
    """The benchmark's 256 experts and rows per expert (Zipf 1.1, top-8 of 8192 tokens, one expert without rows in the
    middle of the list) and a 257th expert without rows at the end; every expert's rows are checked against its own
    fp32 dequantise-then-matmul."""
    m_splits = I.zipf_m_splits_with_idle_expert().tolist() + [0]
    E, Mt = len(m_splits), sum(m_splits)
    assert Mt == 65536 and E == 257 and m_splits.count(0) == 2 and m_splits[128] == 0
    x = _randn(Mt, K, 1.0, 21)
    xq, xs = (G.quant_fp8_e4m3_scale_e8m0(x, (1, 128)) if pow2 else G.quant_act(x))
    del x
    wq = torch.empty(E, N, K, dtype=E4M3, device="cuda")
    ws = torch.empty(E, N // 128, K // 128, dtype=E8M0 if pow2 else torch.float32, device="cuda")
    for e0 in range(0, E, 32):
        e1 = min(e0 + 32, E)
        w = _randn((e1 - e0) * N, K, 0.02, 100 + e0).view(e1 - e0, N, K)
        q, s = (G.quant_fp8_e4m3_scale_e8m0(w, (128, 128)) if pow2 else G.quant_weight(w))
        wq[e0:e1], ws[e0:e1] = q, s
        del w, q, s
    offs = torch.zeros(E + 1, dtype=torch.int32)
    offs[1:] = torch.cumsum(torch.tensor(m_splits), 0)
    say("grouped gemm", proj, "E=", E, "rows=", Mt, "max", max(m_splits), "min", min(m_splits[:-1]), "e8m0" if pow2 else "f32")
    out = G.grouped_gemm_fp8(xq, xs, wq, ws, offs.cuda(), total_rows=Mt)
    assert tuple(out.shape) == (Mt, N) and out.dtype == torch.bfloat16
    worst = (0.0, 1.0)
    order = sorted((e for e in range(E) if m_splits[e] > 0), key=lambda e: m_splits[e])        # the experts that have rows
    assert len(order) == E - 2
    for e in [order[0], order[-1]] + order[1:-1]:          # lightest and heaviest first
        r0, r1 = int(offs[e]), int(offs[e + 1])
        ref = _dequant_a(xq[r0:r1], xs[r0:r1]) @ _dequant_w(wq[e], ws[e]).T
        max_rel, cos = _bars(out[r0:r1], ref, f"{proj} expert {e} rows {r1 - r0}")
        worst = (max(worst[0], max_rel), min(worst[1], cos))
    print(f"    worst expert: max_rel={worst[0]:.3e} cos={worst[1]:.7f}", flush=True)


def _same(a, b):
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a.contiguous().view(torch.uint8), b.contiguous().view(torch.uint8))


@pytest.mark.parametrize("rows,cols", [(256 * 2048, 7168), (256 * 7168, 2048)])
def test_fp4_conversions_at_whole_layer_launch_shapes(G, rows, cols):
    """One launch over the 256 stacked experts of a tensor kind, as the benchmark times it: 128-row slabs of the
    result (first, an expert boundary in the middle, last) equal the same kernel on that slab alone, and one slab is
    checked against the CPU oracle directly."""
    g = torch.Generator(device="cuda").manual_seed(rows + cols)
    packed = torch.empty(rows, cols // 2, dtype=torch.uint8, device="cuda")
    for r in range(0, rows, 65536):
        packed[r:r + 65536] = torch.randint(0, 256, (min(65536, rows - r), cols // 2), generator=g, device="cuda",
                                            dtype=torch.int32).to(torch.uint8)
    scale = torch.randint(117, 128, (rows, cols // 32), generator=g, device="cuda", dtype=torch.int32).to(torch.uint8).view(E8M0)
    packed = packed.view(torch.int8)
    per = rows // 256
    slabs = (0, 101 * per - 128, 101 * per, rows - 128)

    def slab(r):
        return packed[r:r + 128].contiguous(), scale[r:r + 128].contiguous()

    say("whole-layer FP4 -> FP8 fused", rows, cols)
    q, s = G.fp4_to_fp8_blockwise(packed, scale)
    for r in slabs:
        qs, s1 = G.fp4_to_fp8_blockwise(*slab(r))
        assert _same(q[r:r + 128], qs) and _same(s[r // 128:r // 128 + 1], s1), r
    ps, ss = slab(slabs[2])
    rq, rs = T.quant_block_fp32_scale(T.cast_e2m1fn_to_bf16(ps.cpu(), ss.cpu()), (128, 128))
    assert _same(q[slabs[2]:slabs[2] + 128].cpu(), rq) and _same(s[slabs[2] // 128:slabs[2] // 128 + 1].cpu(), rs)
    del q, s
    say("whole-layer FP4 -> FP8 re-basing", rows, cols)
    q, s = G.cast_e2m1fn_to_e4m3fn(packed, scale)
    for r in slabs:
        qs, s1 = G.cast_e2m1fn_to_e4m3fn(*slab(r))
        assert _same(q[r:r + 128], qs) and _same(s[r // 128:r // 128 + 1], s1), r
    del q, s
    say("whole-layer FP4 -> bf16", rows, cols)
    w = G.cast_e2m1fn_to_bf16(packed, scale)
    for r in slabs:
        assert _same(w[r:r + 128], G.cast_e2m1fn_to_bf16(*slab(r))), r
    assert _same(w[slabs[2]:slabs[2] + 128].cpu(), T.cast_e2m1fn_to_bf16(ps.cpu(), ss.cpu()))
