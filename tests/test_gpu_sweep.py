"""Seeded sweeps around the dispatch boundaries of the GEMM entry points: row counts either side of the decode kernels'
limits (8 / 9, 16 / 17, 64 / 65), weight-row counts either side of the tile-width choices (multiples of 224, 256 and
288, a ragged last tile), K from one block to 7168, both scale types and both output types -- every shape against the
fp32 dequantise-then-matmul reference to the path's tolerance.  The grouped sweeps draw the rows per expert from the
values that change a tile class or a padding rule (0, 1, 128, 129, 256, 257, 512, 513) and from ranges."""
import random

import pytest
import torch

from oracle import torch_ref as T
from tests import test_gpu_gemm as t

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gcore_lowp
    return gcore_lowp


ROWS = [1, 2, 7, 8, 9, 15, 16, 17, 31, 32, 33, 47, 48, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300, 511, 512, 513, 777, 1024,
        1500, 2048, 2560, 4096]
WEIGHT_ROWS = [128, 256, 384, 512, 896, 1024, 2048, 2688, 3072, 3584, 4096, 4224, 4352, 5120, 6144, 6272, 7168, 8192, 8320, 9216,
               12288, 16384, 18432, 18560, 20480]
DEPTHS = [128, 256, 384, 512, 640, 896, 1024, 1536, 2048, 2560, 3584, 4096, 7168]


@pytest.mark.parametrize("seed", [11, 12])
def test_dense_gemm_shape_sweep(G, seed):
    rng = random.Random(seed)
    done = 0
    while done < 36:
        M, N, K = rng.choice(ROWS), rng.choice(WEIGHT_ROWS), rng.choice(DEPTHS)
        if M * N * K > 2 ** 35:
            continue
        pow2, wide = rng.random() < 0.5, rng.random() < 0.3
        t.say("dense sweep", seed, done, (M, N, K), "e8m0" if pow2 else "fp32", "f32 out" if wide else "bf16 out")
        xq, xs, wq, ws = t.quantized_problem(M, N, K, seed=seed * 1000 + done, pow2=pow2)
        out = G.gemm_fp8_block_scaling_impl(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(),
                                            out_dtype=torch.float32 if wide else torch.bfloat16)
        t.check(out, t.ref_gemm(xq, xs, wq, ws), f"dense sweep {(M, N, K)}")
        done += 1


def _splits(rng, E, hi):
    return [rng.choice([0, 1, 127, 128, 129, 255, 256, 257, 511, 512, 513, rng.randint(1, hi), rng.randint(1, hi)]) for _ in range(E)]


def test_grouped_gemm_shape_sweep(G):
    rng = random.Random(21)
    done = 0
    while done < 24:
        E = rng.choice([1, 2, 3, 5, 8, 16, 33])
        N, K = rng.choice([128, 256, 384, 512, 768, 1024, 2048]), rng.choice([128, 256, 512, 640, 1024, 2048, 2560])
        m_splits = _splits(rng, E, rng.choice([40, 400, 1200]))
        M = sum(m_splits)
        if M == 0 or M * N * K > 2 ** 32:
            continue
        t.say("grouped sweep", done, E, N, K, m_splits)
        xq, xs, wq, ws = t._grouped_problem(E, N, K, m_splits, seed=2100 + done)
        offs = torch.zeros(E + 1, dtype=torch.int32)
        offs[1:] = torch.cumsum(torch.tensor(m_splits), 0)
        out = G.grouped_gemm_fp8(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), offs.cuda())
        t.check(out, T.grouped_gemm_fp8_ref(xq, xs, wq, ws, m_splits), f"grouped sweep {done}")
        wide = G.grouped_gemm_fp8(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), offs.cuda(), out_dtype=torch.float32)
        assert torch.equal(out, wide.to(torch.bfloat16))
        done += 1


def test_grouped_linear_backward_sweep(G):
    """Forward, data gradient and weight gradient of every expert within 6 % (norm) of bf16 matmuls on that expert's rows:
    an expert that reads another's rows, blocks or padding is off by the order of 100 %."""
    rng = random.Random(31)
    rel = lambda a, b: ((a.float() - b.float()).norm() / b.float().norm().clamp_min(1e-30)).item()
    for case in range(12):
        E = rng.choice([1, 3, 4, 7, 12, 20])
        h_in, h_out = rng.choice([(256, 512), (512, 256), (128, 384), (1024, 256)])
        m_splits = _splits(rng, E, rng.choice([300, 900]))
        if sum(m_splits) == 0:
            continue
        t.say("backward sweep", case, E, h_in, h_out, m_splits)
        torch.manual_seed(3100 + case)
        x = torch.randn(sum(m_splits), h_in, device="cuda", dtype=torch.bfloat16, requires_grad=True)
        w = torch.randn(E, h_out, h_in, device="cuda", dtype=torch.bfloat16, requires_grad=True)
        g = torch.randn(sum(m_splits), h_out, device="cuda", dtype=torch.bfloat16)
        out = G.MyTeGroupedLinearFp8(E)(x, w, m_splits)
        out.backward(g)
        off = 0
        for e, m in enumerate(m_splits):
            xe, ge, we = x.detach()[off:off + m].float(), g[off:off + m].float(), w.detach()[e].float()
            if m == 0:
                assert not w.grad[e].any(), (case, e)
            else:
                assert rel(out[off:off + m], xe @ we.T) < 0.06, (case, e, m, "forward")
                assert rel(x.grad[off:off + m], ge @ we) < 0.06, (case, e, m, "dgrad")
                assert rel(w.grad[e], ge.T @ xe) < 0.06, (case, e, m, "wgrad")
            off += m


def _bits_equal(a, b):
    a, b = a.detach().cpu().contiguous(), b.detach().cpu().contiguous()
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a.view(torch.uint8), b.view(torch.uint8))


def test_quantise_dequantise_shape_sweep(G):
    """The tile and the row-group quantisers and the dequantiser, bit for bit against the oracle, on shapes that end
    inside a launch's unit of work: row counts that are not multiples of the 16 groups a pass takes, tile counts that
    do not fill the XCDs evenly, one tile, one row."""
    from tests import _inputs as I
    rng = random.Random(41)
    for case in range(30):
        tiles = rng.random() < 0.5
        if tiles:
            rows, cols = 128 * rng.choice([1, 2, 3, 5, 7, 8, 9, 17, 31]), 128 * rng.choice([1, 2, 3, 5, 8, 11, 16, 29])
            block = (128, 128)
        else:
            rows, cols = rng.choice([1, 2, 3, 15, 16, 17, 33, 63, 64, 65, 100, 257, 1000, 2049]), 128 * rng.choice([1, 2, 3, 7, 8, 25, 56])
            block = (1, 128)
        dt = torch.float32 if rng.random() < 0.3 else torch.bfloat16
        x = (I.weight_like if tiles else I.act_like)(rows, cols, 4100 + case, dtype=dt)
        t.say("quantise sweep", case, (rows, cols), block, dt)
        rq, rs = T.quant_fp8_e4m3_scale_e8m0(x, block)
        hq, hs = G.quant_fp8_e4m3_scale_e8m0(x.cuda(), block)
        assert _bits_equal(hs, rs) and _bits_equal(hq, rq), ("pow2", case)
        rq2, rs2 = T.quant_block_fp32_scale(x, block, amax_floor=1e-12)
        hq2, hs2 = (G.quant_2d(x.cuda(), block) if tiles else G.quant_1d(x.cuda(), 128))
        assert _bits_equal(hs2, rs2) and _bits_equal(hq2, rq2), ("divide", case)
        want = T.dequant_fp4_e2m1_fp8_scale_e8m0_packed(rq, rs)
        got = G.dequant_fp4_e2m1_fp8_scale_e8m0_packed(hq, hs)
        assert _bits_equal(got, want), ("dequantise", case)


def test_fp4_conversion_shape_sweep(G):
    """FP4 -> bf16, FP4 -> FP8 re-based and FP4 -> FP8 fused (128 x 128, amax / 448) on expert shapes that end inside a
    super tile of 128 x 256 and on single tiles, bit for bit against the oracle."""
    from tests import _inputs as I
    rng = random.Random(51)
    for case in range(16):
        rows, cols = 128 * rng.choice([1, 2, 3, 5, 8, 13]), 128 * rng.choice([1, 2, 3, 5, 7, 12])
        lo = rng.choice([2, 60, 110, 117])
        p, s = I.fp4_expert(rows, cols, 5100 + case, lo, lo + rng.choice([4, 10, 60]))
        t.say("fp4 sweep", case, (rows, cols), lo)
        w = T.cast_e2m1fn_to_bf16(p, s)
        assert _bits_equal(G.cast_e2m1fn_to_bf16(p.cuda(), s.cuda()), w)
        rq, rs = T.cast_e2m1fn_to_e4m3fn(p, s)
        hq, hs = G.cast_e2m1fn_to_e4m3fn(p.cuda(), s.cuda())
        assert _bits_equal(hs, rs) and _bits_equal(hq, rq)
        rq, rs = T.quant_block_fp32_scale(w, (128, 128))
        hq, hs = G.fp4_to_fp8_blockwise(p.cuda(), s.cuda())
        assert _bits_equal(hs, rs)
        a, b = hq.cpu().view(torch.uint8), rq.view(torch.uint8)
        nan = (b & 0x7F) == 0x7F
        assert torch.equal(a[~nan], b[~nan]) and bool(((a[nan] & 0x7F) == 0x7F).all())


def test_fp4_quantiser_and_qat_shape_sweep(G, corc):
    """The FP4 quantiser (1 x 32 blocks), the fake-quantiser and the fused FP4 -> FP8 QAT conversion on shapes with row
    counts and widths that end inside a launch's unit of work: the quantiser against both oracles through its own test's
    comparison, the other two bit for bit against the eager restatement."""
    from gcore_lowp import eager_quant_kernels as Q
    from gcore_lowp.fused_quant_kernels import fp4_qat_then_to_fp8
    from gcore_lowp.qat import fp4_simulate_qat
    from tests import test_gpu_fp4_quant as q4
    Q._corc = corc
    rng = random.Random(61)
    for case in range(14):
        rows, cols = rng.choice([1, 2, 3, 31, 33, 100, 255, 257, 1000, 2049]), 32 * rng.choice([1, 2, 3, 5, 8, 33, 100, 224])
        t.say("fp4 quantiser sweep", case, (rows, cols))
        g = torch.Generator().manual_seed(6100 + case)
        w = torch.randn(rows, cols, generator=g) * torch.logspace(-3, 2, cols // 32).repeat_interleave(32)
        w[0, :32] = 0
        q4.check(Q, w.to(torch.bfloat16 if case % 2 else torch.float32))
        x = w.bfloat16()
        assert torch.equal(fp4_simulate_qat(x.cuda()).cpu().view(torch.int16), T.fp4_simulate(x).view(torch.int16)), case
    for case in range(6):
        m, n = 128 * rng.choice([1, 2, 3, 5, 9]), 128 * rng.choice([1, 2, 3, 7, 12])
        t.say("fp4 qat -> fp8 sweep", case, (m, n))
        g = torch.Generator().manual_seed(6200 + case)
        w = torch.randn(m, n, generator=g)
        w[:, 32:64] *= 2.0 ** -4
        w[:16, :32] = 0
        q, s = fp4_qat_then_to_fp8(w.cuda())
        wq, ws = T.fp4_qat_then_to_fp8(w)
        assert _bits_equal(s, ws) and _bits_equal(q, wq), case


def test_unscaled_nt_gemm_shape_sweep(G):
    """gemm_impl either side of the point where it changes kernels (512 tiles of 128 x 128), with ragged last row and
    column tiles, K in and out of whole groups of 512 bytes, fp8 and bf16 operands, every output type."""
    rng = random.Random(61)
    shapes = [(2048, 4096), (2049, 4096), (2304, 4096), (2300, 4112), (1153, 8192), (4096, 2064), (640, 16400), (8200, 1040),
              (3000, 3000 // 16 * 16), (5000, 1776), (16384, 528), (1024, 8208)]
    for case, (M, N) in enumerate(shapes):
        K = rng.choice([256, 512, 768, 1024, 1536])
        kind = "fp8" if case % 2 == 0 else "bf16"
        t.say("nt sweep", case, (M, N, K), kind)
        g = torch.Generator().manual_seed(6100 + case)
        dt = torch.float8_e4m3fn if kind == "fp8" else torch.bfloat16
        a, b = torch.randn(M, K, generator=g).to(dt).cuda(), torch.randn(N, K, generator=g).to(dt).cuda()
        ref = a.float() @ b.float().T
        for out_dtype in ([torch.float8_e4m3fn, torch.bfloat16] if kind == "fp8" else [torch.bfloat16, torch.float32]):
            c = G.gemm_impl(a, b, 128, 128, 64, dtype=dt, out_dtype=out_dtype)
            assert c.dtype == out_dtype and tuple(c.shape) == (M, N)
            if out_dtype == torch.float8_e4m3fn:
                want = ref.clamp(-448, 448).to(out_dtype)
                ci, wi = c.view(torch.uint8).int(), want.view(torch.uint8).int()
                assert ((ci - wi).abs() <= 1).float().mean() > 0.9999, (M, N, K)
            else:
                err = ((c.float() - ref).abs().max() / ref.abs().max()).item()
                assert err < (1e-2 if out_dtype == torch.bfloat16 else 1e-5), (M, N, K, err)
