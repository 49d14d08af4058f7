"""Pins the block quantisers / dequantisers of the oracle (CPU only).

Two independent restatements (scalar C, eager torch) must agree byte for byte,
and both must reproduce the closed-form cases the reference's own CPU tests use
(tests/test_gfused/test_eager_quantize_kernels.py:154-215).
"""
import numpy as np
import pytest
import torch

from oracle import torch_ref as T
from tests import _inputs as I


def _u8(t):
    return t.contiguous().view(torch.uint8).numpy()


def _bits(t):
    return t.contiguous().view(torch.int32).numpy()


MODES = [
    ("pow2", dict(mode=0, amax_floor=0.0, zero_rule=0)),
    ("pow2_floor", dict(mode=0, amax_floor=1e-12, zero_rule=0)),
    ("div_floor", dict(mode=1, amax_floor=1e-12, zero_rule=0)),
    ("div_zero1", dict(mode=1, amax_floor=0.0, zero_rule=2)),
    ("mul", dict(mode=2, amax_floor=0.0, zero_rule=0)),
]


def _torch_quant(name, x, block):
    if name == "pow2":
        q, s = T.quant_fp8_e4m3_scale_e8m0(x, block)
        return q, s.float()
    if name == "pow2_floor":
        return T.quant_block_pow2_scale(x, block, amax_floor=1e-12)
    if name == "div_floor":
        return T.quant_block_fp32_scale(x, block, amax_floor=1e-12)
    if name == "div_zero1":
        return T.quant_block_fp32_scale(x, block, amax_floor=None, zero_scale_to_one=True)
    q, s = T.quantize_fp8_blockwise(x, block, scale_dtype=torch.float32)
    return q, s


@pytest.mark.parametrize("name,kw", MODES)
@pytest.mark.parametrize("block", [(128, 128), (1, 128), (2, 2), (1, 32)])
def test_c_and_torch_oracles_agree(corc, name, kw, block):
    xs = [I.weight_like(256, 384, 1), I.act_like(256, 384, 2), I.edge_tiles()[:, :1024],
          I.weight_like(256, 256, 3, dtype=torch.float32)]
    for x in xs:
        x = x.float()
        if name != "pow2" and block == (128, 128):
            x[:128, :128] = 0          # a zero tile
        q, s, sb, nan = corc.quant_fp8_block(x.numpy(), block[0], block[1], log2_kind=corc.LOG2_LIBM, **kw)
        tq, ts = _torch_quant(name, x, block)
        assert nan == 0
        assert np.array_equal(q, _u8(tq)), name
        assert np.array_equal(s.view(np.uint32), _bits(ts.float()).view(np.uint32)), name


def test_pow2_with_amax_floor_closed_forms(corc):
    """round_sf branch (tests/test_gfused/test_deepseek_tilekernels_quant.py:32-35): an all-zero block is floored to
    amax = 1e-12, so its scale is 2^ceil(log2(1e-12 / 448)) = 2^-48 (1e-12/448 = 2.23e-15 lies in (2^-49, 2^-48]),
    never 1; any block whose amax exceeds the floor gets exactly the scale of the unfloored power-of-two mode."""
    x = I.weight_like(256, 256, 21).float()
    x[:128, :128] = 0
    for orc in ("c", "torch"):
        if orc == "c":
            q, s, _, _ = corc.quant_fp8_block(x.numpy(), 128, 128, mode=0, amax_floor=1e-12)
            q0, s0, _, _ = corc.quant_fp8_block(x.numpy(), 128, 128, mode=0, amax_floor=0.0)
        else:
            tq, ts = T.quant_block_pow2_scale(x, (128, 128), amax_floor=1e-12)
            tq0, ts0 = T.quant_fp8_e4m3_scale_e8m0(x, (128, 128))
            q, s, q0, s0 = _u8(tq), ts.numpy().reshape(2, 2), _u8(tq0), ts0.float().numpy()
        s, s0 = np.asarray(s, dtype=np.float32).reshape(2, 2), np.asarray(s0, dtype=np.float32).reshape(2, 2)
        assert s[0, 0] == np.float32(2.0 ** -48) and s0[0, 0] == 1.0, orc
        assert (q[:128, :128] == 0).all()
        mask = np.ones((2, 2), bool); mask[0, 0] = False
        assert np.array_equal(s[mask], s0[mask]) and np.array_equal(q[128:], q0[128:]) and np.array_equal(q[:, 128:], q0[:, 128:])


def test_pow2_exact_equals_libm_on_bf16_grid(corc):
    """ceil(log2(amax/448)) from the bit pattern == via log2f == via torch.log2 for EVERY
    positive finite bf16 amax: on the bf16 grid the scale does not depend on the log2 flavour."""
    bits = np.arange(1, 0x7F80, dtype=np.uint32) << 16
    amax = bits.view(np.float32)
    r = np.maximum(amax, np.float32(1.17549435e-38)) / np.float32(448.0)
    exact = np.array([corc.pow2_exponent(float(v), corc.LOG2_EXACT) for v in r])
    libm = np.array([corc.pow2_exponent(float(v), corc.LOG2_LIBM) for v in r])
    tl = torch.ceil(torch.log2(torch.from_numpy(r))).numpy().astype(np.int64)
    assert np.array_equal(exact, libm)
    assert np.array_equal(exact, tl)


def test_pow2_libm_corner_documented(corc):
    """Raw fp32 amax one ulp above 448 * 2^-12: exact math says -11, correctly rounded fp32 log2 says -12.
    This is the only class of inputs where the exact flavour (used on the GPU) leaves the eager reference."""
    r = float(np.float32(2.0 ** -12) * (np.float32(1) + np.float32(2.0 ** -23)))
    assert corc.pow2_exponent(r, corc.LOG2_EXACT) == -11
    assert corc.pow2_exponent(r, corc.LOG2_LIBM) == -12


def test_grid_round_trip_fp8_pow2(corc):
    """Reference test_round_trip_block_128x128: codes x e8m0 scales with +-448 planted in every
    tile survive dequant -> quant byte for byte."""
    torch.manual_seed(1)
    M, N = 512, 1024
    u = torch.rand(M, N) * 896 - 448
    qx = u.to(torch.float8_e4m3fn).float()
    qx[:, 0::128] = 448.0
    qx = qx.to(torch.float8_e4m3fn)
    exp = torch.randint(-10, 10, (M // 128, N // 128)).float()
    sx = torch.pow(2.0, exp).to(torch.float8_e8m0fnu)
    y = T.dequant_fp4_e2m1_fp8_scale_e8m0_packed(qx, sx).float()
    q, s, sb, _ = corc.quant_fp8_block(y.numpy(), 128, 128, corc.POW2)
    assert np.array_equal(q, _u8(qx))
    assert np.array_equal(sb, _u8(sx))
    # and the C dequantiser gives back y
    f, b = corc.dequant_fp8_block(q, s)
    assert np.array_equal(f.view(np.uint32), _bits(y).view(np.uint32))
    assert np.array_equal(b, y.bfloat16().view(torch.int16).numpy().view(np.uint16))


def test_zero_tile(corc):
    x = np.zeros((128, 128), np.float32)
    q, s, sb, _ = corc.quant_fp8_block(x, 128, 128, corc.POW2)
    assert not q.any() and sb[0, 0] == 127 and s[0, 0] == 1.0          # scale pinned to 1.0
    q, s, _, _ = corc.quant_fp8_block(x, 128, 128, corc.DIV, amax_floor=1e-12)
    assert not q.any() and s[0, 0] == np.float32(1e-12) / np.float32(448)
    q, s, _, _ = corc.quant_fp8_block(x, 128, 128, corc.DIV, zero_rule=corc.ZERO_SCALE_TO_ONE)
    assert not q.any() and s[0, 0] == 1.0
    q, s, _, _ = corc.quant_fp8_block(x, 128, 128, corc.MUL)
    assert not q.any() and s[0, 0] == 1.0


def test_quant_invariants(corc):
    """|q| <= 448 and the largest magnitude of a non-zero tile is 448 (DIV, MUL) or within
    (224, 448] (POW2); dequant(quant(x)) is within half an e4m3 ulp of x."""
    x = I.weight_like(512, 512, 7).float().numpy()
    for mode in (corc.POW2, corc.DIV, corc.MUL):
        q, s, _, _ = corc.quant_fp8_block(x, 128, 128, mode)
        v = np.abs(corc.e4m3fn_to_f32(q)).reshape(4, 128, 4, 128).max(axis=(1, 3))
        if mode == corc.POW2:
            assert ((v > 224) & (v <= 448)).all()
        else:
            assert (v == 448).all()
        f, _ = corc.dequant_fp8_block(q, s)
        big = np.abs(x) > np.repeat(np.repeat(s, 128, 0), 128, 1) * 2.0 ** -6      # normal range
        rel = np.abs(f - x)[big] / np.abs(x)[big]
        assert rel.max() <= 2.0 ** -4 + 1e-6


def test_div_vs_mul_forms_differ_somewhere(corc):
    """x / (amax/448) and x * (448/amax) are different roundings: the two entry points must not be merged."""
    x = I.weight_like(1024, 1024, 11).float().numpy()
    qd, sd, _, _ = corc.quant_fp8_block(x, 128, 128, corc.DIV)
    qm, sm, _, _ = corc.quant_fp8_block(x, 128, 128, corc.MUL)
    assert (qd != qm).sum() + (sd.view(np.uint32) != sm.view(np.uint32)).sum() > 0


def test_dequant_fp8_matches_torch(corc):
    torch.manual_seed(3)
    q = torch.randint(0, 255, (256, 384), dtype=torch.uint8)
    q[(q & 0x7F) == 0x7F] = 0x3C                                          # no NaN codes
    for sdt in (torch.float32, torch.bfloat16, torch.float8_e8m0fnu):
        s = (torch.rand(2, 3) * 4 + 0.01).to(sdt)
        want = T.dequant_fp4_e2m1_fp8_scale_e8m0_packed(q.view(torch.float8_e4m3fn), s)
        f, b = corc.dequant_fp8_block(q.numpy(), s.float().numpy())
        if want.dtype == torch.float32:
            assert np.array_equal(f.view(np.uint32), _bits(want).view(np.uint32))
        else:
            assert np.array_equal(b, want.view(torch.int16).numpy().view(np.uint16))
    # the 2 x 2 grid case of the reference (test_convert_deepseek_v4_fp4_to_bf16.py:143-165)
    w = torch.ones(256, 256).to(torch.float8_e4m3fn)
    sf = torch.tensor([[1.0, 4.0], [2.0, 8.0]])
    out = T.cast_e4m3fn_to_bf16(w, sf.to(torch.float8_e8m0fnu)).float()
    f, _ = corc.dequant_fp8_block(_u8(w), sf.numpy())
    for i in range(2):
        for j in range(2):
            assert (out[i * 128:(i + 1) * 128, j * 128:(j + 1) * 128] == sf[i, j]).all()
            assert (f[i * 128:(i + 1) * 128, j * 128:(j + 1) * 128] == float(sf[i, j])).all()


def test_gemm_reference_indexing(corc):
    """Tiny brute force in double vs the torch fp32 restatement: pins the j//128 and kb indexing."""
    torch.manual_seed(5)
    M, N, K = 5, 256, 256
    aq = (torch.randn(M, K) * 50).to(torch.float8_e4m3fn)
    bq = (torch.randn(N, K) * 50).to(torch.float8_e4m3fn)
    a_s = torch.rand(M, K // 128) + 0.5
    b_s = torch.rand(N // 128, K // 128) + 0.5
    c = corc.gemm_fp8_block(_u8(aq), a_s.numpy(), _u8(bq), b_s.numpy())
    want = T.gemm_fp8_block_scaling_ref(aq, a_s, bq, b_s).numpy()
    assert np.allclose(c, want, rtol=1e-5, atol=1e-2)
    # swapping the scale axes must be visible
    wrong = T.gemm_fp8_block_scaling_ref(aq, a_s.flip(1), bq, b_s).numpy()
    assert not np.allclose(c, wrong, rtol=1e-3, atol=1e-2)


def test_c_oracle_mul_floor_equals_published_per_block_cast(corc):
    """The multiply form with a floored amax and a stored scale amax / 448 (the per_block_cast_to_fp8 that the
    weight-update path imports from SGLang): C restatement against the torch restatement, including a tile
    under the 1e-4 clamp and a zero tile.  Neither is pinned by a fixture: the library is not in the reference tree."""
    for x in (I.weight_like(256, 384, 1), I.act_like(256, 384, 2), I.weight_like(256, 256, 3, dtype=torch.float32)):
        x = x.float()
        x[:128, :128] = 0
        x[128:, :128] *= 1e-5
        q, s, _, nan = corc.quant_fp8_block(x.numpy(), 128, 128, corc.SCALE_MUL_FLOOR, amax_floor=1e-4)
        tq, ts = T.per_block_cast_to_fp8(x)
        assert nan == 0
        assert np.array_equal(q, _u8(tq))
        assert np.array_equal(s.view(np.uint32), _bits(ts).view(np.uint32))
        assert s[0, 0] == np.float32(1e-4) / np.float32(448.0)
