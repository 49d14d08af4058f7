"""GPU parity of the FP4 quantiser (lp_quant_fp4_block) against the CPU oracles, bit for bit.

Every case prints its name before touching the GPU so that a fault names its case.
"""
import numpy as np
import pytest
import torch

from oracle import torch_ref as T

pytestmark = pytest.mark.gpu

E8M0 = torch.float8_e8m0fnu


def say(*a):
    print("[case]", *a, flush=True)


def u8(t):
    return t.detach().cpu().contiguous().view(torch.uint8)


@pytest.fixture(scope="module")
def Q(corc):
    from gcore_lowp import eager_quant_kernels
    eager_quant_kernels._corc = corc          # the C oracle rides along for check()
    return eager_quant_kernels


def check(Q, x, block=(1, 32)):
    """Byte equality with the C oracle in its exact-log2 flavour, and with the eager-torch restatement except
    on blocks whose amax / 6 lies within 4 ulps above a power of two: there ceil(log2(.)) depends on how the
    device's log2 rounds (the reference's result on such a block is not pinned by anything)."""
    p, s = Q.quant_fp4_e2m1_scale_e8m0_packed(x.cuda(), block)
    assert p.dtype == torch.int8 and s.dtype == E8M0 and p.is_cuda
    xf = x.float()
    m, n = xf.shape[-2:]
    pc, sc, _ = Q._corc.quant_fp4_block(xf.reshape(-1, n).numpy(), block[0], block[1], 1)
    assert np.array_equal(u8(s).reshape(sc.shape).numpy(), sc), "scales vs C oracle"
    assert np.array_equal(u8(p).reshape(pc.shape).numpy(), pc), "codes vs C oracle"
    wp, ws = T.quant_fp4_e2m1_scale_e8m0_packed(xf, block)
    assert tuple(p.shape) == tuple(wp.shape) and tuple(s.shape) == tuple(ws.shape)
    amax = T._tile_amax(T._tiles(xf, *block))
    r = (amax.clamp(min=torch.finfo(torch.float32).tiny) / 6.0).view(torch.int32)
    corner = ((r & 0x7FFFFF) > 0) & ((r & 0x7FFFFF) <= 4)
    assert int(corner.sum()) <= 4
    same = u8(s) == u8(ws)
    assert bool((same | corner).all()), "scales vs torch restatement"
    blk_ok = T._bcast(same).expand(T._tiles(xf, *block).shape).reshape(xf.shape)
    codes_ok = (u8(p) == u8(wp)).repeat_interleave(2, dim=-1)
    assert bool((codes_ok | ~blk_ok).all()), "codes vs torch restatement"
    return p, s


def test_hardware_encode_matches_software():
    """v_cvt_scalef32_pk_fp4_f32 plus the tie adjustment == round-to-nearest with ties to the smaller
    magnitude, over every finite fp32 at three scales."""
    from gcore_lowp import _probe_abi as probe
    say("selftest 4")
    assert probe.selftest(4) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("shape", [(256, 512), (3, 64, 96), (1, 32), (2048, 7168)], ids=str)
def test_weights(Q, dtype, shape):
    say("fp4 quant weights", dtype, shape)
    g = torch.Generator().manual_seed(sum(shape))
    w = torch.randn(*shape, generator=g) * 0.02
    if w.shape[-1] >= 96:
        w[..., :1, :32] = 0
        w[..., 32:64] *= 2.0 ** -4
        w[..., 64:96] *= 2.0 ** 4
    check(Q, w.to(dtype))


def test_ties_zeros_and_sign(Q):
    say("fp4 quant ties")
    mids = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0]
    rows = []
    for e in (0, -9, 11, -100, 100):
        sc = 2.0 ** e
        vals = [6.0 * sc]
        for m in mids:
            up = float(np.nextafter(np.float32(m * sc), np.float32(np.inf)))
            dn = float(np.nextafter(np.float32(m * sc), np.float32(0)))
            vals += [m * sc, -m * sc, up, -up, dn, -dn]
        vals += [0.0, -0.0] * ((64 - len(vals)) // 2)
        vals = vals[:64] + [0.0] * (64 - len(vals[:64]))
        vals[32] = -6.0 * sc
        rows.append(vals)
    rows.append([0.0] * 64)
    rows.append([-0.0] * 64)
    x = torch.tensor(rows, dtype=torch.float32)
    p, s = check(Q, x)
    assert int(u8(p)[-2].sum()) == 0 and u8(s)[-2].tolist() == [127, 127]
    assert u8(p)[-1].tolist() == [0x88] * 32


def test_extreme_magnitudes(Q):
    """blocks whose scale exponent leaves the fast path: subnormal and near-FLT_MIN amax, near-FLT_MAX amax"""
    say("fp4 quant extremes")
    g = torch.Generator().manual_seed(3)
    base = torch.randn(8, 64, generator=g)
    scales = torch.tensor([1e-45, 1e-40, 1.2e-38, 3e-38, 1e-36, 1e30, 1e37, 5e37]).view(8, 1)
    x = base * scales
    x[:, 0] = scales[:, 0] * 3.0
    check(Q, x)


@pytest.mark.parametrize("block", [(2, 64), (128, 128), (1, 16), (4, 2)], ids=str)
def test_other_block_shapes(Q, block):
    say("fp4 quant generic", block)
    g = torch.Generator().manual_seed(11)
    w = torch.randn(256, 256, generator=g) * 0.3
    w[:4, :16] = 0
    check(Q, w.to(torch.bfloat16), block)
    check(Q, w, block)


def test_grid_round_trip_expert_size(Q):
    """tests/test_gfused/test_eager_quantize_kernels.py:54-110 at its own size (2048 x 4096): codes with +6
    planted per block and scales 2^[-10, 10) come back byte for byte."""
    say("fp4 quant round trip")
    g = torch.Generator().manual_seed(0)
    m, n = 2048, 4096
    codes = torch.randint(0, 16, (m, n), generator=g, dtype=torch.uint8)
    codes[:, 0::32] = 7
    exp = torch.randint(-10, 10, (m, n // 32), generator=g)
    scale = torch.pow(2.0, exp.float()).to(E8M0)
    pair = codes.reshape(m, n // 2, 2)
    packed = (pair[..., 0] | (pair[..., 1] << 4)).view(torch.int8)
    y = Q.dequant_fp4_e2m1_fp8_scale_e8m0_packed(packed.cuda(), scale.cuda())
    p, s = Q.quant_fp4_e2m1_scale_e8m0_packed(y.float())
    assert torch.equal(u8(p), u8(packed)) and torch.equal(u8(s), u8(scale))
    p, s = Q.quant_fp4_e2m1_scale_e8m0_packed(y)                     # bf16 straight in
    assert torch.equal(u8(p), u8(packed)) and torch.equal(u8(s), u8(scale))


def test_errors_and_cpu_inputs(Q):
    say("fp4 quant errors")
    x = torch.randn(4, 64)
    p, s = Q.quant_fp4_e2m1_scale_e8m0_packed(x)                     # CPU in -> CPU out
    assert p.device.type == "cpu" and s.device.type == "cpu"
    wp, ws = T.quant_fp4_e2m1_scale_e8m0_packed(x)
    assert torch.equal(u8(p), u8(wp)) and torch.equal(u8(s), u8(ws))
    with pytest.raises(AssertionError):
        Q.quant_fp4_e2m1_scale_e8m0_packed(torch.randn(4, 48))       # not divisible by 32
    bad = x.clone()
    bad[1, 3] = float("nan")
    with pytest.raises(AssertionError):
        Q.quant_fp4_e2m1_scale_e8m0_packed(bad)


def test_sgl_expert_to_official(Q):
    """tools/dsv4_quant_and_dequant/kernels.py:136-140 and its inverse direction: FP4 -> FP8 rebase is lossless,
    so official -> sgl -> official returns the packed codes whenever every 1 x 32 block holds a +-6
    (and no -0.0)."""
    from gcore_lowp import dsv4_kernels as K
    say("sgl_expert_to_official")
    g = torch.Generator().manual_seed(2)
    w = (torch.randn(256, 512, generator=g) * 0.05).to(torch.bfloat16)
    q, s = T.quant_block_fp32_scale(w.float(), (128, 128))
    p, sb = K.sgl_expert_to_official(q.cuda(), s.cuda())
    wp, wsb = T.sgl_expert_to_official(q, s)
    assert torch.equal(u8(p), u8(wp)) and torch.equal(u8(sb), u8(wsb))
    codes = torch.randint(0, 16, (256, 512), generator=g, dtype=torch.uint8)
    codes[codes == 8] = 0                     # -0.0 does not survive: the FP8 side's table has +0.0 at code 8
    codes[:, 0::32] = 7
    exp = torch.randint(-3, 3, (256, 16), generator=g)
    scale = torch.pow(2.0, exp.float()).to(E8M0)
    pair = codes.reshape(256, 256, 2)
    packed = (pair[..., 0] | (pair[..., 1] << 4)).view(torch.int8)
    q8, s8 = K.official_expert_to_sgl(packed.cuda(), scale.cuda())
    p2, s2 = K.sgl_expert_to_official(q8, s8)
    assert torch.equal(u8(p2), u8(packed)) and torch.equal(u8(s2), u8(scale))
