"""Pins the FP4 quantiser of the oracle (CPU only): the reference's known answers
(tests/test_gfused/test_eager_quantize_kernels.py:54-150), hand-made tie vectors, the closed form of the
scale exponent, and C == torch restatement."""
import math

import numpy as np
import torch

from oracle import torch_ref as T

E8M0 = torch.float8_e8m0fnu


def _both(corc, x, block=(1, 32)):
    """Codes and scale bytes from the torch restatement, checked equal to the C restatement."""
    p, s = T.quant_fp4_e2m1_scale_e8m0_packed(x, block)
    pc, sc, nan = corc.quant_fp4_block(x.float().numpy(), block[0], block[1])
    assert nan == 0
    assert np.array_equal(p.view(torch.uint8).numpy(), pc)
    assert np.array_equal(s.view(torch.uint8).numpy(), sc)
    return p.view(torch.uint8), s.view(torch.uint8)


def _codes(packed):
    lo, hi = packed & 0xF, packed >> 4
    return torch.stack([lo, hi], dim=-1).flatten(-2)


def test_packing_layout_known_answer(corc):
    """:135-150: x[0,0] = 1, x[0,1] = -1 -> scale 2^-2, first byte 0xE6."""
    x = torch.zeros(1, 32)
    x[0, 0], x[0, 1] = 1.0, -1.0
    p, s = _both(corc, x)
    assert p[0, 0].item() == 0xE6 and s.item() == 125
    assert int(p[0, 1:].sum()) == 0


def test_zero_block_and_signed_extremes(corc):
    """:112-133: an all-zero block has scale 1 and codes 0; +-6, 0, -3 at scale 1; -0.0 keeps its sign."""
    p, s = _both(corc, torch.zeros(2, 64))
    assert int(p.sum()) == 0 and s.flatten().tolist() == [127] * 4
    x = torch.tensor([[6.0, -6.0, 0.0, -3.0] * 8])
    p, s = _both(corc, x)
    assert _codes(p)[0, :4].tolist() == [7, 15, 0, 13] and s.item() == 127
    x = torch.tensor([[6.0, -0.0] + [0.0] * 30])
    p, s = _both(corc, x)
    assert _codes(p)[0, :3].tolist() == [7, 8, 0]


def test_ties_go_to_the_smaller_magnitude(corc):
    """bucketize(right=False), eager_quant_kernels.py:116-121: a value on a midpoint takes the lower code,
    the next float above it the upper one -- at every scale."""
    mids = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0]
    for e in (0, -9, 11):
        sc = 2.0 ** e
        vals = [6.0 * sc]
        want = [7]
        for k, m in enumerate(mids):
            up = float(np.nextafter(np.float32(m * sc), np.float32(np.inf)))
            dn = float(np.nextafter(np.float32(m * sc), np.float32(0)))
            vals += [m * sc, -m * sc, up, -up, dn]
            want += [k, 8 + k, k + 1, 8 + k + 1, k]
        vals += [0.0] * (64 - len(vals))
        want += [0] * (64 - len(want))
        x = torch.tensor([vals], dtype=torch.float32)
        x[0, 32] = 6.0 * sc                      # second block: same scale
        want[32] = 7
        p, s = _both(corc, x)
        assert s.flatten().tolist() == [127 + e] * 2
        assert _codes(p)[0].tolist() == want, e


def test_grid_round_trip(corc):
    """:54-110: codes with +6 planted per block and scales 2^[-10, 10) survive dequantise -> quantise."""
    g = torch.Generator().manual_seed(0)
    m, n = 64, 512
    codes = torch.randint(0, 16, (m, n), generator=g, dtype=torch.uint8)
    codes[:, 0::32] = 7
    exp = torch.randint(-10, 10, (m, n // 32), generator=g)
    scale = torch.pow(2.0, exp.float()).to(E8M0)
    pair = codes.reshape(m, n // 2, 2)
    packed = (pair[..., 0] | (pair[..., 1] << 4)).view(torch.int8)
    y = T.dequant_fp4_e2m1_fp8_scale_e8m0_packed(packed, scale).float()
    p, s = _both(corc, y)
    assert torch.equal(p, packed.view(torch.uint8))
    assert torch.equal(s, scale.view(torch.uint8))


def test_scale_exponent_closed_form(corc):
    """2^e is the smallest power of two with 6 * 2^e >= amax: equals ceil(log2(fl(amax / 6))) of both log2
    flavours on every bf16 amax, and of the exact flavour on the floats around every 6 * 2^k."""
    def closed(a):
        if a == 0:
            return 0
        a = max(a, float(np.finfo(np.float32).tiny))
        m, ex = math.frexp(a)                 # a = m * 2^ex, m in [0.5, 1)
        return ex - 3 + (1 if m > 0.75 else 0)

    bits = np.arange(0x0001, 0x7F80, dtype=np.uint32) << 16           # every positive finite bf16
    amax = bits.view(np.float32)
    for kind in (0, 1):
        for chunk in np.array_split(amax, 64):
            x = np.zeros((len(chunk), 32), np.float32)
            x[:, 0] = chunk
            _, sb, _ = corc.quant_fp4_block(x, 1, 32, kind)
            want = np.array([max(closed(float(a)) + 127, 0) for a in chunk])
            assert np.array_equal(sb[:, 0].astype(np.int64), want), kind
    edge = []
    for k in range(-120, 120):
        c = np.float32(6.0 * 2.0 ** k)
        edge += [c, np.nextafter(c, np.float32(np.inf)), np.nextafter(c, np.float32(0))]
    edge = np.array(edge, np.float32)
    x = np.zeros((len(edge), 32), np.float32)
    x[:, 0] = edge
    _, sb, _ = corc.quant_fp4_block(x, 1, 32, 1)
    want = np.array([closed(float(a)) + 127 for a in edge])
    assert np.array_equal(sb[:, 0].astype(np.int64), want)


def test_c_equals_torch_on_weights(corc):
    g = torch.Generator().manual_seed(5)
    w = torch.randn(128, 256, generator=g) * 0.02
    w[:4, :32] = 0
    w[:, 32:64] *= 2.0 ** -4
    w[:, 64:96] *= 2.0 ** 4
    _both(corc, w)
    _both(corc, w.to(torch.bfloat16).float())
    _both(corc, w, (2, 64))
    _both(corc, w, (128, 128))
    q, s = T.quant_block_fp32_scale(w, (128, 128))
    p, sb = T.sgl_expert_to_official(q, s)
    assert p.dtype == torch.int8 and tuple(p.shape) == (128, 128) and sb.dtype == E8M0 and tuple(sb.shape) == (128, 8)
