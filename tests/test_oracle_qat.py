"""Pins the fused-QAT restatements of the oracle (CPU only).  The reference defines these kernels as equal to
compositions of its eager functions (tests/test_gfused/test_fp_qat_128x128.py:30-49,
tests/test_gpatch_v4/test_quantize_kernels.py:61-108,155-186); the compositions are built here from the already
pinned eager restatements and compared byte for byte."""
import numpy as np
import torch

from oracle import torch_ref as T

E4M3, E8M0 = torch.float8_e4m3fn, torch.float8_e8m0fnu


def u8(t):
    return t.contiguous().view(torch.uint8)


def composite_fp4_qat(weight):
    """test_quantize_kernels.py:61-108: eager FP4 quantise, table with -0.0, rebase with the tile scale clamped at 2^-126"""
    packed, fs = T.quant_fp4_e2m1_scale_e8m0_packed(weight)
    m, n = weight.shape
    codes = packed.view(torch.uint8)
    vals = torch.stack([T.LUT_NEG_ZERO[(codes & 0xF).long()], T.LUT_NEG_ZERO[(codes >> 4).long()]], dim=-1).flatten(1)
    vals = vals.view(m // 128, 128, n // 128, 128).transpose(1, 2)
    local = fs.float().view(m // 128, 128, n // 128, -1).transpose(1, 2).flatten(2)
    outer = (local.amax(dim=-1, keepdim=True) / 64.0).clamp(min=2.0 ** -126)
    off = (local / outer).unflatten(-1, (128, -1)).repeat_interleave(32, dim=-1)
    q8 = (vals * off).transpose(1, 2).reshape(m, n)
    return q8.to(E4M3).contiguous(), outer.squeeze(-1).to(E8M0).contiguous()


def test_fp4_qat_equals_eager_composition():
    for m, n in ((128, 128), (256, 512), (384, 640)):
        torch.manual_seed(7)
        w = torch.randn(m, n)
        w[:16, :32] = 0
        w[:, 32:64] *= 2.0 ** -4
        w[:, 64:96] *= 2.0 ** 4
        w[5, 100] = -0.0
        q, s = T.fp4_qat_then_to_fp8(w)
        wq, ws = composite_fp4_qat(w)
        assert torch.equal(u8(s), u8(ws))
        assert torch.equal(u8(q), u8(wq))


def test_fp_qat_equals_eager_composition():
    def qdq(w):
        q, s = T.quant_fp8_e4m3_scale_e8m0(w.float(), (128, 128))
        return T.dequant_fp4_e2m1_fp8_scale_e8m0_packed(q, s)

    for m, n, seed in ((128, 128, 0), (256, 384, 1), (512, 128, 3)):
        torch.manual_seed(seed)
        w = torch.randn(m, n).to(torch.bfloat16)
        assert torch.equal(T.fp_qat_128x128(w).view(torch.int16), qdq(w).view(torch.int16))
    # test_fp_qat_128x128.py:67-86: an independent scale per tile, a zero tile
    pat = torch.linspace(-1.0, 1.0, 128 * 128).reshape(128, 128)
    w = torch.empty(256, 256, dtype=torch.bfloat16)
    w[:128, :128] = pat * 2.0 ** -8
    w[:128, 128:] = pat * 2.0 ** -2
    w[128:, :128] = 0
    w[128:, 128:] = pat * 2.0 ** 5
    assert torch.equal(T.fp_qat_128x128(w).view(torch.int16), qdq(w).view(torch.int16))


def test_act_quant_against_c_restatement_and_invariants(corc):
    torch.manual_seed(3)
    x = (torch.randn(64, 512) * 3).to(torch.bfloat16)
    x[0, :128] = 0                     # amax floor 1e-4 -> scale 1e-4 / 448
    x[1, :128] = 448.0
    for fmt, mode in ((None, 3), ("ue8m0", 4)):
        y, s = T.act_quant(x, 128, fmt)
        q, sc, _, _ = corc.quant_fp8_block(x.float().numpy(), 1, 128, mode, 1e-4)
        assert np.array_equal(u8(y).numpy(), q)
        assert np.array_equal(s.numpy().view(np.uint32), sc.view(np.uint32))
        assert y.dtype == E4M3 and s.dtype == torch.float32 and tuple(s.shape) == (64, 4)
        assert float(s[0, 0]) == (2.0 ** -22 if fmt else float(np.float32(1e-4) * np.float32(1 / 448.0)))
        if fmt:
            m, e = torch.frexp(s)
            assert bool((m == 0.5).all())              # powers of two
            assert bool((s * 448.0 >= x.float().reshape(64, 4, 128).abs().amax(-1).clamp(min=1e-4) * (1 - 1e-6)).all())
        back = y.float().reshape(64, 4, 128) * s.unsqueeze(-1)
        err = (back - x.float().reshape(64, 4, 128)).abs()
        assert bool((err <= s.unsqueeze(-1) * 16.0 + 1e-12).all())     # half an e4m3 step at the top binade


# tests/test_gfused/test_deepseek_v4_fp4_qat.py:37-62: the reference's own known-answer vector for the FP4
# fake-quantiser (amax 6 -> scale 1; the doubled row -> scale 2)
FP4_QAT_VALUES = [-5.5, -4.75, -3.75, -3.25, -2.75, -2.25, -1.85, -1.65, -1.35, -1.15, -0.9, -0.6, -0.4, -0.2, -0.1, 0.0,
                  0.1, 0.2, 0.4, 0.6, 0.9, 1.15, 1.35, 1.65, 1.85, 2.25, 2.75, 3.25, 3.75, 4.75, 5.25, 6.0]
FP4_QAT_EXPECTED = [-6.0, -4.0, -4.0, -3.0, -3.0, -2.0, -2.0, -1.5, -1.5, -1.0, -1.0, -0.5, -0.5, 0.0, 0.0, 0.0,
                    0.0, 0.0, 0.5, 0.5, 1.0, 1.0, 1.5, 1.5, 2.0, 2.0, 3.0, 3.0, 4.0, 4.0, 6.0, 6.0]
FP4_MIDPOINTS = (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0)


def fp4_known_answer():
    v = torch.tensor(FP4_QAT_VALUES, dtype=torch.bfloat16)
    e = torch.tensor(FP4_QAT_EXPECTED, dtype=torch.bfloat16)
    x = torch.stack([torch.cat([v, v]), torch.cat([v * 2, v * 2])]).unsqueeze(1).expand(-1, 3, -1).clone()
    want = torch.stack([torch.cat([e, e]), torch.cat([e * 2, e * 2])]).unsqueeze(1).expand(-1, 3, -1)
    return x, want


def sgl_export_effective(weight):
    """test_deepseek_v4_fp4_qat.py:29-35: what the sampler multiplies by after the export of an FP4-QAT expert"""
    q, s = T.fp4_qat_then_to_fp8(weight.bfloat16().float())
    return T.dequant_fp4_e2m1_fp8_scale_e8m0_packed(q, s).float()


def test_fp4_simulate_known_answer_and_export_agreement():
    x, want = fp4_known_answer()
    got = T.fp4_simulate(x)
    assert torch.equal(got.float().abs(), want.float().abs()) and torch.equal(torch.signbit(got) | (got == 0), torch.signbit(want) | (want == 0))
    # :97-133: the training forward equals the exported weight, on random data and on exact midpoints
    torch.manual_seed(29)
    w = torch.randn(256, 512).bfloat16().float()
    assert torch.equal(T.fp4_simulate(w.bfloat16()).float(), sgl_export_effective(w))
    row = torch.tensor(FP4_MIDPOINTS).repeat(16)
    w = row.expand(128, 128).clone()
    w[1::2] *= -1.0
    assert torch.equal(T.fp4_simulate(w.bfloat16()).float(), sgl_export_effective(w))
    # :136-160: still equal after a step that crosses the group-scale boundaries
    torch.manual_seed(31)
    w = T.fp4_simulate(torch.randn(256, 512).bfloat16()).float()
    signs = torch.randint(0, 2, w.shape).float()
    stepped = w + (signs * 2.0 - 1.0) * 1e-6
    assert torch.equal(T.fp4_simulate(stepped.bfloat16()).float(), sgl_export_effective(stepped))
    # scale bits: the product with fl32(1/6) gives the smallest 2^e with 6 * 2^e >= amax for every bf16 amax
    bits = torch.arange(0x01C0, 0x7F00, dtype=torch.int32)          # from the floor 6 * 2^-126 up
    amax = (bits << 16).view(torch.float32)
    e = T._log2_ceil_bits(amax * torch.tensor(1.0 / 6.0, dtype=torch.float32)).double()
    a = amax.double()
    assert bool((6.0 * torch.exp2(e) >= a).all()) and bool((6.0 * torch.exp2(e - 1) < a).all())


def test_fp8_simulate_and_inplace_branch():
    torch.manual_seed(5)
    x = (torch.randn(6, 5, 256) * torch.logspace(-6, 3, 6).view(6, 1, 1)).bfloat16()
    for bs in (64, 128):
        y = T.fp8_simulate(x, bs)
        # quantise (pinned act_quant) then multiply back: every product is exact and fits bf16
        q, s = T.act_quant(x, bs, "ue8m0")
        ref = (q.float().reshape(6, 5, 256 // bs, bs).double() * s.double().unsqueeze(-1)).reshape(x.shape)
        assert torch.equal(y.double(), ref)
        # with a power-of-two scale the in-place branch of the activation quantiser is the identity:
        # the quotient is exact, bf16 holds it, and the product restores x
        assert torch.equal(T.act_quant_inplace(x, bs, "ue8m0").view(torch.int16), x.view(torch.int16))
        # without rounding of the scale it is a genuine double rounding through bf16, within 2 ulp of x
        z = T.act_quant_inplace(x, bs, None)
        rel = ((z.double() - x.double()).abs() / x.double().abs().clamp(min=1e-30)).max()
        assert 0 < rel < 2.0 ** -7
