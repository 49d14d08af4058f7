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
