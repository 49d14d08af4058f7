"""GPU parity of the fused QAT kernels (fp4_qat_then_to_fp8, fp_qat_128x128, act_quant) against the CPU oracle,
byte for byte, on the shapes and patterns of the reference's own tests."""
import numpy as np
import pytest
import torch

from oracle import torch_ref as T

pytestmark = pytest.mark.gpu

E4M3, E8M0 = torch.float8_e4m3fn, torch.float8_e8m0fnu


def say(*a):
    print("[case]", *a, flush=True)


def u8(t):
    return t.detach().cpu().contiguous().view(torch.uint8)


@pytest.mark.parametrize(("m", "n"), [(128, 128), (256, 512), (384, 640), (2048, 4096)])
def test_fp4_qat_then_to_fp8(m, n):
    """tests/test_gpatch_v4/test_quantize_kernels.py:155-186"""
    from gcore_lowp.fused_quant_kernels import fp4_qat_then_to_fp8
    say("fp4_qat_then_to_fp8", m, n)
    torch.manual_seed(7)
    w = torch.randn(m, n)
    w[:16, :32] = 0
    w[:, 32:64] *= 2.0 ** -4
    w[:, 64:96] *= 2.0 ** 4
    w[5, 100] = -0.0
    w[7, :32] = torch.tensor([6.0, 0.75, 1.75, 3.5, -0.75, -1.75, -3.5, 0.25, 1.25, 2.5, 5.0] + [0.0] * 21)
    q, s = fp4_qat_then_to_fp8(w.cuda())
    assert q.dtype == E4M3 and s.dtype == E8M0 and tuple(s.shape) == (m // 128, n // 128)
    wq, ws = T.fp4_qat_then_to_fp8(w)
    assert torch.equal(u8(s), u8(ws))
    bad = (u8(q) != u8(wq)).nonzero()
    assert bad.numel() == 0, (bad[:4].tolist(), int(bad.shape[0]))


def test_fp4_qat_tiny_and_errors():
    from gcore_lowp.fused_quant_kernels import fp4_qat_then_to_fp8
    say("fp4_qat tiny magnitudes")
    g = torch.Generator().manual_seed(1)
    w = torch.randn(128, 256, generator=g)
    w[:, :32] *= 1e-37            # group scales at and below 2^-120: software rounding branch
    w[:, 32:64] *= 1e-39
    w[:64, 128:] *= 1e-38         # a tile whose scale is clamped at 2^-126
    w[64:, 128:] *= 1e-40
    q, s = fp4_qat_then_to_fp8(w.cuda())
    wq, ws = T.fp4_qat_then_to_fp8(w)
    assert torch.equal(u8(s), u8(ws)) and torch.equal(u8(q), u8(wq))
    with pytest.raises(TypeError):
        fp4_qat_then_to_fp8(w.cuda().bfloat16())
    with pytest.raises(ValueError):
        fp4_qat_then_to_fp8(w.cuda()[:, :100])
    with pytest.raises(ValueError):
        fp4_qat_then_to_fp8(w)                                   # not on the GPU


@pytest.mark.parametrize(("m", "n", "seed"), [(128, 128, 0), (256, 384, 1), (128, 512, 2), (512, 128, 3), (512, 512, 4),
                                              (4096, 4096, 5)])
def test_fp_qat_128x128(m, n, seed):
    """tests/test_gfused/test_fp_qat_128x128.py:52-65"""
    from gcore_lowp.fused_quant_kernels import fp_qat_128x128
    say("fp_qat_128x128", m, n)
    torch.manual_seed(seed)
    w = torch.randn(m, n).to(torch.bfloat16)
    out = fp_qat_128x128(w.cuda())
    assert out.dtype == torch.bfloat16 and out.shape == w.shape
    assert torch.equal(out.cpu().view(torch.int16), T.fp_qat_128x128(w).view(torch.int16))


def test_fp_qat_128x128_tiles_and_edges():
    """:67-120: independent scale per tile, zero tile, a single outlier in each 128 x 32 stripe"""
    from gcore_lowp.fused_quant_kernels import fp_qat_128x128
    say("fp_qat_128x128 patterns")
    pat = torch.linspace(-1.0, 1.0, 128 * 128).reshape(128, 128)
    w = torch.empty(256, 256, dtype=torch.bfloat16)
    w[:128, :128] = pat * 2.0 ** -8
    w[:128, 128:] = pat * 2.0 ** -2
    w[128:, :128] = 0
    w[128:, 128:] = pat * 2.0 ** 5
    assert torch.equal(fp_qat_128x128(w.cuda()).cpu().view(torch.int16), T.fp_qat_128x128(w).view(torch.int16))
    for stripe in range(4):
        w = torch.full((128, 128), 0.01, dtype=torch.bfloat16)
        w[77, stripe * 32 + 5] = -300.0
        assert torch.equal(fp_qat_128x128(w.cuda()).cpu().view(torch.int16), T.fp_qat_128x128(w).view(torch.int16))
    w = (torch.randn(128, 256) * 1e-33).to(torch.bfloat16)        # below the 1e-30 floor
    w[:, 128:] = (torch.randn(128, 128).clamp(-3, 3) * 1e37).to(torch.bfloat16)      # near the top of the range
    assert torch.equal(fp_qat_128x128(w.cuda()).cpu().view(torch.int16), T.fp_qat_128x128(w).view(torch.int16))
    with pytest.raises(TypeError):
        fp_qat_128x128(w.cuda().float())


@pytest.mark.parametrize("fmt", [None, "ue8m0"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_act_quant(fmt, dtype):
    from gcore_lowp.qat import act_quant
    say("act_quant", fmt, dtype)
    torch.manual_seed(3)
    x = (torch.randn(4, 96, 512) * 3).to(dtype)
    x[0, 0, :128] = 0
    x[0, 1, :128] = 448.0
    x[0, 2, :128] *= 1e-6
    y, s = act_quant(x.cuda(), 128, fmt)
    wy, ws = T.act_quant(x, 128, fmt)
    assert y.dtype == E4M3 and s.dtype == torch.float32 and tuple(s.shape) == (4, 96, 4)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), ws.numpy().view(np.uint32))
    assert torch.equal(u8(y), u8(wy))
    y, s = act_quant(x.cuda()[..., :256].contiguous(), 64, fmt)          # another group size
    wy, ws = T.act_quant(x[..., :256].contiguous(), 64, fmt)
    assert torch.equal(u8(y), u8(wy)) and np.array_equal(s.cpu().numpy().view(np.uint32), ws.numpy().view(np.uint32))
    with pytest.raises(NotImplementedError):
        act_quant(x.cuda(), 128, fmt, inplace=True)
