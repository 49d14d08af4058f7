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


# ---------------------------------------------------------------------------------------------------------------
# fake-quantisers of training with their straight-through wrappers (gpatch_v4/kernel/quantize/qat.py:226-431)

def bits16(t):
    return t.detach().cpu().contiguous().view(torch.int16)


def test_fp4_simulate_qat_known_answer_and_ste():
    """tests/test_gfused/test_deepseek_v4_fp4_qat.py:37-80"""
    from gcore_lowp.qat import fp4_simulate_qat
    from tests.test_oracle_qat import fp4_known_answer
    say("fp4_simulate_qat known answer")
    x, want = fp4_known_answer()
    x = x.cuda().requires_grad_()
    g = torch.randn_like(x)
    y = fp4_simulate_qat(x)
    y.backward(g)
    assert y.shape == x.shape and y.dtype == x.dtype and torch.isfinite(y).all()
    assert torch.equal(y.detach().cpu(), want)
    assert torch.equal(x.grad, g)


@pytest.mark.parametrize("shape", [(256, 512), (3, 5, 96), (1, 32), (4096, 7168), (1000, 1056)])
def test_fp4_simulate_qat_matches_oracle(shape):
    from gcore_lowp.qat import fp4_simulate_qat
    say("fp4_simulate_qat", shape)
    torch.manual_seed(29)
    x = torch.randn(shape) * torch.logspace(-3, 3, shape[-1] // 32).repeat_interleave(32)
    x.view(-1)[:32] = 0
    x.view(-1)[5] = -0.0
    x = x.bfloat16()
    got = fp4_simulate_qat(x.cuda())
    assert torch.equal(bits16(got), bits16(T.fp4_simulate(x)))


def test_fp4_simulate_qat_equals_export_weight():
    """test_deepseek_v4_fp4_qat.py:97-160: the training forward equals the weight the export path produces, on random
    data, on exact midpoints and after a step across the group-scale boundaries (two different kernels here)."""
    from gcore_lowp.eager_quant_kernels import dequant_fp4_e2m1_fp8_scale_e8m0_packed
    from gcore_lowp.fused_quant_kernels import fp4_qat_then_to_fp8
    from gcore_lowp.qat import fp4_simulate_qat
    from tests.test_oracle_qat import FP4_MIDPOINTS

    def export(w):
        q, s = fp4_qat_then_to_fp8(w.bfloat16().float())
        return dequant_fp4_e2m1_fp8_scale_e8m0_packed(q, s).float()

    say("fp4 qat forward == export")
    torch.manual_seed(29)
    w = torch.randn(256, 512, device="cuda").bfloat16().float()
    assert torch.equal(fp4_simulate_qat(w.bfloat16()).float(), export(w))
    row = torch.tensor(FP4_MIDPOINTS, device="cuda").repeat(16)
    w = row.expand(128, 128).clone()
    w[1::2] *= -1.0
    assert torch.equal(fp4_simulate_qat(w.bfloat16()).float(), export(w))
    torch.manual_seed(31)
    w = fp4_simulate_qat(torch.randn(256, 512, device="cuda").bfloat16()).float()
    signs = torch.randint(0, 2, w.shape, device="cuda").float()
    stepped = w + (signs * 2.0 - 1.0) * 1e-6
    assert torch.equal(fp4_simulate_qat(stepped.bfloat16()).float(), export(stepped))


def test_fp4_simulate_qat_tiny_magnitudes():
    from gcore_lowp.qat import fp4_simulate_qat
    say("fp4_simulate_qat tiny")
    g = torch.Generator().manual_seed(2)
    x = torch.randn(64, 256, generator=g)
    x[:, :64] *= 1e-36
    x[:, 64:128] *= 1e-38
    x[:, 128:160] = 0
    x = x.bfloat16()
    assert torch.equal(bits16(fp4_simulate_qat(x.cuda())), bits16(T.fp4_simulate(x)))


@pytest.mark.parametrize("bs", [64, 128])
def test_fp8_simulate_qat_and_ste(bs):
    from gcore_lowp.qat import fp8_simulate_qat
    say("fp8_simulate_qat", bs)
    torch.manual_seed(5)
    x = (torch.randn(6, 5, 512) * torch.logspace(-6, 3, 6).view(6, 1, 1)).bfloat16()
    xg = x.cuda().requires_grad_()
    y = fp8_simulate_qat(xg, bs)
    g = torch.randn_like(xg)
    y.backward(g)
    assert torch.equal(bits16(y), bits16(T.fp8_simulate(x, bs)))
    assert torch.equal(xg.grad, g)
    big = torch.randn(4096, 7168, generator=torch.Generator().manual_seed(1)).bfloat16()
    assert torch.equal(bits16(fp8_simulate_qat(big.cuda(), bs)), bits16(T.fp8_simulate(big, bs)))


def test_fp8_simulate_qat_128x128_and_linears():
    """tests/test_gfused/test_fp_qat_128x128.py:204-221,279-292,337-353"""
    from gcore_lowp.qat import fp4_qat_linear, fp8_qat_linear, fp8_simulate_qat_128x128
    say("fp8_simulate_qat_128x128 + linears")
    torch.manual_seed(3)
    w = torch.randn(128, 256, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    g = torch.randn_like(w)
    y = fp8_simulate_qat_128x128(w)
    assert torch.equal(bits16(y), bits16(T.fp_qat_128x128(w.detach().cpu())))
    y.backward(g)
    assert torch.equal(w.grad, g)
    torch.manual_seed(29)
    gate_up = torch.randn(2, 256, 128, device="cuda", dtype=torch.bfloat16)
    stacked = fp8_simulate_qat_128x128(gate_up)
    per = torch.stack([fp8_simulate_qat_128x128(gate_up[i]) for i in range(2)])
    assert torch.equal(bits16(stacked), bits16(per))
    assert torch.equal(bits16(stacked), bits16(T.fp_qat_128x128(gate_up.cpu().view(-1, 128)).view_as(gate_up)))
    with pytest.raises(ValueError):
        fp8_simulate_qat_128x128(torch.zeros(128, device="cuda"))
    torch.manual_seed(23)
    lin = torch.nn.Linear(128, 256, bias=False, device="cuda", dtype=torch.bfloat16)
    x = torch.randn(4, 128, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        want = torch.nn.functional.linear(x, T.fp_qat_128x128(lin.weight.detach().cpu()).cuda())
    assert torch.equal(bits16(fp8_qat_linear(lin, x, 128)), bits16(want))
    with pytest.raises(AssertionError):
        fp8_qat_linear(lin, x, 64)
    mod = torch.nn.Linear(64, 32, device="cuda", dtype=torch.bfloat16)
    xi = torch.randn(4, 64, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    out = fp4_qat_linear(mod, xi)
    out.float().square().mean().backward()
    assert out.shape == (4, 32) and torch.isfinite(out).all()
    assert mod.weight.grad is not None and torch.isfinite(mod.weight.grad).all()
    with torch.no_grad():
        want = torch.nn.functional.linear(xi, T.fp4_simulate(mod.weight.detach().cpu()).cuda(), mod.bias)
    assert torch.equal(bits16(out), bits16(want))


@pytest.mark.parametrize("fmt", [None, "ue8m0"])
def test_act_quant_inplace_branch(fmt):
    from gcore_lowp.qat import act_quant
    say("act_quant inplace", fmt)
    torch.manual_seed(9)
    x = (torch.randn(7, 33, 384) * torch.logspace(-6, 3, 7).view(7, 1, 1)).bfloat16()
    xg = x.cuda()
    r = act_quant(xg, 128, fmt, inplace=True)
    assert r is xg
    assert torch.equal(bits16(xg), bits16(T.act_quant_inplace(x, 128, fmt)))
