"""Pins the FP4 paths of the oracle (CPU only): hand-decoded vectors of the reference's
CPU tests, exactness invariants of the rebase, and C == torch restatement."""
import numpy as np
import torch

from oracle import torch_ref as T
from tests import _inputs as I

E8M0 = torch.float8_e8m0fnu


def _bf16_bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def test_nibble_order_and_table(corc):
    """tests/test_tools/test_convert_deepseek_v4_fp4_to_bf16.py:66-93: byte i = ((2i+1)%16)<<4 | (2i)%16
    decodes to table[k % 16] at logical position k."""
    packed = torch.tensor([(((2 * i + 1) % 16) << 4) | ((2 * i) % 16) for i in range(16)], dtype=torch.uint8)
    packed = packed.view(torch.int8).reshape(1, 16)
    scale = torch.ones(1, 1).to(E8M0)
    want = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, 0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0] * 2)
    out = T.cast_e2m1fn_to_bf16(packed, scale)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (1, 32)
    assert torch.equal(out.float().flatten(), want)
    assert not torch.signbit(out.float()).flatten()[8]                 # code 8 -> +0.0 here
    f, b = corc.fp4_dequant(packed.numpy(), scale.view(torch.uint8).numpy(), neg_zero=0)
    assert np.array_equal(b, _bf16_bits(out))
    # the eager_quant_kernels flavour keeps -0.0
    f, b = corc.fp4_dequant(packed.numpy(), scale.view(torch.uint8).numpy(), neg_zero=1)
    assert np.signbit(f[0, 8]) and f[0, 8] == 0


def test_scale_broadcast_direction(corc):
    """:95-121: bytes 0x21, scale[r, b] = 2^(r+b)."""
    w = torch.full((2, 32), 0x21, dtype=torch.uint8).view(torch.int8)
    sf = torch.tensor([[1.0, 2.0], [2.0, 4.0]])
    out = T.cast_e2m1fn_to_bf16(w, sf.to(E8M0)).float()
    pat = torch.tensor([0.5, 1.0]).repeat(16)
    for r in range(2):
        for blk in range(2):
            assert torch.equal(out[r, blk * 32:(blk + 1) * 32], pat * sf[r, blk])
    f, _ = corc.fp4_dequant(w.numpy(), sf.to(E8M0).view(torch.uint8).numpy(), neg_zero=0)
    assert np.array_equal(f, out.numpy())


def test_negative_nibbles(corc):
    """:123-141: 0xF0 -> (0.0, -6.0); 0x9A -> (-1.0, -0.5)."""
    w = torch.tensor([0xF0, 0x9A] + [0] * 14, dtype=torch.uint8).view(torch.int8).reshape(1, 16)
    s = torch.ones(1, 1).to(E8M0)
    f, _ = corc.fp4_dequant(w.numpy(), s.view(torch.uint8).numpy(), neg_zero=0)
    assert f[0, :4].tolist() == [0.0, -6.0, -1.0, -0.5] and not f[0, 4:].any()
    assert T.cast_e2m1fn_to_bf16(w, s).float()[0, :4].tolist() == [0.0, -6.0, -1.0, -0.5]


def test_fp4_dequant_all_bytes_all_edge_scales(corc):
    """All 256 packed bytes x scale bytes {0, 1, 2, 117..127, 252, 253, 254, 255}: C == torch, both flavours."""
    sbytes = [0, 1, 2] + list(range(117, 128)) + [252, 253, 254, 255]
    packed = torch.arange(256, dtype=torch.int32).to(torch.uint8).repeat(len(sbytes), 1)          # [S, 256]
    packed = packed.repeat_interleave(16, dim=1).reshape(len(sbytes), 256, 16).reshape(len(sbytes) * 256, 16)
    scale = torch.tensor(sbytes, dtype=torch.uint8).repeat_interleave(256).reshape(-1, 1)
    want = T.cast_e2m1fn_to_bf16(packed.view(torch.int8), scale.view(E8M0))
    f, b = corc.fp4_dequant(packed.numpy(), scale.numpy(), neg_zero=0)
    wb = _bf16_bits(want)
    nan = torch.isnan(want.float()).numpy()
    assert np.array_equal(b[~nan], wb[~nan]) and ((b[nan] & 0x7FFF) > 0x7F80).all()
    want = T.dequant_fp4_e2m1_fp8_scale_e8m0_packed(packed.view(torch.int8), scale.view(E8M0))
    f, b = corc.fp4_dequant(packed.numpy(), scale.numpy(), neg_zero=1)
    wb = _bf16_bits(want)
    assert np.array_equal(b[~nan], wb[~nan])


def test_rebase_matches_torch_and_is_lossless(corc):
    """tools/dsv4_quant_and_dequant/test_kernels.py:53-76 and test_cuda_parity.py:91-109 shapes."""
    for seed, (rows, cols), (lo, hi) in [(1, (128, 128), (125, 129)), (2, (256, 256), (119, 135)),
                                         (3, (256, 384), (117, 127)), (4, (128, 256), (100, 140))]:
        packed, scale = I.fp4_expert(rows, cols, seed, lo, hi)
        tq, ts = T.cast_e2m1fn_to_e4m3fn(packed, scale)
        q, of, ob = corc.fp4_to_e4m3_rebase(packed.numpy(), scale.view(torch.uint8).numpy())
        assert np.array_equal(q, tq.view(torch.uint8).numpy())
        assert np.array_equal(ob, ts.view(torch.uint8).numpy())
        tq2, ts2 = T.official_expert_to_sgl(packed, scale)
        assert np.array_equal(of, ts2.numpy()) and torch.equal(tq2.view(torch.uint8), tq.view(torch.uint8))
        # lossless wherever the block's scale is within 2^14 of the tile maximum
        direct, _ = corc.fp4_dequant(packed.numpy(), scale.view(torch.uint8).numpy(), neg_zero=0, want_bf16=False)
        back = corc.e4m3fn_to_f32(q) * np.repeat(np.repeat(of, 128, 0), 128, 1)
        sb = scale.view(torch.uint8).numpy().astype(np.int32)
        smax = sb.reshape(rows // 128, 128, cols // 128, 4).max(axis=(1, 3))
        ok = (np.repeat(np.repeat(smax, 128, 0), 4, 1) - sb) <= 14
        ok = np.repeat(ok, 32, 1)
        assert np.array_equal(back[ok], direct[ok])
        # code 8 (+0.0) must give byte 0x00, negative values that underflow give 0x80
        codes = np.stack([packed.view(torch.uint8).numpy() & 0xF, packed.view(torch.uint8).numpy() >> 4], -1).reshape(rows, cols)
        assert (q[codes == 8] == 0).all() and (q[codes == 0] == 0).all()


def test_fused_fp4_to_fp8_composition():
    """The fused conversion is defined as the two-step composition; its bf16 intermediate is exact."""
    packed, scale = I.fp4_expert(256, 256, 9)
    w = T.cast_e2m1fn_to_bf16(packed, scale)
    exact = T.unpack_fp4(packed, T.LUT_POS_ZERO) * scale.float().repeat_interleave(32, -1)
    assert torch.equal(w.float(), exact)
    q, s = T.fp4_to_fp8_amax(packed, scale)
    q2, s2 = T.quant_block_fp32_scale(w, (128, 128))
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s, s2)
