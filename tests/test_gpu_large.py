"""Tensors of more than 2^32 elements through the bandwidth kernels (65536 x 73728 = 4.83 G elements, 9.7 GB as
bf16): the results on three 128-row slabs -- the first, the one in which the element index crosses 2^32, the last
-- must equal the same kernel run on that slab alone (which the small-size tests pin against the oracle), and the
crossing slab is also checked against the CPU oracle directly.  A 32-bit offset anywhere on the path shows up as a
mismatch in the second or third slab."""
import pytest
import torch

from oracle import torch_ref as T

pytestmark = pytest.mark.gpu

ROWS, COLS = 65536, 73728
CROSS = (1 << 32) // COLS // 128 * 128          # first row of the 128-row slab that holds element 2^32
SLABS = (0, CROSS, ROWS - 128)


def say(*a):
    print("[case]", *a, flush=True)


def same(a, b):
    a, b = a.detach().cpu().contiguous(), b.detach().cpu().contiguous()
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a.view(torch.uint8), b.view(torch.uint8))


@pytest.fixture(scope="module")
def big_bf16():
    assert ROWS * COLS > 1 << 32 and 0 < CROSS < ROWS - 128
    say("building a", ROWS, "x", COLS, "bf16 tensor on the GPU")
    g = torch.Generator(device="cuda").manual_seed(123)
    x = torch.empty(ROWS, COLS, dtype=torch.bfloat16, device="cuda")
    for r in range(0, ROWS, 8192):                       # in pieces: keeps the generator's temporaries small
        x[r:r + 8192].normal_(0.0, 0.02, generator=g)
    yield x
    del x
    torch.cuda.empty_cache()


def test_large_quant_and_dequant(big_bf16):
    import gcore_lowp as G
    x = big_bf16
    say("large: 128 x 128 quant, fp32 scales")
    q, s = G.quant_2d(x)
    for r in SLABS:
        qs, ss = G.quant_2d(x[r:r + 128].contiguous())
        assert same(q[r:r + 128], qs) and same(s[r // 128:r // 128 + 1], ss), r
    rq, rs = T.quant_block_fp32_scale(x[CROSS:CROSS + 128].cpu(), (128, 128))
    assert same(q[CROSS:CROSS + 128], rq) and same(s[CROSS // 128:CROSS // 128 + 1], rs)
    del q, s
    say("large: 1 x 128 quant")
    q, s = G.quant_1d(x)
    for r in SLABS:
        qs, ss = G.quant_1d(x[r:r + 128].contiguous())
        assert same(q[r:r + 128], qs) and same(s[r:r + 128], ss), r
    del q, s
    say("large: 128 x 128 power-of-two quant, then dequant to bf16")
    q, s = G.quant_fp8_e4m3_scale_e8m0(x)
    d = G.dequant_fp4_e2m1_fp8_scale_e8m0_packed(q, s)
    assert d.dtype == torch.bfloat16
    for r in SLABS:
        qs, ss = G.quant_fp8_e4m3_scale_e8m0(x[r:r + 128].contiguous())
        assert same(q[r:r + 128], qs) and same(s[r // 128:r // 128 + 1], ss), r
        assert same(d[r:r + 128], G.dequant_fp4_e2m1_fp8_scale_e8m0_packed(qs, ss)), r
    rd = T.dequant_fp4_e2m1_fp8_scale_e8m0_packed(q[CROSS:CROSS + 128].cpu(), s[CROSS // 128:CROSS // 128 + 1].cpu())
    assert same(d[CROSS:CROSS + 128], rd)
    del q, s, d
    say("large: bf16 -> packed FP4")
    p, s = G.quant_fp4_e2m1_scale_e8m0_packed(x)
    for r in SLABS:
        ps, ss = G.quant_fp4_e2m1_scale_e8m0_packed(x[r:r + 128].contiguous())
        assert same(p[r:r + 128], ps) and same(s[r:r + 128], ss), r


def test_large_fp4_conversions():
    import gcore_lowp as G
    say("large: building", ROWS, "x", COLS, "packed FP4 codes and e8m0 scales")
    g = torch.Generator(device="cuda").manual_seed(321)
    packed = torch.empty(ROWS, COLS // 2, dtype=torch.uint8, device="cuda")
    for r in range(0, ROWS, 8192):
        packed[r:r + 8192] = torch.randint(0, 256, (8192, COLS // 2), generator=g, device="cuda", dtype=torch.int32).to(torch.uint8)
    scale = torch.randint(117, 128, (ROWS, COLS // 32), generator=g, device="cuda", dtype=torch.int32).to(torch.uint8).view(
        torch.float8_e8m0fnu)
    packed = packed.view(torch.int8)

    def slab(r):
        return packed[r:r + 128].contiguous(), scale[r:r + 128].contiguous()

    say("large: FP4 -> bf16")
    w = G.cast_e2m1fn_to_bf16(packed, scale)
    for r in SLABS:
        assert same(w[r:r + 128], G.cast_e2m1fn_to_bf16(*slab(r))), r
    ps, ss = slab(CROSS)
    assert same(w[CROSS:CROSS + 128], T.cast_e2m1fn_to_bf16(ps.cpu(), ss.cpu()))
    del w
    say("large: FP4 -> FP8, lossless re-basing")
    q, s = G.cast_e2m1fn_to_e4m3fn(packed, scale)
    for r in SLABS:
        qs, s1 = G.cast_e2m1fn_to_e4m3fn(*slab(r))
        assert same(q[r:r + 128], qs) and same(s[r // 128:r // 128 + 1], s1), r
    del q, s
    say("large: FP4 -> bf16 -> FP8, fused")
    q, s = G.fp4_to_fp8_blockwise(packed, scale)
    for r in SLABS:
        qs, s1 = G.fp4_to_fp8_blockwise(*slab(r))
        assert same(q[r:r + 128], qs) and same(s[r // 128:r // 128 + 1], s1), r
    rq, rs = T.quant_block_fp32_scale(T.cast_e2m1fn_to_bf16(ps.cpu(), ss.cpu()), (128, 128))
    assert same(q[CROSS:CROSS + 128], rq) and same(s[CROSS // 128:CROSS // 128 + 1], rs)
