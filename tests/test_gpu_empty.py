"""Empty inputs through the Python drop-ins: zero rows (a tensor that a caller slices to nothing, an expert list in
which nobody received a token) give empty outputs of the right shape and dtype, never a launch with a zero grid or
a failed shape check -- the behaviour of the reference's eager functions on the same inputs."""
import pytest
import torch

pytestmark = pytest.mark.gpu

E4M3, E8M0 = torch.float8_e4m3fn, torch.float8_e8m0fnu


def say(*a):
    print("[case]", *a, flush=True)


def test_zero_rows_quantise_dequantise_convert():
    import gcore_lowp as G
    from gcore_lowp import qat
    dev = "cuda"
    say("empty: quantisers")
    x0 = torch.empty(0, 256, dtype=torch.bfloat16, device=dev)
    for name, f, sdt, scols in (("quant_2d", G.quant_2d, torch.float32, 2), ("quant_1d", G.quant_1d, torch.float32, 2),
                                ("quant_fp8_e4m3_scale_e8m0", G.quant_fp8_e4m3_scale_e8m0, E8M0, 2)):
        q, s = f(x0)
        assert q.dtype == E4M3 and tuple(q.shape) == (0, 256) and s.dtype == sdt and tuple(s.shape) == (0, scols), name
    p, s = G.quant_fp4_e2m1_scale_e8m0_packed(x0)
    assert p.dtype == torch.int8 and tuple(p.shape) == (0, 128) and s.dtype == E8M0 and tuple(s.shape) == (0, 8)
    q, s = G.quantize_fp8_blockwise(x0, (128, 128))
    assert not q.is_cuda and tuple(q.shape) == (0, 256) and s.dtype == torch.bfloat16 and tuple(s.shape) == (0, 2)
    y, s = qat.act_quant(x0)
    assert tuple(y.shape) == (0, 256) and tuple(s.shape) == (0, 2)
    say("empty: FP4 / FP8 -> bf16 and FP4 -> FP8")
    p0, ps0 = torch.empty(0, 128, dtype=torch.int8, device=dev), torch.empty(0, 8, dtype=E8M0, device=dev)
    w = G.cast_e2m1fn_to_bf16(p0, ps0)
    assert w.dtype == torch.bfloat16 and tuple(w.shape) == (0, 256)
    w = G.cast_e4m3fn_to_bf16(torch.empty(0, 256, dtype=E4M3, device=dev), torch.empty(0, 2, dtype=E8M0, device=dev))
    assert w.dtype == torch.bfloat16 and tuple(w.shape) == (0, 256)
    for f in (G.cast_e2m1fn_to_e4m3fn, G.fp4_to_fp8_blockwise, G.official_expert_to_sgl):
        q, s = f(p0, ps0)
        assert q.dtype == E4M3 and tuple(q.shape) == (0, 256) and tuple(s.shape) == (0, 2)


def test_zero_rows_gemm_and_grouped_linear():
    import gcore_lowp as G
    dev = "cuda"
    say("empty: GEMM with M = 0")
    wq = torch.randint(0, 120, (256, 512), device=dev, dtype=torch.uint8).view(E4M3)
    ws = torch.rand(2, 4, device=dev) + 0.5
    c = G.gemm_fp8_block_scaling_impl(torch.empty(0, 512, dtype=E4M3, device=dev), torch.empty(0, 4, device=dev), wq, ws)
    assert c.dtype == torch.bfloat16 and tuple(c.shape) == (0, 256)
    say("empty: grouped GEMM, no expert has rows")
    wq3 = torch.randint(0, 120, (3, 256, 512), device=dev, dtype=torch.uint8).view(E4M3)
    ws3 = torch.rand(3, 2, 4, device=dev) + 0.5
    offs = torch.zeros(4, dtype=torch.int32, device=dev)
    c = G.grouped_gemm_fp8(torch.empty(0, 512, dtype=E4M3, device=dev), torch.empty(0, 4, device=dev), wq3, ws3, offs)
    assert tuple(c.shape) == (0, 256)
    say("empty: grouped linear forward and backward")
    lin = G.MyTeGroupedLinearFp8(3)
    x = torch.empty(0, 512, dtype=torch.bfloat16, device=dev, requires_grad=True)
    w = torch.randn(3, 256, 512, device=dev, requires_grad=True)
    y = lin(x, w, [0, 0, 0])
    assert tuple(y.shape) == (0, 256)
    y.sum().backward()
    assert tuple(x.grad.shape) == (0, 512) and tuple(w.grad.shape) == (3, 256, 512) and not w.grad.any()


def test_measurement_probes_launch_and_reject_bad_arguments():
    """The measurement aids of the probe library (bare stream, register-only matrix-pipe loop, L2-to-LDS copy loop) are what the benchmark's
    floor figures come from: they must launch for every variant the benchmark uses and refuse what they do not implement."""
    from gcore_lowp import _probe_abi as A
    L = A.lib()
    st = torch.cuda.current_stream().cuda_stream
    src = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    dst = torch.empty(1 << 19, dtype=torch.uint8, device="cuda")
    say("probes: stream")
    A.check(L.lp_probe_stream(src.data_ptr(), src.numel(), dst.data_ptr(), dst.numel(), 64, st))
    A.check(L.lp_probe_stream(None, 0, None, 0, 8, st))
    ops = (torch.arange(4096, device="cuda") % 120).to(torch.uint8)
    for k in (0, 2, 4, 6, 8):
        say("probes: matrix pipe, FMAs per instruction", k)
        A.check(L.lp_probe_mfma(k, 10, ops.data_ptr(), 16, st))
        A.check(L.lp_probe_mfma(k, 10, None, 16, st))
    # the copy probe: every variant at the smallest and at the GEMM's row stride; the source is exactly as large as it asks for
    sink = torch.zeros(2048, dtype=torch.uint8, device="cuda")
    for stride in (1024, 7168):
        rows = torch.zeros(4 * 512 * stride, dtype=torch.uint8, device="cuda")
        for to_lds in (1, 0):
            for waves in (4, 8):
                say("probes: copy", stride, to_lds, waves)
                A.check(L.lp_probe_copy(to_lds, waves, 9, rows.data_ptr(), rows.numel(), stride, sink.data_ptr(), 24, st))
        torch.cuda.synchronize()
        assert L.lp_probe_copy(1, 8, 9, rows.data_ptr(), rows.numel() - 16, stride, sink.data_ptr(), 24, st) != 0      # source too small
    assert not sink.any()
    assert L.lp_probe_copy(1, 6, 9, rows.data_ptr(), rows.numel(), 7168, sink.data_ptr(), 24, st) != 0
    assert L.lp_probe_copy(1, 8, 9, rows.data_ptr(), rows.numel(), 512, sink.data_ptr(), 24, st) != 0
    assert L.lp_probe_copy(1, 8, 9, None, 0, 1024, sink.data_ptr(), 24, st) != 0
    torch.cuda.synchronize()
    assert L.lp_probe_mfma(3, 10, None, 16, st) != 0
    assert L.lp_probe_mfma(4, 0, None, 16, st) != 0
    assert L.lp_probe_stream(src.data_ptr(), 15, dst.data_ptr(), 16, 8, st) != 0
