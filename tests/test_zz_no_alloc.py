"""The GEMM entry point that allocates nothing (lp_gemm_fp8_block_static: K-split partial sums in a buffer that is part
of the library's device image) against lp_gemm_fp8_block with a caller workspace, through the C ABI: two calls in a
row on shapes that take the K split, the second smaller than the first, must give the same bits as the existing
entry point, and those lie within the GEMM bars of the fp32 dequantise-then-matmul reference (max relative error
<= 2e-2, cosine >= 0.9999).  Collected last: the whole suite has then run in this process before it."""
import pytest
import torch

from oracle import torch_ref as T
from tests import _inputs as I

pytestmark = pytest.mark.gpu


def say(*a):
    print("[case]", *a, flush=True)


def _problem(M, N, K, seed, pow2):
    x, w = I.act_like(M, K, seed), I.weight_like(N, K, seed + 1, outliers=False)
    if pow2:
        xq, xs = T.quant_fp8_e4m3_scale_e8m0(x, (1, 128))
        wq, ws = T.quant_fp8_e4m3_scale_e8m0(w, (128, 128))
    else:
        xq, xs = T.quant_block_fp32_scale(x, (1, 128))
        wq, ws = T.quant_block_fp32_scale(w, (128, 128))
    return xq, xs, wq, ws


@pytest.mark.parametrize("pow2", [False, True], ids=["f32scale", "e8m0scale"])
def test_static_scratch_gemm_equals_workspace_gemm(pow2):
    from gcore_lowp import _abi as A
    L = A.lib()
    dev = A.require_gpu()
    sdt = A.E8M0 if pow2 else A.F32
    # a large K split first, then a small one that re-uses the start of the buffer
    for M, N, K in ((384, 512, 7168), (200, 256, 5120)):
        need = L.lp_gemm_workspace_bytes(M, N, K)
        assert 0 < need <= L.lp_gemm_static_scratch_bytes(), (M, N, K, need)
        # the workspace also holds fp32 copies of e8m0 scales (a tuning aid): what is left must be the K split's partial
        # sums, or this shape would not touch the built-in buffer at all
        r256 = lambda x: (x + 255) // 256 * 256
        scale_copies = r256(M * (K // 128) * 4) + r256((N // 128) * (K // 128) * 4) if M > 64 and K % 512 == 0 else 0
        assert need - scale_copies > 0 and (need - scale_copies) % (M * N * 4) == 0, (need, scale_copies)
        xq, xs, wq, ws = _problem(M, N, K, M + N + K, pow2)
        ref = T.gemm_fp8_block_scaling_ref(xq, xs.float(), wq, ws.float())
        xq, xs, wq, ws = (t.to(dev).contiguous() for t in (xq, xs, wq, ws))
        for out_dtype, code in ((torch.bfloat16, A.BF16), (torch.float32, A.F32)):
            say("static-scratch gemm", (M, N, K), "e8m0" if pow2 else "f32", out_dtype)
            want = torch.full((M, N), float("nan"), dtype=out_dtype, device=dev)
            got = torch.full((M, N), float("nan"), dtype=out_dtype, device=dev)
            wsp = torch.empty(need, dtype=torch.uint8, device=dev)
            with torch.cuda.device(dev):
                A.check(L.lp_gemm_fp8_block(xq.data_ptr(), xs.data_ptr(), wq.data_ptr(), ws.data_ptr(), sdt, M, N, K,
                                            want.data_ptr(), code, wsp.data_ptr(), need, A.stream_ptr()))
                A.check(L.lp_gemm_fp8_block_static(xq.data_ptr(), xs.data_ptr(), wq.data_ptr(), ws.data_ptr(), sdt, M, N, K,
                                                   got.data_ptr(), code, A.stream_ptr()))
            torch.cuda.synchronize()
            assert torch.equal(got, want), (got.float() - want.float()).abs().max().item()
            # nothing is allocated by the call: the device's free memory is the same after three more calls
            free0 = torch.cuda.mem_get_info()[0]
            with torch.cuda.device(dev):
                for _ in range(3):
                    A.check(L.lp_gemm_fp8_block_static(xq.data_ptr(), xs.data_ptr(), wq.data_ptr(), ws.data_ptr(), sdt, M, N, K,
                                                       got.data_ptr(), code, A.stream_ptr()))
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free0
            assert torch.equal(got, want)
            o = got.float().cpu()
            rel = (o - ref).abs().max().item() / ref.abs().max().item()
            cos = torch.nn.functional.cosine_similarity(o.flatten().double(), ref.flatten().double(), dim=0).item()
            assert rel <= 2e-2 and cos >= 0.9999, (rel, cos)


def test_static_scratch_entry_takes_shapes_without_a_k_split():
    """Shapes that never use scratch are served whatever their size: a decode shape whose K split would need more than
    the built-in buffer if it were taken (it is not: the single-launch decode kernel runs), and a prefill shape."""
    from gcore_lowp import _abi as A
    L = A.lib()
    dev = A.require_gpu()
    for M, N, K in ((16, 4096, 7168), (512, 2048, 512)):
        xq, xs, wq, ws = _problem(M, N, K, M + N + K, False)
        ref = T.gemm_fp8_block_scaling_ref(xq, xs.float(), wq, ws.float())
        xq, xs, wq, ws = (t.to(dev).contiguous() for t in (xq, xs, wq, ws))
        got = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
        say("static-scratch gemm without a split", (M, N, K))
        with torch.cuda.device(dev):
            A.check(L.lp_gemm_fp8_block_static(xq.data_ptr(), xs.data_ptr(), wq.data_ptr(), ws.data_ptr(), A.F32, M, N, K,
                                               got.data_ptr(), A.BF16, A.stream_ptr()))
        torch.cuda.synchronize()
        o = got.float().cpu()
        assert (o - ref).abs().max().item() / ref.abs().max().item() <= 2e-2
