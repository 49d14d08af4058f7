"""MI355X drop-in for gfused/mygemm_fp8.py: block-scaled FP8 GEMM and the plain NT GEMM.

The reference functions are TileLang JIT kernels whose keyword arguments pick
tile sizes; they are accepted here for signature compatibility and otherwise
ignored (tiling is chosen by the HIP kernels).
"""
from __future__ import annotations

import torch

from . import _abi as A
from . import ops

__all__ = ["gemm_fp8_block_scaling_impl", "gemm_impl"]

def _get_workspace(dev: torch.device, nbytes: int) -> torch.Tensor | None:
    """Scratch for the K-split kernels: a fresh tensor per call.  The caching allocator hands the block back to
    the stream that used it last, so two GEMMs on different streams never share partial sums (a cached buffer
    per device would) and a block that is still being read is not given to another stream."""
    if nbytes <= 0:
        return None
    return torch.empty(nbytes, dtype=torch.uint8, device=dev)


def _scale_arg(s: torch.Tensor, dev) -> tuple[torch.Tensor, int]:
    s = s.to(dev)
    if s.dtype == ops.E8M0:
        return s.contiguous(), A.E8M0
    return s.to(torch.float32).contiguous(), A.F32


def gemm_fp8_block_scaling_impl(Aq, As, Bq, Bs, BLK_M=64, BLK_N=128, BLK_K=128, FP8_BLK_SZ=128,
                                dtype=torch.float8_e4m3fn, scale_dtype=torch.float8_e8m0fnu,
                                out_dtype=torch.bfloat16, accum_dtype=torch.float32):
    """gfused/mygemm_fp8.py:44-97.  Aq [M,K] e4m3fn, As [M,K/128], Bq [N,K] e4m3fn,
    Bs [N/128,K/128] -> C [M,N] of out_dtype; the scales may be e8m0 or any real
    float dtype (read as fp32)."""
    assert max(BLK_N, FP8_BLK_SZ) % min(BLK_N, FP8_BLK_SZ) == 0
    assert BLK_K == FP8_BLK_SZ
    assert FP8_BLK_SZ == 128, "only 128-wide scale blocks are built"
    assert dtype == torch.float8_e4m3fn and accum_dtype == torch.float32
    assert Aq.dtype == torch.float8_e4m3fn and Bq.dtype == torch.float8_e4m3fn
    assert Aq.ndim == 2 and Bq.ndim == 2 and Aq.shape[1] == Bq.shape[1]
    M, K = Aq.shape
    N = Bq.shape[0]
    assert K % FP8_BLK_SZ == 0 and N % FP8_BLK_SZ == 0
    assert tuple(As.shape) == (M, K // FP8_BLK_SZ), (tuple(As.shape), (M, K // FP8_BLK_SZ))
    assert tuple(Bs.shape) == (N // FP8_BLK_SZ, K // FP8_BLK_SZ)
    assert out_dtype in (torch.bfloat16, torch.float32)
    a, home = A.to_device(Aq)
    dev = a.device
    a = a.contiguous()
    b = Bq.to(dev).contiguous()
    sa, ca = _scale_arg(As, dev)
    sb, cb = _scale_arg(Bs, dev)
    if ca != cb:
        sa, sb, ca = sa.to(torch.float32), sb.to(torch.float32), A.F32
    C = torch.empty((M, N), dtype=out_dtype, device=dev)
    with torch.cuda.device(dev):
        nws = A.lib().lp_gemm_workspace_bytes(M, N, K)
        ws = _get_workspace(dev, nws)
        A.check(A.lib().lp_gemm_fp8_block(
            a.data_ptr(), sa.data_ptr(), b.data_ptr(), sb.data_ptr(), ca, M, N, K, C.data_ptr(),
            A.BF16 if out_dtype == torch.bfloat16 else A.F32,
            ws.data_ptr() if ws is not None else None, nws, A.stream_ptr()))
    return C.to(home)


_NT_CODES = {torch.float8_e4m3fn: A.E4M3, torch.bfloat16: A.BF16, torch.float32: A.F32}


def gemm_impl(A_, B_, block_M=128, block_N=128, block_K=64, dtype=torch.bfloat16, out_dtype=torch.bfloat16,
              accum_dtype=torch.float32):
    """gfused/mygemm_fp8.py:12-41: C[M,N] = A[M,K] B[N,K]^T, operands of `dtype` (e4m3fn or bf16),
    fp32 accumulation, result cast to `out_dtype` (an e4m3fn result saturates at +-448, as the tile
    compiler's fp8 conversion does)."""
    assert accum_dtype == torch.float32
    if dtype not in (torch.float8_e4m3fn, torch.bfloat16):
        raise TypeError(f"gemm_impl: operands must be float8_e4m3fn or bfloat16, got {dtype}")
    if out_dtype not in _NT_CODES:
        raise TypeError(f"gemm_impl: unsupported out_dtype {out_dtype}")
    assert A_.dtype == dtype and B_.dtype == dtype, (A_.dtype, B_.dtype, dtype)
    assert A_.ndim == 2 and B_.ndim == 2 and A_.shape[1] == B_.shape[1]
    M, K = A_.shape
    N = B_.shape[0]
    a, home = A.to_device(A_)
    dev = a.device
    a = a.contiguous()
    b = B_.to(dev).contiguous()
    C = torch.empty((M, N), dtype=out_dtype, device=dev)
    with torch.cuda.device(dev):
        A.check(A.lib().lp_gemm_nt(a.data_ptr(), b.data_ptr(), _NT_CODES[dtype], M, N, K, C.data_ptr(),
                                   _NT_CODES[out_dtype], A.stream_ptr()))
    return C.to(home)


class _GemmProfiler:
    """`kernel.get_profiler(...).do_bench()` of the tile compiler's kernel objects: average latency in ms."""

    def __init__(self, kernel):
        self._k = kernel

    def do_bench(self, warmup: int = 5, rep: int = 20) -> float:
        k = self._k
        dev = A.require_gpu()
        g = torch.Generator(device=dev).manual_seed(0)
        # small integers (exact in e4m3 and bf16), like the reference's TensorSupplyType.Integer
        a = torch.randint(-3, 4, (k.M, k.K), generator=g, device=dev).to(torch.float32).to(k.dtype)
        b = torch.randint(-3, 4, (k.N, k.K), generator=g, device=dev).to(torch.float32).to(k.dtype)
        for _ in range(max(warmup, 1)):
            k(a, b)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(max(rep, 1)):
            k(a, b)
        stop.record()
        stop.synchronize()
        return start.elapsed_time(stop) / max(rep, 1)


class _CompiledGemm:
    """What `gemm_impl.compile(M=, N=, K=, ...)` returns in the reference (tests/test_gfused/test_my_gemm_fp8.py:141-163):
    a callable fixed to one shape and dtype pair, with a profiler.  Nothing is compiled here; the shape is checked
    when the object is called."""

    def __init__(self, M, N, K, block_M=128, block_N=128, block_K=64, dtype=torch.bfloat16, out_dtype=torch.bfloat16,
                 accum_dtype=torch.float32):
        if dtype not in (torch.float8_e4m3fn, torch.bfloat16):
            raise TypeError(f"gemm_impl: operands must be float8_e4m3fn or bfloat16, got {dtype}")
        if out_dtype not in _NT_CODES:
            raise TypeError(f"gemm_impl: unsupported out_dtype {out_dtype}")
        self.M, self.N, self.K = int(M), int(N), int(K)
        self.dtype, self.out_dtype, self.accum_dtype = dtype, out_dtype, accum_dtype
        self.blocks = (block_M, block_N, block_K)

    def __call__(self, A_, B_):
        assert tuple(A_.shape) == (self.M, self.K) and tuple(B_.shape) == (self.N, self.K), (A_.shape, B_.shape)
        return gemm_impl(A_, B_, *self.blocks, dtype=self.dtype, out_dtype=self.out_dtype, accum_dtype=self.accum_dtype)

    def get_profiler(self, tensor_supply_type=None):
        return _GemmProfiler(self)


gemm_impl.compile = _CompiledGemm
