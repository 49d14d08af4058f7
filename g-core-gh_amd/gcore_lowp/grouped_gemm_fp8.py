"""Grouped (MoE) block-scaled FP8 GEMM, MI355X drop-ins.

* m_grouped_gemm_fp8_fp8_bf16_nt_contiguous -- the DeepGEMM-style call the
  reference makes at tests/test_gpatch_v4/test_deep_gemm_grouped_gemm_fp8.py:106-109.
* MyTeGroupedLinearFp8 -- forward of gpatch_v4/models/deepseek_v4/fp8.py:346-394:
  activations are quantised per 1 x 128, weights per 128 x 128 (or taken
  pre-quantised), one grouped GEMM; no per-expert row padding copies.
"""
from __future__ import annotations

import torch

from . import _abi as A
from . import ops

__all__ = ["grouped_gemm_fp8", "m_grouped_gemm_fp8_fp8_bf16_nt_contiguous", "MyTeGroupedLinearFp8"]


def _scale_arg(s, dev):
    s = s.to(dev)
    if s.dtype == ops.E8M0:
        return s.contiguous(), A.E8M0
    return s.to(torch.float32).contiguous(), A.F32


def grouped_gemm_fp8(xq, xs, wq, ws, m_offsets: torch.Tensor, out: torch.Tensor | None = None,
                     out_dtype=torch.bfloat16) -> torch.Tensor:
    """xq [M,K] e4m3fn, xs [M,K/128], wq [E,N,K] e4m3fn, ws [E,N/128,K/128],
    m_offsets int32 [E+1] on the GPU (rows of expert e: m_offsets[e]..m_offsets[e+1]-1)."""
    M, K = xq.shape
    E, N, K2 = wq.shape
    assert K == K2 and K % 128 == 0 and N % 128 == 0
    assert tuple(xs.shape) == (M, K // 128) and tuple(ws.shape) == (E, N // 128, K // 128)
    dev = xq.device
    assert dev.type == "cuda", "grouped_gemm_fp8 takes GPU tensors"
    sa, ca = _scale_arg(xs, dev)
    sb, cb = _scale_arg(ws, dev)
    if ca != cb:
        sa, sb, ca = sa.to(torch.float32), sb.to(torch.float32), A.F32
    if out is None:
        out = torch.zeros((M, N), dtype=out_dtype, device=dev)
    assert out.is_contiguous() and tuple(out.shape) == (M, N) and out.dtype in (torch.bfloat16, torch.float32)
    offs = m_offsets.to(device=dev, dtype=torch.int32).contiguous()
    assert offs.numel() == E + 1
    with torch.cuda.device(dev):
        A.check(A.lib().lp_gemm_fp8_grouped(
            xq.contiguous().data_ptr(), sa.data_ptr(), wq.contiguous().data_ptr(), sb.data_ptr(), ca,
            offs.data_ptr(), E, M, N, K, out.data_ptr(),
            A.BF16 if out.dtype == torch.bfloat16 else A.F32, A.stream_ptr()))
    return out


def m_grouped_gemm_fp8_fp8_bf16_nt_contiguous(lhs, rhs, out: torch.Tensor, m_indices: torch.Tensor) -> None:
    """lhs = (x_fp8 [M,K], x_scale [M,K/128]); rhs = (w_fp8 [E,N,K], w_scale [E,N/128,K/128]);
    m_indices int32 [M], non-decreasing expert id per row; writes `out` [M,N] bf16 in place."""
    xq, xs = lhs
    wq, ws = rhs
    E = wq.shape[0]
    counts = torch.bincount(m_indices.to(torch.int64).clamp(min=0), minlength=E)[:E]
    offs = torch.zeros(E + 1, dtype=torch.int32, device=xq.device)
    offs[1:] = torch.cumsum(counts, 0).to(torch.int32)
    grouped_gemm_fp8(xq, xs, wq, ws, offs, out=out)


class MyTeGroupedLinearFp8(torch.nn.Module):
    """Forward of fp8.py:346-394 without TransformerEngine: weight is passed in
    ([E,N,K] bf16/fp32, or a pre-quantised (data, scale) pair / object with
    `_data` and `_scale`), rows of `inp` are concatenated in expert order."""

    def __init__(self, num_gemms: int, recipe=None):
        super().__init__()
        self.num_gemms = num_gemms
        self.recipe = recipe

    def forward(self, inp: torch.Tensor, weight, m_splits: list) -> torch.Tensor:
        assert len(m_splits) == self.num_gemms, (len(m_splits), self.num_gemms)
        m_splits = [int(x) for x in m_splits]
        if hasattr(weight, "_data") and hasattr(weight, "_scale"):
            wq, ws = weight._data, weight._scale
        elif isinstance(weight, (tuple, list)):
            wq, ws = weight
        else:
            wq, ws = None, None
        shape = weight.shape if wq is None else wq.shape
        assert len(shape) == 3 and shape[0] == self.num_gemms, (tuple(shape), m_splits)
        n_out, k_in = shape[1], shape[2]
        assert inp.size(-1) == k_in, (inp.size(-1), k_in)
        x = inp.reshape(-1, k_in)
        assert sum(m_splits) == x.shape[0], (sum(m_splits), x.shape[0])
        from .eager_quant_kernels import quant_fp8_e4m3_scale_e8m0
        # Float8BlockScaling recipe: power-of-two scales for activations and weights
        xq, xs = quant_fp8_e4m3_scale_e8m0(x, block_size=(1, 128))
        if wq is None:
            wq, ws = quant_fp8_e4m3_scale_e8m0(weight, block_size=(128, 128))
        if wq.dtype == torch.uint8:
            wq = wq.view(ops.E4M3)
        offs = torch.zeros(self.num_gemms + 1, dtype=torch.int32)
        offs[1:] = torch.cumsum(torch.tensor(m_splits, dtype=torch.int64), 0).to(torch.int32)
        out = grouped_gemm_fp8(xq, xs, wq, ws, offs.to(x.device), out_dtype=inp.dtype
                               if inp.dtype in (torch.bfloat16, torch.float32) else torch.bfloat16)
        return out.view(*inp.shape[:-1], n_out)
