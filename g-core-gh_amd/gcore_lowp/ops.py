"""Tensor-level front end of the C-ABI: allocation with torch, one call each.

Inputs may live on the CPU or the GPU; outputs follow the input's device
(CPU inputs are staged through the GPU -- there is no CPU compute path).
"""
from __future__ import annotations

import torch

from . import _abi as A

E4M3 = torch.float8_e4m3fn
E8M0 = torch.float8_e8m0fnu


def _as_input(x: torch.Tensor) -> tuple[torch.Tensor, int]:
    """bf16 and fp32 are consumed natively; anything else is widened to fp32 (exact for fp16)."""
    if x.dtype == torch.bfloat16:
        return x.contiguous(), A.BF16
    return x.to(torch.float32).contiguous(), A.F32


def quant_fp8_block(x: torch.Tensor, block_size, *, scale_mode: int, scale_dtype: torch.dtype,
                    amax_floor: float = 0.0, zero_rule: int = A.ZERO_NONE, count_nan: bool = False):
    """[..., M, N] -> (e4m3fn [..., M, N], scale [..., M/bm, N/bn]) and, when
    count_nan, the number of blocks holding a NaN (forces a sync)."""
    bm, bn = int(block_size[0]), int(block_size[1])
    m, n = x.shape[-2:]
    xg, home = A.to_device(x)
    xg, code = _as_input(xg)
    lead = tuple(x.shape[:-2])
    rows = m
    for d in lead:
        rows *= d
    q = torch.empty(x.shape, dtype=torch.uint8, device=xg.device)
    scale = torch.empty(lead + (m // max(bm, 1), n // max(bn, 1)), dtype=scale_dtype, device=xg.device)
    nan = torch.zeros(1, dtype=torch.int32, device=xg.device) if count_nan else None
    with torch.cuda.device(xg.device):
        A.check(A.lib().lp_quant_fp8_block(
            xg.data_ptr(), code, rows, n, bm, bn, scale_mode, float(amax_floor), zero_rule,
            q.data_ptr(), scale.data_ptr(), A.scale_code(scale_dtype),
            nan.data_ptr() if count_nan else None, A.stream_ptr()))
    n_nan = int(nan.item()) if count_nan else 0
    return q.view(E4M3).to(home), scale.to(home), n_nan


def quant_fp4_block(x: torch.Tensor, block_size=(1, 32), *, count_nan: bool = False):
    """[..., M, N] -> (packed e2m1 int8 [..., M, N/2], e8m0 scales [..., M/bm, N/bn]) and, when count_nan,
    the number of NaN inputs (forces a sync)."""
    bm, bn = int(block_size[0]), int(block_size[1])
    m, n = x.shape[-2:]
    xg, home = A.to_device(x)
    xg, code = _as_input(xg)
    lead = tuple(x.shape[:-2])
    rows = m
    for d in lead:
        rows *= d
    packed = torch.empty(lead + (m, n // 2), dtype=torch.int8, device=xg.device)
    scale = torch.empty(lead + (m // max(bm, 1), n // max(bn, 1)), dtype=E8M0, device=xg.device)
    nan = torch.zeros(1, dtype=torch.int32, device=xg.device) if count_nan else None
    with torch.cuda.device(xg.device):
        A.check(A.lib().lp_quant_fp4_block(xg.data_ptr(), code, rows, n, bm, bn, packed.data_ptr(), scale.data_ptr(),
                                           nan.data_ptr() if count_nan else None, A.stream_ptr()))
    n_nan = int(nan.item()) if count_nan else 0
    return packed.to(home), scale.to(home), n_nan


def _block_from_shapes(rows, cols, scales, what):
    sr, sc = scales.shape[-2:]
    if sr == 0 or sc == 0 or rows % sr or cols % sc:
        raise ValueError(f"{what} shape ({rows}, {cols}) not divisible by scale grid ({sr}, {sc}).")
    return rows // sr, cols // sc


def dequant_block(codes: torch.Tensor, scales: torch.Tensor, *, fp4: bool, fp4_neg_zero: bool = True,
                  out_dtype: torch.dtype = torch.bfloat16, block: tuple[int, int] | None = None) -> torch.Tensor:
    """e4m3fn [..., M, N] or packed e2m1 [..., M, N/2] times block scales -> out_dtype [..., M, N].  The block is
    the ratio of the two shapes unless the caller's format fixes it (`block`; then an empty tensor is fine too)."""
    cg, home = A.to_device(codes)
    sg = scales.to(cg.device).contiguous()
    cg = cg.contiguous()
    m = cg.shape[-2]
    n = cg.shape[-1] * (2 if fp4 else 1)
    bm, bn = block if block is not None else _block_from_shapes(m, n, sg, "Weight")
    lead = tuple(cg.shape[:-2])
    if tuple(sg.shape[:-2]) != lead:
        raise ValueError(f"leading dims of codes {lead} and scales {tuple(sg.shape[:-2])} differ")
    rows = m
    for d in lead:
        rows *= d
    out = torch.empty(lead + (m, n), dtype=out_dtype, device=cg.device)
    oc = {torch.bfloat16: A.BF16, torch.float32: A.F32}[out_dtype]
    with torch.cuda.device(cg.device):
        if fp4:
            A.check(A.lib().lp_dequant_fp4_block(
                cg.data_ptr(), sg.data_ptr(), A.scale_code(sg.dtype), rows, n, bm, bn,
                A.FP4_NEG_ZERO if fp4_neg_zero else A.FP4_POS_ZERO, out.data_ptr(), oc, A.stream_ptr()))
        else:
            A.check(A.lib().lp_dequant_fp8_block(
                cg.data_ptr(), sg.data_ptr(), A.scale_code(sg.dtype), rows, n, bm, bn,
                out.data_ptr(), oc, A.stream_ptr()))
    return out.to(home)


def fp4_to_fp8_rebase(x: torch.Tensor, scale: torch.Tensor, *, scale_dtype: torch.dtype = E8M0):
    xg, home = A.to_device(x)
    xg = xg.contiguous()
    sg = scale.to(xg.device).contiguous()
    o, half = xg.shape
    i = half * 2
    q = torch.empty((o, i), dtype=torch.uint8, device=xg.device)
    s = torch.empty((o // 128, i // 128), dtype=scale_dtype, device=xg.device)
    with torch.cuda.device(xg.device):
        A.check(A.lib().lp_fp4_to_fp8_rebase(xg.data_ptr(), sg.data_ptr(), o, i, q.data_ptr(), s.data_ptr(),
                                             A.scale_code(scale_dtype), A.stream_ptr()))
    return q.view(E4M3).to(home), s.to(home)


def fp4_to_fp8_amax(x: torch.Tensor, scale: torch.Tensor, *, scale_mode: int = A.SCALE_DIV,
                    scale_dtype: torch.dtype = torch.float32, amax_floor: float = 1e-12,
                    zero_rule: int = A.ZERO_NONE, return_bf16: bool = False):
    xg, home = A.to_device(x)
    xg = xg.contiguous()
    sg = scale.to(xg.device).contiguous()
    o, half = xg.shape
    i = half * 2
    q = torch.empty((o, i), dtype=torch.uint8, device=xg.device)
    s = torch.empty((o // 128, i // 128), dtype=scale_dtype, device=xg.device)
    w = torch.empty((o, i), dtype=torch.bfloat16, device=xg.device) if return_bf16 else None
    with torch.cuda.device(xg.device):
        A.check(A.lib().lp_fp4_to_fp8_amax(xg.data_ptr(), sg.data_ptr(), o, i, scale_mode, float(amax_floor), zero_rule,
                                           q.data_ptr(), s.data_ptr(), A.scale_code(scale_dtype),
                                           w.data_ptr() if return_bf16 else None, A.stream_ptr()))
    if return_bf16:
        return q.view(E4M3).to(home), s.to(home), w.to(home)
    return q.view(E4M3).to(home), s.to(home)


def selftest(which: int) -> int:
    dev = A.require_gpu()
    out = torch.zeros(1, dtype=torch.int64, device=dev)
    with torch.cuda.device(dev):
        A.check(A.lib().lp_selftest(which, out.data_ptr(), A.stream_ptr()))
    return int(out.item())


def debug_cast(kind: int, x: torch.Tensor) -> torch.Tensor:
    dev = A.require_gpu()
    xg = x.to(dev, torch.float32).contiguous()
    out = torch.empty(xg.shape, dtype=torch.int16 if kind == 3 else torch.uint8, device=dev)
    with torch.cuda.device(dev):
        A.check(A.lib().lp_debug_cast(kind, xg.data_ptr(), out.data_ptr(), xg.numel(), A.stream_ptr()))
    return out.cpu()
