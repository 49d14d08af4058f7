"""MI355X drop-in for gpatch_v4/kernel/quantize/fused_quant_kernels.py: the two fused conversions of the
DeepSeek-V4 weight-export path, same names, checks and exceptions (the reference builds them with TileLang)."""
from __future__ import annotations

import torch

from . import _abi as A

__all__ = ["fp4_qat_then_to_fp8", "fp_qat_128x128"]

_FP8_BLOCK_SIZE = 128


def fp4_qat_then_to_fp8(weight: torch.Tensor):
    """fused_quant_kernels.py:239-274: fp32 QAT master weight -> (e4m3fn weight, e8m0 128 x 128 scale) through
    e2m1 with 1 x 32 e8m0 scales; equals quant_fp4_e2m1_scale_e8m0_packed followed by the lossless rebase."""
    if weight.ndim != 2:
        raise ValueError(f"Expected a 2D weight, got shape {tuple(weight.shape)}")
    if weight.dtype != torch.float32:
        raise TypeError(f"Expected an FP32 master weight, got {weight.dtype}")
    if not weight.is_cuda:
        raise ValueError("fp4_qat_then_to_fp8 requires a CUDA tensor")
    m, n = weight.shape
    if m % _FP8_BLOCK_SIZE != 0 or n % _FP8_BLOCK_SIZE != 0:
        raise ValueError(f"FP4-to-SGL FP8 conversion requires 128x128-aligned weights, got {(m, n)}")
    weight = weight.contiguous()
    fp8_weight = torch.empty_like(weight, dtype=torch.float8_e4m3fn)
    fp8_scale = torch.empty((m // _FP8_BLOCK_SIZE, n // _FP8_BLOCK_SIZE), dtype=torch.float8_e8m0fnu, device=weight.device)
    with torch.cuda.device(weight.device):
        A.check(A.lib().lp_fp4_qat_to_fp8(weight.data_ptr(), m, n, fp8_weight.data_ptr(), fp8_scale.data_ptr(), A.stream_ptr()))
    return fp8_weight, fp8_scale


def fp_qat_128x128(weight: torch.Tensor) -> torch.Tensor:
    """fused_quant_kernels.py:363-403: bf16 -> e4m3fn (one power-of-two scale per 128 x 128 tile) -> bf16; equals
    quant_fp8_e4m3_scale_e8m0 followed by dequant_fp4_e2m1_fp8_scale_e8m0_packed."""
    if weight.ndim != 2:
        raise ValueError(f"Expected a 2D weight, got shape {tuple(weight.shape)}")
    if weight.dtype != torch.bfloat16:
        raise TypeError(f"Expected bfloat16 weight, got {weight.dtype}")
    if not weight.is_cuda:
        raise ValueError("fp_qat_128x128 requires a CUDA tensor")
    m, n = weight.shape
    if m % _FP8_BLOCK_SIZE != 0 or n % _FP8_BLOCK_SIZE != 0:
        raise ValueError(f"fp_qat_128x128 requires 128x128-aligned weights, got {(m, n)}")
    weight = weight.contiguous()
    out = torch.empty_like(weight)
    with torch.cuda.device(weight.device):
        A.check(A.lib().lp_qdq_fp8_tile128(weight.data_ptr(), m, n, out.data_ptr(), A.stream_ptr()))
    return out
