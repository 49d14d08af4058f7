"""MI355X drop-in for the two cast functions of tools/convert_deepseek_v4_fp4_to_bf16.py."""
from __future__ import annotations

import torch

from . import ops

__all__ = ["cast_e2m1fn_to_bf16", "cast_e4m3fn_to_bf16"]


def cast_e2m1fn_to_bf16(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """tools/convert_deepseek_v4_fp4_to_bf16.py:24-46: int8-packed e2m1 [out, in/2] with an
    e8m0 scale per 1 x 32 block -> bf16 [out, in]; code 8 decodes to +0.0."""
    assert x.dtype == torch.int8
    assert x.ndim == 2
    out_dim, in_dim = x.size()
    in_dim *= 2
    assert in_dim % 32 == 0
    assert scale.size(0) == out_dim and scale.size(1) == in_dim // 32
    sc = scale if scale.dtype in (torch.float32, torch.bfloat16, ops.E8M0) else scale.float()
    return ops.dequant_block(x.view(torch.uint8), sc, fp4=True, fp4_neg_zero=False, out_dtype=torch.bfloat16)


def cast_e4m3fn_to_bf16(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """tools/convert_deepseek_v4_fp4_to_bf16.py:51-63: e4m3fn [out, in] with a 128 x 128 block
    scale -> bf16."""
    assert x.dtype == torch.float8_e4m3fn
    assert x.ndim == 2
    out_dim, in_dim = x.size()
    assert out_dim % 128 == 0 and in_dim % 128 == 0
    assert scale.size() == (out_dim // 128, in_dim // 128)
    sc = scale if scale.dtype in (torch.float32, torch.bfloat16, ops.E8M0) else scale.float()
    return ops.dequant_block(x.view(torch.uint8), sc, fp4=False, out_dtype=torch.bfloat16)
