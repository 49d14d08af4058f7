"""MI355X drop-in for gpatch_v4/kernel/quantize/eager_quant_kernels.py.

Same names, arguments, return dtypes/shapes and exceptions as the reference
functions; the arithmetic runs in hand-written HIP kernels.
"""
from __future__ import annotations

import torch

from . import _abi as A
from . import ops

__all__ = ["quant_fp4_e2m1_scale_e8m0_packed", "quant_fp8_e4m3_scale_e8m0", "dequant_fp4_e2m1_fp8_scale_e8m0_packed"]


def quant_fp4_e2m1_scale_e8m0_packed(value: torch.Tensor, block_size: tuple[int, int] = (1, 32)):
    """eager_quant_kernels.py:63-129: packed e2m1 codes (int8 [..., M, N/2], low nibble = even column) + one
    power-of-two (e8m0) scale per block, s = 2^ceil(log2(amax/6)), all-zero block -> s = 1; a value half way
    between two code points takes the one of smaller magnitude; -0.0 keeps its sign (code 8)."""
    m, n = value.shape[-2:]
    bm, bn = block_size
    assert m % bm == 0 and n % bn == 0, f"value shape ({m}, {n}) not divisible by block ({bm}, {bn})"
    assert n % 2 == 0, f"FP4 packing requires N (={n}) to be even (two nibbles per byte)"
    packed, scale, n_nan = ops.quant_fp4_block(value, (bm, bn), count_nan=True)
    assert n_nan == 0, "quant_fp4_e2m1_scale_e8m0_packed: input contains NaN"
    return packed, scale


def quant_fp8_e4m3_scale_e8m0(value: torch.Tensor, block_size: tuple[int, int] = (128, 128)):
    """eager_quant_kernels.py:132-181: e4m3fn codes + one power-of-two (e8m0) scale
    per block, s = 2^ceil(log2(amax/448)), all-zero block -> s = 1.

    ceil(log2(.)) is evaluated exactly from the bit pattern; this equals the
    reference's libm evaluation for every input on the bf16 grid and can differ
    only when amax/448 lies within a few fp32 ulps above a power of two.
    """
    m, n = value.shape[-2:]
    bm, bn = block_size
    assert m % bm == 0 and n % bn == 0, f"value shape ({m}, {n}) not divisible by block ({bm}, {bn})"
    q, s, n_nan = ops.quant_fp8_block(value, (bm, bn), scale_mode=A.SCALE_POW2, scale_dtype=ops.E8M0,
                                      count_nan=True)
    assert n_nan == 0, "quant_fp8_e4m3_scale_e8m0: input contains NaN"
    return q, s


def dequant_fp4_e2m1_fp8_scale_e8m0_packed(quantized: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """eager_quant_kernels.py:200-233: block size = shape ratio; int8 /
    float4_e2m1fn_x2 inputs are packed FP4 (code 8 = -0.0), anything else is
    read as e4m3fn; result dtype = scales.dtype if it is a float of >= 2 bytes,
    else bf16."""
    fp4x2 = getattr(torch, "float4_e2m1fn_x2", None)
    is_fp4 = quantized.dtype == torch.int8 or (fp4x2 is not None and quantized.dtype == fp4x2)
    out_dtype = scales.dtype if scales.dtype.is_floating_point and scales.element_size() >= 2 else torch.bfloat16
    codes = quantized
    if is_fp4:
        codes = quantized.view(torch.uint8)
    elif quantized.dtype != ops.E4M3:
        raise TypeError(f"expected int8 (packed FP4) or float8_e4m3fn codes, got {quantized.dtype}")
    kernel_out = torch.float32 if out_dtype != torch.bfloat16 else torch.bfloat16
    sc = scales if scales.dtype in (torch.float32, torch.bfloat16, ops.E8M0) else scales.to(torch.float32)
    out = ops.dequant_block(codes.view(torch.uint8), sc, fp4=is_fp4, fp4_neg_zero=True, out_dtype=kernel_out)
    return out if out.dtype == out_dtype else out.to(out_dtype)
