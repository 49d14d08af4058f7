"""Block-FP8 quantisers with fp32 (or caller-chosen) scales, MI355X drop-ins.

* quantize_fp8_blockwise -- tools/convert_fp8/qwen3_5/qwen3_mtp_fp8_postprocess.py:102-151
  (multiply form, HF fine-grained FP8 compatible).
* quant_2d / quant_1d    -- the divide-form helpers every GEMM test of the
  reference quantises with: tests/test_gfused/test_te_gemm_fp8.py:82-101,
  tests/test_gfused/test_deepseek_tilekernels_quant.py:22-58.
* quant_act / quant_weight -- tests/test_gpatch_v4/test_deep_gemm_grouped_gemm_fp8.py:29-72.
"""
from __future__ import annotations

import torch

from . import _abi as A
from . import ops

__all__ = ["quantize_fp8_blockwise", "quant_1d", "quant_2d", "quant_act", "quant_weight"]


def quantize_fp8_blockwise(weight: torch.Tensor, block_size: tuple[int, int], *, device=None,
                           scale_dtype: torch.dtype = torch.bfloat16):
    """f = 448/amax (1 for an all-zero tile), q = cast(clamp(w * f)), scale_inv = 1/f.

    Returns CPU tensors like the reference (`:151`).  `device` is accepted for
    signature compatibility; the work always runs on the current GPU.
    """
    if weight.ndim != 2:
        raise ValueError(f"Expected a 2D weight, got shape={tuple(weight.shape)}")
    bm, bn = block_size
    rows, cols = weight.shape
    if rows % bm != 0 or cols % bn != 0:
        raise ValueError(f"Matrix dimensions ({rows}, {cols}) must be divisible by block sizes ({bm}, {bn})")
    if device is not None and torch.device(device).type == "cuda":
        weight = weight.to(device)
    elif not weight.is_cuda:
        weight = weight.to(A.require_gpu())
    kdt = scale_dtype if scale_dtype in (torch.float32, torch.bfloat16, ops.E8M0) else torch.float32
    q, s, _ = ops.quant_fp8_block(weight, (bm, bn), scale_mode=A.SCALE_MUL, scale_dtype=kdt)
    if s.dtype != scale_dtype:
        s = s.to(scale_dtype)
    return q.cpu(), s.cpu()


def _div_quant(x, block, *, round_sf, amax_floor, zero_rule):
    if round_sf:
        # s = 2^ceil(log2(max(amax, floor) / 448)) as an fp32 tensor; a floored block has no all-zero rule
        # (tests/test_gfused/test_deepseek_tilekernels_quant.py:32-35,51-54)
        q, s, _ = ops.quant_fp8_block(x, block, scale_mode=A.SCALE_POW2, scale_dtype=torch.float32,
                                      amax_floor=amax_floor, zero_rule=A.ZERO_NONE)
        return q, s
    q, s, _ = ops.quant_fp8_block(x, block, scale_mode=A.SCALE_DIV, scale_dtype=torch.float32,
                                  amax_floor=amax_floor, zero_rule=zero_rule)
    return q, s


def quant_1d(x: torch.Tensor, block_size: int = 128, *, round_sf: bool = False):
    """Row-wise 1 x block_size activation quant, s = max(amax, 1e-12)/448 (round_sf: rounded up to a power of two).
    Returns (e4m3fn [M, K], fp32 scale [M, K/block_size])."""
    return _div_quant(x, (1, block_size), round_sf=round_sf, amax_floor=1e-12, zero_rule=A.ZERO_NONE)


def quant_2d(w: torch.Tensor, block_size: tuple[int, int] = (128, 128), *, round_sf: bool = False):
    """bm x bn weight quant, s = max(amax, 1e-12)/448 (round_sf: rounded up to a power of two).
    Returns (e4m3fn [N, K], fp32 scale [N/bm, K/bn])."""
    return _div_quant(w, tuple(block_size), round_sf=round_sf, amax_floor=1e-12, zero_rule=A.ZERO_NONE)


def quant_act(x: torch.Tensor):
    """1 x 128 activation quant, s = amax/448 with s == 0 -> 1 (no floor)."""
    return _div_quant(x, (1, 128), round_sf=False, amax_floor=0.0, zero_rule=A.ZERO_SCALE_TO_ONE)


def quant_weight(w: torch.Tensor):
    """[E, N, K] (or [N, K]) 128 x 128 weight quant, s = amax/448 with s == 0 -> 1."""
    return _div_quant(w, (128, 128), round_sf=False, amax_floor=0.0, zero_rule=A.ZERO_SCALE_TO_ONE)
