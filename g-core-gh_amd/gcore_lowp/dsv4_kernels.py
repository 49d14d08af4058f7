"""MI355X drop-in for the arithmetic of tools/dsv4_quant_and_dequant/kernels.py
(official DeepSeek-V4 FP4/E8M0 layout <-> SGLang FP8/fp32 layout)."""
from __future__ import annotations

import torch

from . import ops
import re

from .eager_quant_kernels import (dequant_fp4_e2m1_fp8_scale_e8m0_packed, quant_fp4_e2m1_scale_e8m0_packed,
                                  quant_fp8_e4m3_scale_e8m0)

__all__ = [
    "dequant_fp8_block", "cast_e2m1fn_to_e4m3fn", "official_expert_to_sgl", "official_dense_to_sgl",
    "sgl_dense_to_official", "official_wo_a_to_sgl", "sgl_wo_a_to_official", "sgl_expert_to_official",
    "fp4_to_fp8_blockwise", "is_expert_weight", "is_wo_a_weight", "scale_key",
]

# weight roles by checkpoint key (kernels.py:68-83)
_EXPERT_WEIGHT_RE = re.compile(r"(?:^|\.)experts\.\d+\.w[123]\.weight$")
_SHARED_EXPERT_RE = re.compile(r"shared_experts")
_WO_A_WEIGHT_RE = re.compile(r"(?:^|\.)attn\.wo_a\.weight$")


def is_expert_weight(name: str) -> bool:
    return _EXPERT_WEIGHT_RE.search(name) is not None and _SHARED_EXPERT_RE.search(name) is None


def is_wo_a_weight(name: str) -> bool:
    return _WO_A_WEIGHT_RE.search(name) is not None


def scale_key(weight_key: str) -> str:
    assert weight_key.endswith(".weight"), weight_key
    return weight_key[:-len(".weight")] + ".scale"


def dequant_fp8_block(weight: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """kernels.py:86-88."""
    return dequant_fp4_e2m1_fp8_scale_e8m0_packed(weight, scale)


def cast_e2m1fn_to_e4m3fn(x: torch.Tensor, scale: torch.Tensor):
    """kernels.py:91-126: lossless FP4 -> e4m3fn, 128 x 128 e8m0 outer scale = max(e8m0)/64."""
    assert x.dtype == torch.int8
    assert x.ndim == 2
    out_dim, in_dim = x.size()
    in_dim *= 2
    assert in_dim % 128 == 0 and out_dim % 128 == 0
    assert scale.size(0) == out_dim and scale.size(1) == in_dim // 32
    sc = scale if scale.dtype == ops.E8M0 else scale.float().to(ops.E8M0)
    return ops.fp4_to_fp8_rebase(x.view(torch.uint8), sc, scale_dtype=ops.E8M0)


def official_expert_to_sgl(weight: torch.Tensor, scale: torch.Tensor):
    """kernels.py:129-133: as above with the outer scale widened to fp32."""
    assert weight.dtype == torch.int8
    assert weight.ndim == 2
    out_dim, in_dim = weight.size()
    in_dim *= 2
    assert in_dim % 128 == 0 and out_dim % 128 == 0
    assert scale.size(0) == out_dim and scale.size(1) == in_dim // 32
    sc = scale if scale.dtype == ops.E8M0 else scale.float().to(ops.E8M0)
    return ops.fp4_to_fp8_rebase(weight.view(torch.uint8), sc, scale_dtype=torch.float32)


def official_dense_to_sgl(weight: torch.Tensor, scale: torch.Tensor):
    """kernels.py:143-146: bytes kept, e8m0 scale widened to fp32."""
    return weight, scale.float().contiguous()


def sgl_dense_to_official(weight: torch.Tensor, scale: torch.Tensor):
    """kernels.py:149-152: bytes kept, fp32 scale rounded to e8m0."""
    return weight, scale.float().to(torch.float8_e8m0fnu).contiguous()


def official_wo_a_to_sgl(weight: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """kernels.py:155-157."""
    return dequant_fp8_block(weight, scale).to(torch.bfloat16).contiguous()


def sgl_wo_a_to_official(weight: torch.Tensor):
    """kernels.py:160-162."""
    return quant_fp8_e4m3_scale_e8m0(weight.float(), block_size=(128, 128))


def sgl_expert_to_official(weight: torch.Tensor, scale: torch.Tensor):
    """kernels.py:136-140: FP8 expert (fp32 128 x 128 scales) -> packed FP4 + e8m0 1 x 32 scales.  The
    intermediate is the bf16 dequantised weight, as in the reference; it stays on the GPU."""
    dev = ops.A.require_gpu()
    home = weight.device
    full = dequant_fp8_block(weight.to(dev), scale.to(dev))
    q, s = quant_fp4_e2m1_scale_e8m0_packed(full, block_size=(1, 32))
    return q.to(home), s.to(home)


def fp4_to_fp8_blockwise(x: torch.Tensor, scale: torch.Tensor, *, return_bf16: bool = False):
    """FP4 (1 x 32 e8m0) -> bf16 -> e4m3fn with a 128 x 128 fp32 scale = max(amax, 1e-12)/448, fused:
    byte-identical to cast_e2m1fn_to_bf16 followed by the divide-form 128 x 128 quantiser."""
    assert x.dtype == torch.int8 and x.ndim == 2
    out_dim, in_dim = x.size()
    in_dim *= 2
    assert in_dim % 128 == 0 and out_dim % 128 == 0
    assert scale.size(0) == out_dim and scale.size(1) == in_dim // 32
    sc = scale if scale.dtype == ops.E8M0 else scale.float().to(ops.E8M0)
    return ops.fp4_to_fp8_amax(x.view(torch.uint8), sc, return_bf16=return_bf16)
