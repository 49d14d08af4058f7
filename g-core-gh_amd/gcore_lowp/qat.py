"""MI355X drop-in for gpatch_v4/kernel/quantize/qat.py: the activation quantiser, the FP8 / FP4 fake-quantisers of
quantisation-aware training with their straight-through autograd wrappers, and the two QAT linear helpers.

Every quantise-dequantise below is one fused HIP kernel; gradients pass through unchanged, as in the reference."""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn

from . import _abi as A
from . import ops
from .fused_quant_kernels import fp_qat_128x128

__all__ = ["act_quant", "fp4_qat_linear", "fp4_simulate_qat", "fp8_qat_linear", "fp8_simulate_qat",
           "fp8_simulate_qat_128x128"]

_FP8_WEIGHT_BLOCK = (128, 128)


def _on_gpu(x: torch.Tensor):
    """x as a contiguous GPU tensor (CPU inputs are staged through the card, like the other wrappers here)."""
    dev = x.device if x.is_cuda else A.require_gpu()
    return x.contiguous().to(dev), dev


def _act_qdq(z: torch.Tensor, group: int, pow2: bool, through_bf16: bool, want_scale: bool = False):
    """One launch of the 1 x group quantise-dequantise kernel on a contiguous bf16 GPU tensor."""
    if z.dtype != torch.bfloat16:
        raise TypeError(f"the activation quantiser takes bfloat16 (the reference kernel is built for it), got {z.dtype}")
    out = torch.empty_like(z)
    s = z.new_empty(*z.shape[:-1], z.size(-1) // group, dtype=torch.float32) if want_scale else None
    with torch.cuda.device(z.device):
        A.check(A.lib().lp_act_qdq_group(z.data_ptr(), z.numel(), group, int(pow2), int(through_bf16), out.data_ptr(),
                                         s.data_ptr() if s is not None else None, A.stream_ptr()))
    return out, s


def act_quant(x: torch.Tensor, block_size: int = 128, scale_fmt: Optional[str] = None, inplace: bool = False):
    """qat.py:188-223: e4m3fn codes + fp32 scales per 1 x block_size group of the last dim,
    s = max(amax, 1e-4) * fl32(1/448), rounded up to a power of two when scale_fmt is set (e.g. "ue8m0");
    returns (y, s) with s of shape [..., N / block_size].

    inplace=True overwrites x and returns it.  The reference's branch casts the quotient to its output type,
    which in that branch is the input type (qat.py:131,163-175): x <- bf16(fp32(bf16(clamp(x / s))) * s).
    That is what is computed here too, e4m3 is never involved; for an FP8 quantise-dequantise use
    fp8_simulate_qat."""
    n = x.size(-1)
    assert n % block_size == 0
    if inplace:
        z, _ = _on_gpu(x)
        y, _ = _act_qdq(z, block_size, scale_fmt is not None, True)
        x.copy_(y)
        return x
    z = x.contiguous()
    mode = A.SCALE_RCP if scale_fmt is None else A.SCALE_RCP_POW2
    y, s, _ = ops.quant_fp8_block(z.view(-1, n), (1, block_size), scale_mode=mode, scale_dtype=torch.float32,
                                  amax_floor=1e-4)
    return y.view(z.shape), s.view(*z.shape[:-1], n // block_size)


# ------------------------------------------------------------------------------------------------------------
# FP8 fake-quantisers

def _fp8_simulate(x: torch.Tensor, block_size: int) -> torch.Tensor:
    """qat.py:286-301: act_quant(x, block_size, "ue8m0") then the cast back with the same scales, fused."""
    assert x.size(-1) % block_size == 0
    z, _ = _on_gpu(x)
    out, _ = _act_qdq(z, block_size, True, False)
    return out.to(device=x.device, dtype=x.dtype)


def _fp8_simulate_128x128(x: torch.Tensor) -> torch.Tensor:
    """qat.py:310-329: e4m3 + power-of-two scale per 128 x 128 tile on the bf16 view; tensors of rank 3 and more
    (MoE [E, N, K]) are taken as (-1, K)."""
    if x.ndim < 2:
        raise ValueError(f"fp8_simulate_qat_128x128 requires ndim>=2, got {tuple(x.shape)}")
    z, _ = _on_gpu(x)
    out = fp_qat_128x128(z.view(-1, z.shape[-1]).bfloat16())
    return out.view(z.shape).to(device=x.device, dtype=x.dtype)


class _FP8SimulateQAT(torch.autograd.Function):
    """qat.py:332-340."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, block_size: int = 128) -> torch.Tensor:
        return _fp8_simulate(x, block_size)

    @staticmethod
    def backward(ctx, grad: torch.Tensor):
        return grad, None


fp8_simulate_qat = _FP8SimulateQAT.apply


class _FP8SimulateQAT128x128(torch.autograd.Function):
    """qat.py:346-354."""

    @staticmethod
    def forward(ctx, x: torch.Tensor) -> torch.Tensor:
        return _fp8_simulate_128x128(x)

    @staticmethod
    def backward(ctx, grad: torch.Tensor):
        return grad


fp8_simulate_qat_128x128 = _FP8SimulateQAT128x128.apply


# ------------------------------------------------------------------------------------------------------------
# FP4 fake-quantiser

def _fp4_simulate(x: torch.Tensor, block_size: int) -> torch.Tensor:
    """qat.py:350-366: bf16 -> e2m1 with a power-of-two scale per 1 x 32 group (ties to the smaller magnitude, the
    rule of the export kernel) -> bf16."""
    assert x.dtype == torch.bfloat16, f"FP4 QAT requires bfloat16 input, got {x.dtype}"
    assert block_size == 32, f"FP4 QAT requires 1x32 blocks, got {block_size}"
    assert x.size(-1) % block_size == 0
    z, _ = _on_gpu(x)
    out = torch.empty_like(z)
    with torch.cuda.device(z.device):
        A.check(A.lib().lp_fp4_qdq_row32(z.data_ptr(), z.numel(), out.data_ptr(), None, A.stream_ptr()))
    return out.to(x.device)


class _FP4SimulateQAT(torch.autograd.Function):
    """qat.py:369-377."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, block_size: int = 32) -> torch.Tensor:
        return _fp4_simulate(x, block_size)

    @staticmethod
    def backward(ctx, grad: torch.Tensor):
        return grad, None


fp4_simulate_qat = _FP4SimulateQAT.apply


# ------------------------------------------------------------------------------------------------------------
# nn.Linear forwards on fake-quantised weights

def fp8_qat_linear(module: nn.Linear, x: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """qat.py:386-400: module(x) with the weight passed through fp8_simulate_qat_128x128; bias unchanged."""
    assert block_size == 128, f"fp8_qat_linear uses 128×128 weight tiles, got block_size={block_size}"
    weight = fp8_simulate_qat_128x128(module.weight)
    return F.linear(x, weight, module.bias)


def fp4_qat_linear(module: nn.Linear, x: torch.Tensor, block_size: int = 32) -> torch.Tensor:
    """qat.py:403-431: module(x) with the (bfloat16) weight passed through fp4_simulate_qat."""
    weight = fp4_simulate_qat(module.weight, block_size)
    return F.linear(x, weight, module.bias)
