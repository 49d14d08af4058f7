"""MI355X drop-in for the activation quantiser of gpatch_v4/kernel/quantize/qat.py."""
from __future__ import annotations

from typing import Optional

import torch

from . import _abi as A
from . import ops

__all__ = ["act_quant"]


def act_quant(x: torch.Tensor, block_size: int = 128, scale_fmt: Optional[str] = None, inplace: bool = False):
    """qat.py:188-223: e4m3fn codes + fp32 scales per 1 x block_size group of the last dim,
    s = max(amax, 1e-4) * fl32(1/448), rounded up to a power of two when scale_fmt is set (e.g. "ue8m0");
    returns (y, s) with s of shape [..., N / block_size].

    inplace=True is not built: the reference's branch rounds through the input dtype (bf16) instead of e4m3
    (qat.py:131,163-175), which is not a quantise-dequantise of FP8; use fp_qat_128x128 or
    act_quant + dequantise for that."""
    if inplace:
        raise NotImplementedError("act_quant(inplace=True) is not built (see the docstring)")
    n = x.size(-1)
    assert n % block_size == 0
    z = x.contiguous()
    mode = A.SCALE_RCP if scale_fmt is None else A.SCALE_RCP_POW2
    y, s, _ = ops.quant_fp8_block(z.view(-1, n), (1, block_size), scale_mode=mode, scale_dtype=torch.float32,
                                  amax_floor=1e-4)
    return y.view(z.shape), s.view(*z.shape[:-1], n // block_size)
