"""Tensor wrappers that carry block-quantised expert weights into the grouped FP8 GEMM; MI355X drop-in for
gpatch_v4/models/deepseek_v4/fp8_tensor.py.

* Fp8TensorAg (fp8_tensor.py:65-244): the parameter a sharded-data-parallel wrapper keeps resident.  It looks and
  behaves like its fp32 backing tensor; the two hooks that FSDP2 calls around its all-gather turn the local shard
  [E_local, N, K] into (e4m3 codes, e8m0 scales per 128 x 128 block) as uint8 before the gather and assemble the
  gathered bytes into an Fp8TensorTrain afterwards.  The quantisation is quant_fp8_e4m3_scale_e8m0 (one HIP
  kernel launch on the shard).  Nothing here communicates: the gather itself belongs to the caller.
* Fp8TensorTrain (fp8_tensor.py:247-320): the gathered weight; claims the compute dtype, holds `_data` (codes
  [E, N, K]) and `_scale` (e8m0 [E, N/128, K/128]).  MyTeGroupedLinearFp8 consumes `_data` / `_scale` directly.
"""
from __future__ import annotations

from typing import Any

import torch
from torch.utils import _pytree

from .eager_quant_kernels import quant_fp8_e4m3_scale_e8m0

__all__ = ["Fp8TensorAg", "Fp8TensorTrain"]

BLOCK = (128, 128)
_aten = torch.ops.aten

# Ops whose result stays an Fp8TensorAg (the structural and copy ops that sharding, CPU offload and reload use;
# fp8_tensor.py:36-47).  Everything else computes on the backing tensor and returns a plain tensor.
_AG_KEEPS_WRAPPER = frozenset((
    _aten.as_strided.default, _aten.clone.default, _aten.copy_.default, _aten.empty_like.default,
    _aten.new_zeros.default, _aten.slice.Tensor, _aten.split.Tensor, _aten._pin_memory.default,
    _aten._to_copy.default, _aten.view.default,
))
# Structural ops an Fp8TensorTrain supports: applied to the codes, scales carried along (fp8_tensor.py:294-308).
_TRAIN_STRUCTURAL = frozenset((_aten.as_strided.default, _aten.clone.default, _aten.slice.Tensor, _aten.view.default))


def _shell(cls, like: torch.Tensor, dtype: torch.dtype, requires_grad: bool):
    """A storage-less tensor of class cls with the geometry of `like`."""
    return torch.Tensor._make_wrapper_subclass(
        cls, like.size(), strides=like.stride(), storage_offset=like.storage_offset(), dtype=dtype,
        layout=like.layout, device=like.device, pin_memory=like.is_pinned(), requires_grad=requires_grad)


def new_hook_stats() -> dict[str, Any]:
    """Counters the hooks keep on `module._fp8_all_gather_stats` (fp8_tensor.py:50-62)."""
    return {"pre_calls": 0, "post_new_calls": 0, "post_reuse_calls": 0, "compute_dtype": None, "payload_dtype": None,
            "payload_bytes": 0, "fp8_bytes": 0, "scale_bytes": 0, "high_precision_bytes": 0}


class Fp8TensorTrain(torch.Tensor):
    """Gathered expert weights: logical dtype `dtype`, storage = FP8 codes + e8m0 block scales."""

    @staticmethod
    def __new__(cls, data: torch.Tensor, scale: torch.Tensor, dtype: torch.dtype):
        return _shell(cls, data, dtype, False)

    def __init__(self, data: torch.Tensor, scale: torch.Tensor, dtype: torch.dtype) -> None:
        self._data, self._scale, self._logical_dtype = data, scale, dtype

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        me = args[0]
        if func is _aten.detach.default:
            return cls(me._data.detach(), me._scale, me._logical_dtype)
        if func in _TRAIN_STRUCTURAL:
            return cls(func(me._data, *args[1:], **(kwargs or {})), me._scale, me._logical_dtype)
        raise NotImplementedError(f"{cls.__name__} does not implement {func}")

    def __tensor_flatten__(self):
        return ["_data", "_scale"], {"dtype": self._logical_dtype}

    @staticmethod
    def __tensor_unflatten__(inner_tensors, metadata, outer_size, outer_stride):
        return Fp8TensorTrain(inner_tensors["_data"], inner_tensors["_scale"], metadata["dtype"])

    def __repr__(self):
        return (f"Fp8TensorTrain(shape={tuple(self.shape)}, dtype={self._logical_dtype}, "
                f"scale_shape={tuple(self._scale.shape)})")


class Fp8TensorAg(torch.Tensor):
    """fp32 (or bf16) parameter whose all-gather payload is FP8 codes + block scales."""

    @staticmethod
    def __new__(cls, tensor: torch.Tensor):
        return _shell(cls, tensor, tensor.dtype, tensor.requires_grad)

    def __init__(self, tensor: torch.Tensor) -> None:
        self._tensor = tensor

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        if func is _aten.detach.default:
            return cls(args[0]._tensor.detach())
        seen: list[torch.dtype] = []

        def backing(t):
            seen.append(t._tensor.dtype)
            assert t._tensor.dtype == seen[0], (t._tensor.dtype, seen[0])
            return t._tensor

        plain_args, plain_kwargs = _pytree.tree_map_only(cls, backing, (args, kwargs or {}))
        result = func(*plain_args, **plain_kwargs)
        if func in _AG_KEEPS_WRAPPER:
            return _pytree.tree_map_only(torch.Tensor, cls, result)
        return result

    def __tensor_flatten__(self):
        return ["_tensor"], None

    @staticmethod
    def __tensor_unflatten__(inner_tensors, metadata, outer_size, outer_stride):
        return Fp8TensorAg(inner_tensors["_tensor"])

    def __repr__(self):
        return f"Fp8TensorAg({self._tensor!r})"

    # -- the hooks FSDP2 calls around the all-gather of this parameter ------------------------------------------
    def fsdp_pre_all_gather(self, mesh, orig_size, contiguous_orig_stride, module, mp_policy):
        """Local shard -> ((codes uint8 [chunk, N, K], scale bytes), metadata); fp8_tensor.py:133-212.

        The parameter is sharded along its first dimension in chunks of ceil(E / world): a rank holds
        min(chunk, max(E - rank * chunk, 0)) experts, anything else is a ValueError.  Every rank sends `chunk`
        experts (short and empty shards are zero-padded, a zero block quantises to codes 0 and scale 1.0).  Block
        scales differ between ranks, so they travel as a second gather input.  When E does not divide evenly the
        gather's inputs must have equal shapes on every rank AND the scale bytes cannot be trimmed by a slice of
        the first dimension afterwards, so they ride at the front of a zero buffer shaped like the codes."""
        world = mesh.size()
        experts = orig_size[0]
        chunk = -(-experts // world)
        mine = min(chunk, max(experts - mesh.get_local_rank() * chunk, 0))
        local = self._tensor.detach()
        tail = tuple(orig_size[1:])
        if tuple(local.shape) != (mine,) + tail:
            raise ValueError(f"FP8 all-gather local shape {tuple(local.shape)} != expected {(mine,) + tail}")
        assert orig_size[-2] % BLOCK[0] == 0 and orig_size[-1] % BLOCK[1] == 0, (
            f"global shape {tuple(orig_size)} not divisible by block {BLOCK}")
        if mine != chunk:
            padded = local.new_zeros((chunk,) + tail)
            if mine:
                padded[:mine].copy_(local)
            local = padded
        codes, scale = quant_fp8_e4m3_scale_e8m0(local, block_size=BLOCK)
        codes_u8 = codes.view(torch.uint8)
        scale_u8 = scale.view(torch.uint8).contiguous()
        uneven = experts % world != 0
        if uneven:
            carrier = torch.zeros_like(codes_u8)
            carrier.view(-1)[:scale_u8.numel()].copy_(scale_u8.view(-1))
        else:
            carrier = scale_u8
        stats = module._fp8_all_gather_stats
        stats["pre_calls"] += 1
        stats["payload_dtype"] = str(codes_u8.dtype)
        stats["fp8_bytes"] = codes_u8.numel()
        stats["scale_bytes"] = carrier.numel()
        stats["payload_bytes"] = stats["fp8_bytes"] + stats["scale_bytes"]
        stats["high_precision_bytes"] = local.numel() * local.element_size()
        meta = {"stats": stats, "is_uneven": uneven, "mesh_size": world, "orig_outer": experts, "chunk_outer": chunk,
                "scale_tail_shape": tuple(scale_u8.shape[1:]), "scale_numel_per_rank": scale_u8.numel()}
        return (codes_u8, carrier), meta

    def fsdp_post_all_gather(self, all_gather_outputs, metadata, param_dtype, *, out=None):
        """Gathered bytes -> Fp8TensorTrain (first call), or refresh the one from the first call (`out`);
        fp8_tensor.py:214-244.  Both gather outputs are rank-major along the first dimension."""
        gathered_codes, gathered_carrier = all_gather_outputs
        stats = metadata["stats"]
        if metadata["is_uneven"]:
            world, chunk, experts = metadata["mesh_size"], metadata["chunk_outer"], metadata["orig_outer"]
            data = gathered_codes[:experts]
            per_rank = gathered_carrier.reshape(world, -1)[:, :metadata["scale_numel_per_rank"]]
            scale_u8 = per_rank.reshape(world * chunk, *metadata["scale_tail_shape"])[:experts]
        else:
            data, scale_u8 = gathered_codes, gathered_carrier
        scale = scale_u8.view(torch.float8_e8m0fnu)
        stats["compute_dtype"] = str(param_dtype)
        if out is not None:
            assert isinstance(out, Fp8TensorTrain)
            out._data, out._scale = data, scale
            stats["post_reuse_calls"] += 1
            return None
        stats["post_new_calls"] += 1
        return Fp8TensorTrain(data, scale, param_dtype), (gathered_codes, gathered_carrier)
