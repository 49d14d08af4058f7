"""Adds the Qwen3 multi-token-prediction (MTP) weights to an FP8 checkpoint; MI355X drop-in for
tools/convert_fp8/qwen3_5/qwen3_mtp_fp8_postprocess.py.

The top-level `mtp.*` tensors of the bf16 checkpoint are read directly, the stacked expert tensors are split into
per-expert `gate_proj` / `up_proj` / `down_proj` weights, every weight whose module is not on the skip list is
quantised block-wise (f = 448 / amax, codes = e4m3(clamp(w * f)), `weight_scale_inv` = 1 / f in `scale_dtype`) and
the result goes into its own shard `mtp.safetensors`, with the index rewritten (:345-388).  The quantiser is the
HIP kernel behind `quantize_fp8_blockwise` (:102-151); a stacked expert tensor is quantised in one launch (tiles of
the stack are the tiles of its experts when the block height divides the rows of each part) and cut up on the host
afterwards.  `device` is accepted for signature compatibility: the work runs on the current GPU.
"""
from __future__ import annotations

import json
import math
import os
import re
from glob import glob
from typing import Any

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from . import _abi as A
from . import ops
from .fp8_blockwise import quantize_fp8_blockwise

__all__ = ["append_mtp_weights_to_fp8_checkpoint", "quantize_fp8_blockwise"]

MTP_SHARD = "mtp.safetensors"
INDEX = "model.safetensors.index.json"
_ALWAYS_REQUIRED = ("mtp.fc.weight", "mtp.norm.weight", "mtp.pre_fc_norm_embedding.weight", "mtp.pre_fc_norm_hidden.weight")
_REQUIRED_PER_MOE_LAYER = (
    "input_layernorm.weight", "post_attention_layernorm.weight",
    "self_attn.q_proj.weight", "self_attn.k_proj.weight", "self_attn.v_proj.weight", "self_attn.o_proj.weight",
    "self_attn.q_norm.weight", "self_attn.k_norm.weight",
    "mlp.experts.gate_up_proj", "mlp.experts.down_proj", "mlp.gate.weight",
    "mlp.shared_expert.gate_proj.weight", "mlp.shared_expert.up_proj.weight", "mlp.shared_expert.down_proj.weight",
    "mlp.shared_expert_gate.weight",
)
_SAFETENSORS_ITEMSIZE = {"BOOL": 1, "U8": 1, "I8": 1, "F8_E4M3": 1, "F8_E5M2": 1, "I16": 2, "U16": 2, "F16": 2, "BF16": 2,
                         "I32": 4, "U32": 4, "F32": 4, "I64": 8, "U64": 8, "F64": 8}


def _text_config(input_hf_path: str) -> dict[str, Any]:
    with open(os.path.join(input_hf_path, "config.json")) as f:
        cfg = json.load(f)
    return cfg.get("text_config", cfg)


def _required_moe_mtp_keys(num_layers: int) -> set[str]:
    return set(_ALWAYS_REQUIRED) | {f"mtp.layers.{i}.{s}" for i in range(num_layers) for s in _REQUIRED_PER_MOE_LAYER}


def _should_convert_module(module: str, skip: list[str] | None) -> bool:
    """A module is left alone when a skip entry matches its name as a regex prefix or is its suffix (:86-93)."""
    if skip is None:
        return True
    return not any(re.match(pat, module) or module.endswith(pat) for pat in skip)


def _module_of(weight_key: str) -> str:
    return weight_key[: -len(".weight")] if weight_key.endswith(".weight") else weight_key


def _read_mtp_tensors(input_hf_path: str) -> dict[str, torch.Tensor]:
    found: dict[str, torch.Tensor] = {}
    for shard in sorted(glob(os.path.join(input_hf_path, "*.safetensors"))):
        with safe_open(shard, framework="pt", device="cpu") as f:
            for key in f.keys():
                if key.startswith("mtp."):
                    found[key] = f.get_tensor(key)
    return found


def _validate(input_hf_path: str, tensors: dict[str, torch.Tensor]) -> None:
    """:188-209: MTP configured but absent -> ValueError; more than one MTP layer -> NotImplementedError; a MoE
    model with an incomplete MTP layer -> KeyError."""
    text = _text_config(input_hf_path)
    layers = int(text.get("mtp_num_hidden_layers", 0) or 0)
    if layers == 0:
        return
    if not tensors:
        raise ValueError(f"{input_hf_path} config enables MTP (mtp_num_hidden_layers={layers}) "
                         "but no top-level mtp.* tensors were found")
    if layers != 1:
        raise NotImplementedError(f"Only one Qwen3 MTP layer is currently supported, got mtp_num_hidden_layers={layers}")
    is_moe = "moe" in text.get("model_type", "") or int(text.get("num_experts", 0) or 0) > 1
    if not is_moe:
        return
    missing = sorted(_required_moe_mtp_keys(layers) - set(tensors))
    if missing:
        raise KeyError("Missing required MoE MTP tensors: " + ", ".join(missing[:20]) + (" ..." if len(missing) > 20 else ""))


def _quantize_stack(stack: torch.Tensor, parts: int, block_size, scale_dtype):
    """[E, parts * R, C] -> per expert and part (codes [R, C], scale_inv [R/bm, C/bn]) on the host, from one launch;
    None when a tile would straddle two parts."""
    bm, bn = block_size
    experts, rows, cols = stack.shape
    if rows % parts or (rows // parts) % bm or cols % bn:
        return None
    kdt = scale_dtype if scale_dtype in (torch.float32, torch.bfloat16, ops.E8M0) else torch.float32
    q, s, _ = ops.quant_fp8_block(stack.to(A.require_gpu()), (bm, bn), scale_mode=A.SCALE_MUL, scale_dtype=kdt)
    q, s = q.cpu(), s.to(scale_dtype).cpu()
    r, sr = rows // parts, rows // parts // bm
    return [[(q[e, p * r:(p + 1) * r].contiguous(), s[e, p * sr:(p + 1) * sr].contiguous()) for p in range(parts)]
            for e in range(experts)]


def _build_mtp_state_dict(tensors, *, block_size, modules_to_not_convert, device, scale_dtype) -> dict[str, torch.Tensor]:
    out: dict[str, torch.Tensor] = {}

    def emit(key, weight, pre=None):
        module = _module_of(key)
        if not _should_convert_module(module, modules_to_not_convert):
            out[key] = weight.cpu()
            return
        q, s = pre if pre is not None else quantize_fp8_blockwise(weight, block_size, device=device, scale_dtype=scale_dtype)
        out[key], out[f"{module}.weight_scale_inv"] = q, s

    for key in sorted(tensors):
        w = tensors[key]
        stacked = {".mlp.experts.gate_up_proj": ("gate_proj", "up_proj"), ".mlp.experts.down_proj": ("down_proj",)}
        names = next((n for suffix, n in stacked.items() if key.endswith(suffix)), None)
        if names is not None:
            base = key[: key.rindex(".")]
            pre = _quantize_stack(w, len(names), block_size, scale_dtype) if w.dim() == 3 else None
            for e, expert in enumerate(w):
                for p, (name, part) in enumerate(zip(names, expert.chunk(len(names), dim=0))):
                    emit(f"{base}.{e}.{name}.weight", part, None if pre is None else pre[e][p])
        elif key.endswith(".weight"):
            emit(key, w)
        else:
            out[key] = w.cpu()
    return out


def _total_size(ckpt_dir: str) -> int:
    total = 0
    for shard in sorted(glob(os.path.join(ckpt_dir, "*.safetensors"))):
        with safe_open(shard, framework="pt", device="cpu") as f:
            for key in f.keys():
                sl = f.get_slice(key)
                dtype = sl.get_dtype()
                if dtype not in _SAFETENSORS_ITEMSIZE:
                    raise ValueError(f"Unknown safetensors dtype {dtype!r}")
                total += math.prod(sl.get_shape()) * _SAFETENSORS_ITEMSIZE[dtype]
    return total


def _current_index(ckpt_dir: str) -> tuple[dict[str, Any], dict[str, str]]:
    path = os.path.join(ckpt_dir, INDEX)
    if os.path.exists(path):
        with open(path) as f:
            index = json.load(f)
        return dict(index.get("metadata", {})), dict(index["weight_map"])
    weight_map = {}
    for shard in sorted(glob(os.path.join(ckpt_dir, "*.safetensors"))):
        if os.path.basename(shard) == MTP_SHARD:
            continue
        with safe_open(shard, framework="pt", device="cpu") as f:
            weight_map.update({key: os.path.basename(shard) for key in f.keys()})
    return {}, weight_map


def append_mtp_weights_to_fp8_checkpoint(input_hf_path: str, output_fp8_path: str, *, block_size: tuple[int, int],
                                         modules_to_not_convert: list[str], device=None,
                                         scale_dtype: torch.dtype = torch.bfloat16) -> int:
    """Returns the number of tensors written to `mtp.safetensors` (0 when the input has no `mtp.*` tensors)."""
    tensors = _read_mtp_tensors(input_hf_path)
    _validate(input_hf_path, tensors)
    if not tensors:
        return 0
    state = _build_mtp_state_dict(tensors, block_size=block_size, modules_to_not_convert=modules_to_not_convert,
                                  device=device, scale_dtype=scale_dtype)
    save_file(state, os.path.join(output_fp8_path, MTP_SHARD))
    metadata, weight_map = _current_index(output_fp8_path)
    weight_map = {k: shard for k, shard in weight_map.items() if not k.startswith("mtp.") and shard != MTP_SHARD}
    weight_map.update({k: MTP_SHARD for k in state})
    metadata["total_size"] = _total_size(output_fp8_path)
    with open(os.path.join(output_fp8_path, INDEX), "w") as f:
        json.dump({"metadata": metadata, "weight_map": weight_map}, f, indent=2, sort_keys=True)
        f.write("\n")
    return len(state)
