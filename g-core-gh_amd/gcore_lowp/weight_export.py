"""MI355X drop-in for the per-tensor part of gpatch_v4/models/deepseek_v4/weight_export.py: one model tensor ->
the disk-format checkpoint tensors it becomes (key renaming, per-expert split, dtype class, quantisation).

The quantising classes run on the HIP kernels of this package (FP4 e2m1 1 x 32 for routed experts, e4m3fn
128 x 128 with power-of-two scales for the FP8 whitelist), on the bf16 view of the master weight, as in the
reference.  What is not here is the gathering of sharded parameters (DTensor / expert-parallel all-gather,
weight_export.py:329-408): this build runs on one GPU, so `export_deepseek_v4_weights_for_vllm` walks a plain
`state_dict()` and refuses sharded tensors.
"""
from __future__ import annotations

import re
from collections.abc import Iterator
from typing import Literal

import torch
from torch.nn import Module

from .eager_quant_kernels import quant_fp4_e2m1_scale_e8m0_packed, quant_fp8_e4m3_scale_e8m0

# ------------------------------------------------------------------------------------------------------------
# dtype class of a disk key (weight_export.py:55-122).  FP8 is an explicit whitelist: a shape heuristic would also
# quantise embed / head / compressor linears, which the checkpoint format keeps in bf16.
_LAYER, _MTP = r"^(?:.*\.)?layers\.\d+\.", r"^mtp\.\d+\."
_FP8_TAILS = (r"attn\.(?:wq_a|wq_b|wkv|wo_a|wo_b)\.weight$", r"attn\.indexer\.wq_b\.weight$",
              r"ffn\.shared_experts\.w[123]\.weight$")
_FP8_DISK_KEY_PATTERNS: tuple[str, ...] = tuple(
    [_LAYER + tail for tail in _FP8_TAILS] + [_MTP + tail for tail in _FP8_TAILS]
    + [r"^mtp\.\d+\.(?:e_proj|h_proj)\.weight$", r"^mtp\.0\.main_proj\.weight$"])
_FP8_DISK_KEY_RE = re.compile("|".join(_FP8_DISK_KEY_PATTERNS))

_F32_TAILS = (r"attn\.attn_sink$", r"attn\.(?:.*\.)?compressor\.ape$", r"ffn\.gate\.bias$")
_F32_DISK_KEY_PATTERNS: tuple[str, ...] = tuple(
    [r"^(?:.*\.)?hc_(?:attn|ffn|head)_(?:fn|base|scale)$"] + [_LAYER + tail for tail in _F32_TAILS]
    + [_MTP + tail for tail in _F32_TAILS])
_F32_DISK_KEY_RE = re.compile("|".join(_F32_DISK_KEY_PATTERNS))

_WO_A_DISK_KEY_RE = re.compile(r"^(?:.*\.)?layers\.\d+\.attn\.wo_a\.weight$|^mtp\.\d+\.attn\.wo_a\.weight$")
_EXPERT_DISK_KEY_RE = re.compile(r"\.experts\.\d+\.w[123]\.weight$")


def _classify_for_save(name: str, t: torch.Tensor, *, is_sgl_ckpt_fmt: bool = False) -> str:
    """(:104-122) int_passthrough | fp4_expert | fp8_e4m3 | f32_passthrough | bf16_passthrough.  The wo_a rule of
    the SGLang-format checkpoint (stored dequantised, bf16) must come before the FP8 whitelist, which also
    matches wo_a."""
    if not t.dtype.is_floating_point:
        return "int_passthrough"
    if _EXPERT_DISK_KEY_RE.search(name) is not None:
        return "fp4_expert"
    if is_sgl_ckpt_fmt and _WO_A_DISK_KEY_RE.search(name) is not None:
        return "bf16_passthrough"
    if _FP8_DISK_KEY_RE.search(name) is not None:
        return "fp8_e4m3"
    if _F32_DISK_KEY_RE.search(name) is not None:
        return "f32_passthrough"
    return "bf16_passthrough"


def resolve_dsv4_export_dtypes(config) -> tuple[str, bool]:
    """(:125-135) (expert_dtype, is_sgl_ckpt_fmt); experts default to fp8 for an SGLang-format checkpoint, else fp4."""
    is_sgl_ckpt_fmt = bool(getattr(config, "is_sgl_ckpt_fmt", False))
    expert_dtype = getattr(config, "expert_dtype", None)
    if expert_dtype is None:
        expert_dtype = "fp8" if is_sgl_ckpt_fmt else "fp4"
    assert expert_dtype in ("fp4", "fp8"), f"Unsupported DeepSeek-V4 expert_dtype={expert_dtype!r}"
    return expert_dtype, is_sgl_ckpt_fmt


def _scale_key(weight_disk_key: str) -> str:
    assert weight_disk_key.endswith(".weight"), weight_disk_key
    return weight_disk_key[:-len(".weight")] + ".scale"


# ------------------------------------------------------------------------------------------------------------
# model key -> disk key (weight_export.py:143-246).  Rules are tried in order and re-applied until none fires;
# the specific ones come before the two catch-alls (self_attn -> attn, mlp -> ffn) that they feed.
_L = r"^layers\.(\d+)\."


def _rules():
    r = [(r"^embed_tokens\.weight$", "embed.weight"), (r"^lm_head\.weight$", "head.weight")]
    r += [(rf"^hc_head\.hc_{x}$", f"hc_head_{x}") for x in ("fn", "base", "scale")]
    for hc in ("attn", "ffn"):
        r += [(_L + rf"{hc}_hc\.{x}$", rf"layers.\1.hc_{hc}_{x}") for x in ("fn", "base", "scale")]
    r += [(_L + r"hc_head\.hc_(fn|base|scale)$", r"layers.\1.hc_head_\2"),
          (_L + r"input_layernorm\.", r"layers.\1.attn_norm."),
          (_L + r"post_attention_layernorm\.", r"layers.\1.ffn_norm.")]
    ci = r"self_attn\.compressor\.indexer\."
    r += [(_L + ci + r"kv_proj\.", r"layers.\1.self_attn.indexer.compressor.wkv."),
          (_L + ci + r"gate_proj\.", r"layers.\1.self_attn.indexer.compressor.wgate."),
          (_L + ci + r"kv_norm\.", r"layers.\1.self_attn.indexer.compressor.norm."),
          (_L + ci + r"_position_bias_holder\.weight$", r"layers.\1.self_attn.compressor.indexer.position_bias"),
          (_L + ci + r"position_bias$", r"layers.\1.self_attn.indexer.compressor.ape"),
          (_L + ci + r"q_b_proj\.", r"layers.\1.self_attn.indexer.wq_b."),
          (_L + ci + r"weights_proj\.", r"layers.\1.self_attn.indexer.weights_proj.")]
    c = r"self_attn\.compressor\."
    r += [(_L + c + r"kv_proj\.", r"layers.\1.self_attn.compressor.wkv."),
          (_L + c + r"gate_proj\.", r"layers.\1.self_attn.compressor.wgate."),
          (_L + c + r"kv_norm\.", r"layers.\1.self_attn.compressor.norm."),
          (_L + c + r"_position_bias_holder\.weight$", r"layers.\1.self_attn.compressor.position_bias"),
          (_L + c + r"position_bias$", r"layers.\1.self_attn.compressor.ape")]
    for src, dst in (("q_a_proj", "wq_a"), ("q_b_proj", "wq_b"), ("kv_proj", "wkv"), ("o_a_proj", "wo_a"),
                     ("o_b_proj", "wo_b"), ("q_a_norm", "q_norm")):
        r.append((_L + rf"self_attn\.{src}\.", rf"layers.\1.self_attn.{dst}."))
    r += [(_L + r"self_attn\._sink_holder\.weight$", r"layers.\1.self_attn.sinks"),
          (_L + r"self_attn\.sinks$", r"layers.\1.self_attn.attn_sink"),
          (_L + r"mlp\.gate\.e_score_correction_bias$", r"layers.\1.mlp.gate.bias")]
    for src, dst in (("gate_proj", "w1"), ("down_proj", "w2"), ("up_proj", "w3")):
        r.append((_L + rf"mlp\.shared_experts\.{src}\.", rf"layers.\1.mlp.shared_experts.{dst}."))
    r += [(_L + r"self_attn\.", r"layers.\1.attn."), (_L + r"mlp\.", r"layers.\1.ffn.")]
    return tuple((re.compile(a), b) for a, b in r)


_MODEL_TO_DISK_RENAMES_COMPILED = _rules()
_EXPERT_STACKED_KEY_RE = re.compile(r"^(layers|mtp\.layers)\.(\d+)\.mlp\.experts\.(gate_up_proj|down_proj)$")
_MTP_LAYER_KEY_RE = re.compile(r"^mtp\.layers\.(\d+)\.(.+)$")


def _model_key_to_disk_key(model_key: str) -> str:
    for _ in range(8):
        for rgx, repl in _MODEL_TO_DISK_RENAMES_COMPILED:
            new_key, n = rgx.subn(repl, model_key, count=1)
            if n:
                model_key = new_key
                break
        else:
            return model_key
    raise AssertionError(f"_model_key_to_disk_key did not converge on {model_key!r}")


def _model_to_disk_key(model_key: str) -> str:
    """(:236-243) MTP layers are renamed as if they were layer `depth`, then moved under mtp.<depth>."""
    m = _MTP_LAYER_KEY_RE.match(model_key)
    if m is None:
        return _model_key_to_disk_key(model_key)
    depth = int(m.group(1))
    return _model_key_to_disk_key(f"layers.{depth}.{m.group(2)}").replace(f"layers.{depth}.", f"mtp.{depth}.", 1)


def _split_per_expert(model_key: str, t: torch.Tensor) -> dict[str, torch.Tensor]:
    """(:205-233) stacked expert parameters -> one tensor per expert: down_proj[i] -> w2, the two halves of
    gate_up_proj[i] along dim 1 -> w1, w3; anything else passes as it is."""
    m = _EXPERT_STACKED_KEY_RE.match(model_key)
    if m is None:
        assert ".experts." not in model_key or ".shared_experts." in model_key, (
            f"unexpected expert key not handled by _split_per_expert: {model_key!r}")
        return {model_key: t}
    prefix, layer, kind = m.groups()
    base = f"{prefix}.{layer}.mlp.experts."
    if kind == "down_proj":
        return {f"{base}{i}.w2.weight": t[i].contiguous() for i in range(t.shape[0])}
    assert t.shape[1] % 2 == 0, f"{model_key} shape {tuple(t.shape)} not divisible by 2 on dim=1 (cannot split into w1/w3)"
    w1, w3 = t.chunk(2, dim=1)
    out: dict[str, torch.Tensor] = {}
    for i in range(t.shape[0]):
        out[f"{base}{i}.w1.weight"] = w1[i].contiguous()
        out[f"{base}{i}.w3.weight"] = w3[i].contiguous()
    return out


def iter_disk_checkpoint_tensors(model_key: str, tensor: torch.Tensor, *,
                                 dtype_format: Literal["quantized", "bf16"] = "quantized",
                                 expert_dtype: Literal["fp4", "fp8"] = "fp4", is_sgl_ckpt_fmt: bool = False,
                                 include_mtp: bool = True) -> Iterator[tuple[str, torch.Tensor]]:
    """(:246-326) One model tensor -> its disk-format tensors.  "quantized": experts to packed e2m1 + e8m0 1 x 32
    (or e4m3fn when expert_dtype is fp8), the FP8 whitelist to e4m3fn + e8m0 128 x 128, each followed by its
    `.scale`; both from the bf16 view of the master so that group scales flip together with the QAT forward.
    "bf16": the same keys, quantisable weights left as they are for the receiver to quantise."""
    for mk, mv in _split_per_expert(model_key, tensor).items():
        if not include_mtp and mk.startswith("mtp."):
            continue
        disk_key = _model_to_disk_key(mk)
        cls = _classify_for_save(disk_key, mv, is_sgl_ckpt_fmt=is_sgl_ckpt_fmt)
        if cls == "fp4_expert" and expert_dtype == "fp8":
            cls = "fp8_e4m3"
        if cls == "int_passthrough":
            yield disk_key, mv
        elif cls == "f32_passthrough":
            yield disk_key, mv.to(torch.float32)
        elif cls == "bf16_passthrough":
            yield disk_key, mv.to(torch.bfloat16)
        elif cls not in ("fp4_expert", "fp8_e4m3"):
            raise RuntimeError(f"unhandled save class {cls!r} for {disk_key}")
        elif dtype_format != "quantized":
            yield disk_key, mv
        else:
            quant = quant_fp4_e2m1_scale_e8m0_packed if cls == "fp4_expert" else quant_fp8_e4m3_scale_e8m0
            q, scale = quant(mv.bfloat16().float())
            yield disk_key, q
            yield _scale_key(disk_key), scale


def export_deepseek_v4_weights_for_vllm(model: Module, *, dtype_format: Literal["quantized", "bf16"] = "bf16"):
    """(:411-434) Disk-format tensors of a whole model for a weight reload, on the GPU.  One-GPU build: the
    parameters must be plain tensors (the reference gathers DTensor / expert-parallel shards first)."""
    expert_dtype, is_sgl_ckpt_fmt = resolve_dsv4_export_dtypes(model.config)
    for name, tensor in model.state_dict().items():
        if name.startswith("mtp."):
            continue
        if type(tensor).__name__ == "DTensor":
            raise NotImplementedError("sharded parameters (DTensor) need the multi-GPU gather, which this build does not have")
        for disk_key, disk_tensor in iter_disk_checkpoint_tensors(
                name.removeprefix("model."), tensor.detach(), dtype_format=dtype_format, expert_dtype=expert_dtype,
                is_sgl_ckpt_fmt=is_sgl_ckpt_fmt, include_mtp=False):
            yield disk_key, (disk_tensor if disk_tensor.is_cuda else disk_tensor.cuda()).contiguous()


def export_deepseek_v4_bf16_weights(model: Module):
    """(:437-439) bf16 disk-format tensors, quantised by the receiver."""
    yield from export_deepseek_v4_weights_for_vllm(model, dtype_format="bf16")


def export_deepseek_v4_quantized_weights(model: Module):
    """(:442-443) pre-quantised disk-format tensors."""
    yield from export_deepseek_v4_weights_for_vllm(model, dtype_format="quantized")
