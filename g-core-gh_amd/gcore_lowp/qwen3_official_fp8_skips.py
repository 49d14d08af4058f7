"""Which modules of a Qwen3.5 / Qwen3.6 checkpoint stay in bf16 when the rest goes to block-wise FP8: the
`modules_to_not_convert` list that the block-wise quantiser's callers consult (drop-in for
tools/convert_fp8/qwen3_5/qwen3_official_fp8_skips.py; the list matches the FP8 checkpoints published on the hub:
experts and the large projections are quantised; routers, norms, the small GatedDeltaNet weights that are not
128-aligned, the vision tower, the embedding and lm_head are not).  Pure configuration logic, no tensors."""
from __future__ import annotations

import json
import os
from typing import Any

__all__ = ["build_qwen3_official_modules_to_not_convert", "build_qwen3_official_modules_to_not_convert_from_path",
           "load_config_dict", "load_modules_to_not_convert_from_reference"]

# GatedDeltaNet members kept in bf16 (:14-22)
_LINEAR_ATTN_KEPT = ("A_log", "conv1d", "dt_bias", "in_proj_ba", "in_proj_b", "in_proj_a", "norm")
# multi-token-prediction modules kept in bf16 (:24-35)
_MTP_KEPT = ("mtp.layers.0.input_layernorm", "mtp.layers.0.post_attention_layernorm", "mtp.layers.0.mlp.gate",
             "mtp.layers.0.mlp.shared_expert_gate", "mtp.layers.0.self_attn.q_norm", "mtp.layers.0.self_attn.k_norm",
             "mtp.fc", "mtp.norm", "mtp.pre_fc_norm_embedding", "mtp.pre_fc_norm_hidden")


def load_config_dict(config_path: str) -> dict[str, Any]:
    """config.json of a checkpoint directory, or the file itself."""
    if os.path.isdir(config_path):
        config_path = os.path.join(config_path, "config.json")
    with open(config_path) as f:
        return json.load(f)


def load_modules_to_not_convert_from_reference(reference_path: str) -> list[str]:
    """The explicit list of a reference FP8 checkpoint (:47-56); ValueError when it has none."""
    qcfg = load_config_dict(reference_path).get("quantization_config")
    if not qcfg or "modules_to_not_convert" not in qcfg:
        raise ValueError(f"No quantization_config.modules_to_not_convert in {reference_path}")
    modules = qcfg["modules_to_not_convert"]
    if not isinstance(modules, list) or not modules:
        raise ValueError("modules_to_not_convert must be a non-empty list")
    return list(modules)


def _section(value: Any) -> dict[str, Any]:
    if value is None:
        return {}
    if isinstance(value, dict):
        return value
    return value.to_dict() if hasattr(value, "to_dict") else dict(value)


def _layer_types(text: dict[str, Any]) -> list[str]:
    if text.get("layer_types") is not None:
        return list(text["layer_types"])
    every = int(text.get("full_attention_interval", 4))
    return ["full_attention" if (i + 1) % every == 0 else "linear_attention" for i in range(int(text["num_hidden_layers"]))]


def _vision_modules(vision: dict[str, Any]) -> list[str]:
    out = ["visual", "model.visual"]
    n_deepstack = len(vision.get("deepstack_visual_indexes") or []) or 3
    for root in ("model.visual", "visual"):
        out += [f"{root}.patch_embed.proj", f"{root}.pos_embed", f"{root}.merger.linear_fc1", f"{root}.merger.linear_fc2",
                f"{root}.merger.norm"]
        for i in range(n_deepstack):
            out += [f"{root}.deepstack_merger_list.{i}.{leaf}" for leaf in ("linear_fc1", "linear_fc2", "norm")]
    for i in range(int(vision.get("depth", 0))):
        out += [f"model.visual.blocks.{i}.attn.proj", f"model.visual.blocks.{i}.attn.qkv",
                f"model.visual.blocks.{i}.mlp.linear_fc1", f"model.visual.blocks.{i}.mlp.linear_fc2",
                f"visual.blocks.{i}.attn.proj", f"visual.blocks.{i}.attn.qkv_proj",
                f"visual.blocks.{i}.mlp.linear_fc1", f"visual.blocks.{i}.mlp.linear_fc2"]
    return out


def build_qwen3_official_modules_to_not_convert(config: dict[str, Any], *, include_mtp: bool = True,
                                                include_vision: bool | None = None) -> list[str]:
    """:153-212.  `config` is a parsed config.json (vision-language MoE, vision-language dense or text only);
    include_vision None = whenever the config has a vision section."""
    text = _section(config["text_config"]) if "text_config" in config else config
    arch = str((config.get("architectures") or [""])[0])
    nested = "ConditionalGeneration" in arch or "ImageTextToText" in arch or "text_config" in config
    lm = "model.language_model" if nested else "model"
    is_moe = "moe" in text.get("model_type", "") or int(text.get("num_experts", 0) or 0) > 1
    vision = _section(config["vision_config"]) if "vision_config" in config else None
    if include_vision is None:
        include_vision = vision is not None
    kinds = _layer_types(text)
    modules = ["lm_head", "model.embed_tokens"]
    for i in range(int(text["num_hidden_layers"])):
        layer = f"{lm}.layers.{i}"
        modules += [f"{layer}.input_layernorm", f"{layer}.post_attention_layernorm"]
        if is_moe:
            modules += [f"{layer}.mlp.gate", f"{layer}.mlp.shared_expert_gate"]
        if kinds[i] == "linear_attention":
            modules += [f"{layer}.linear_attn.{leaf}" for leaf in _LINEAR_ATTN_KEPT]
        elif kinds[i] in ("full_attention", "sliding_attention"):
            modules += [f"{layer}.self_attn.q_norm", f"{layer}.self_attn.k_norm"]
        else:
            raise ValueError(f"Unknown layer_type[{i}]={kinds[i]!r}")
    if include_mtp:
        modules += _MTP_KEPT
    if include_vision and vision is not None:
        modules += _vision_modules(vision)
    return modules


def build_qwen3_official_modules_to_not_convert_from_path(config_path: str) -> list[str]:
    return build_qwen3_official_modules_to_not_convert(load_config_dict(config_path))
