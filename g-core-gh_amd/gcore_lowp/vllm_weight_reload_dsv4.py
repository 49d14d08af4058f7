"""Worker-side quantisation of a DeepSeek-V4 bf16 weight bucket before it is loaded into a live vLLM model;
MI355X drop-in for the quantising part of
gpatch_v4/generation_backend/vllm_model_specific/vllm_weight_reload_dsv4.py (:35-74 rename table, :324-353 and
:814-840 name variants, :1050-1126 module reflection, :1129-1178 iter_model_aware_quantized_weights).

Routed-expert weights are always quantised (packed FP4 with 1 x 32 e8m0 scales, or e4m3 with 128 x 128 e8m0
scales, by `expert_dtype`); any other `.weight` is quantised to e4m3 only when the module that owns it in the live
model is a vLLM linear layer whose weight is stored as e4m3.  Both quantisers are single HIP kernel launches on the
tensor's device.  Loading the result into vLLM parameters, MoE parameter surgery and sleep / wake-up stay with
vLLM's worker and are not part of this module.
"""
from __future__ import annotations

import re
from collections.abc import Iterable

import torch
from torch import nn

from .eager_quant_kernels import quant_fp4_e2m1_scale_e8m0_packed, quant_fp8_e4m3_scale_e8m0

__all__ = ["DSV4_EXPERT_WEIGHT_RE", "DSV4_VLLM_LOAD_RENAMES", "apply_shared_expert_alias", "base_reload_name_variants",
           "candidate_param_names_for_reflection", "get_module_from_param_name", "iter_model_aware_quantized_weights",
           "loaded_name_candidates", "map_checkpoint_key_to_vllm_param_name", "module_from_param_name",
           "with_model_prefix_variants"]

_MEGA_MOE_CLS = "DeepseekV4MegaMoEExperts"
_LAYER = r"^(layers\.\d+)\."

# checkpoint key -> name of the (often fused) vLLM parameter that receives it
DSV4_VLLM_LOAD_RENAMES: tuple[tuple[re.Pattern[str], str], ...] = tuple((re.compile(a), b) for a, b in (
    (r"^embed\.weight$", "embed_tokens.weight"),
    (r"^head\.weight$", "lm_head.weight"),
    (_LAYER + r"attn\.(?:wq_a|wkv)\.weight$", r"\1.attn.fused_wqa_wkv.weight"),
    (_LAYER + r"attn\.(?:wq_a|wkv)\.scale$", r"\1.attn.fused_wqa_wkv.weight_scale_inv"),
    (_LAYER + r"attn\.compressor\.(?:wkv|wgate)\.weight$", r"\1.attn.mla_attn.compressor.fused_wkv_wgate.weight"),
    (_LAYER + r"attn\.compressor\.norm\.weight$", r"\1.attn.mla_attn.compressor.norm.weight"),
    (_LAYER + r"attn\.compressor\.ape$", r"\1.attn.mla_attn.compressor.ape"),
    (_LAYER + r"attn\.indexer\.compressor\.(?:wkv|wgate)\.weight$", r"\1.attn.indexer.compressor.fused_wkv_wgate.weight"),
    (_LAYER + r"ffn\.experts\.\d+\.w[13]\.weight$", r"\1.ffn.experts.w13_weight"),
    (_LAYER + r"ffn\.experts\.\d+\.w2\.weight$", r"\1.ffn.experts.w2_weight"),
))
DSV4_EXPERT_WEIGHT_RE = re.compile(r"^layers\.\d+\.ffn\.experts\.\d+\.w[123]\.weight$")


def _unique(names: Iterable[str]) -> list[str]:
    return list(dict.fromkeys(names))


def apply_shared_expert_alias(name: str, *, include_gate_up: bool) -> str:
    """shared_experts.w1 / w3 -> gate_up_proj (only when asked), w2 -> down_proj; a trailing `.scale` becomes
    `.weight_scale_inv`."""
    if include_gate_up and ".shared_experts.w1" in name:
        name = name.replace(".shared_experts.w1", ".shared_experts.gate_up_proj", 1)
    elif include_gate_up and ".shared_experts.w3" in name:
        name = name.replace(".shared_experts.w3", ".shared_experts.gate_up_proj", 1)
    elif ".shared_experts.w2" in name:
        name = name.replace(".shared_experts.w2", ".shared_experts.down_proj", 1)
    if name.endswith(".scale"):
        name = name[: -len(".scale")] + ".weight_scale_inv"
    return name


def map_checkpoint_key_to_vllm_param_name(model: nn.Module, name: str) -> str:
    """The model's own `hf_to_vllm_mapper` if it has one, else the built-in rules."""
    map_name = getattr(getattr(model, "hf_to_vllm_mapper", None), "_map_name", None)
    if callable(map_name):
        mapped = map_name(name)
        if mapped is not None:
            return str(mapped)
    mapped = apply_shared_expert_alias(name.removeprefix("model."), include_gate_up=False)
    if mapped.startswith(("layers.", "embed.")):
        return f"model.{mapped}"
    return "lm_head.weight" if mapped == "head.weight" else mapped


def base_reload_name_variants(name: str) -> list[str]:
    raw = name.removeprefix("model.")
    out = [name, raw]
    for rgx, repl in DSV4_VLLM_LOAD_RENAMES:
        renamed, hits = rgx.subn(repl, raw, count=1)
        if hits:
            out.append(renamed)
    return _unique(out)


def with_model_prefix_variants(names: Iterable[str]) -> list[str]:
    out: list[str] = []
    for n in names:
        out.append(n)
        if not n.startswith("model."):
            out.append(f"model.{n}")
    return _unique(out)


def loaded_name_candidates(name: str) -> set[str]:
    """Names under which vLLM's `load_weights` may report that checkpoint key `name` was loaded (:843-861): every
    variant with and without the `model.` prefix, and for a `.scale` key also `.weight_scale` / `.weight_scale_inv`."""
    base = base_reload_name_variants(name)
    out = set(with_model_prefix_variants(base))
    for b in base:
        if b.endswith(".scale"):
            stem = b[: -len(".scale")]
            for alias in (f"{stem}.weight_scale", f"{stem}.weight_scale_inv"):
                out.add(alias)
                if not alias.startswith("model."):
                    out.add(f"model.{alias}")
    return out


def candidate_param_names_for_reflection(model: nn.Module, name: str) -> list[str]:
    """Every parameter path under which the live model may hold checkpoint key `name`, most direct first."""
    raw = name.removeprefix("model.")
    out = [raw, map_checkpoint_key_to_vllm_param_name(model, raw)]
    alias = apply_shared_expert_alias(raw, include_gate_up=True)
    if alias != raw:
        out += [alias, map_checkpoint_key_to_vllm_param_name(model, alias)]
    for renamed in base_reload_name_variants(raw):
        if renamed != raw:
            out += [renamed, map_checkpoint_key_to_vllm_param_name(model, renamed)]
    return with_model_prefix_variants(_unique(out))


def _class_names(obj) -> set[str]:
    return {c.__name__ for c in type(obj).__mro__}


def _is_moe_module_for_reload(module) -> bool:
    if module is None:
        return False
    if type(module).__name__ == _MEGA_MOE_CLS:
        return True
    try:
        from vllm.model_executor.layers.fused_moe import FusedMoE
    except ImportError:
        return "FusedMoE" in _class_names(module)
    return isinstance(module, FusedMoE)


def _is_vllm_linear_module(module) -> bool:
    """vLLM's LinearBase; without vLLM in the process (unit tests), a class of that name in the module's bases."""
    if module is None:
        return False
    try:
        from vllm.model_executor.layers.linear import LinearBase
    except ImportError:
        return "LinearBase" in _class_names(module)
    return isinstance(module, LinearBase)


def _module_weight_dtype(module) -> torch.dtype | None:
    for attr in ("weight", "w13_weight", "w2_weight"):
        w = getattr(module, attr, None) if module is not None else None
        if w is not None and hasattr(w, "dtype"):
            return w.dtype
    return None


def module_from_param_name(model: nn.Module, param_name: str) -> nn.Module | None:
    """Walks the dotted path down to the module that owns the parameter; a fused-MoE module on the way owns
    everything below it."""
    here: object = model
    for part in param_name.split(".")[:-1]:
        if _is_moe_module_for_reload(here):
            return here
        try:
            here = here[int(part)] if isinstance(here, nn.ModuleList) else getattr(here, part)
        except (AttributeError, IndexError, ValueError):
            return None
    return here if isinstance(here, nn.Module) else None


def get_module_from_param_name(model: nn.Module, name: str) -> nn.Module | None:
    if hasattr(model, "runnable") and "ACLGraphWrapper" in type(model).__name__:
        model = model.runnable
    for cand in candidate_param_names_for_reflection(model, name):
        module = module_from_param_name(model, cand)
        if module is not None:
            return module
    return None


def _as_bf16_values(t: torch.Tensor) -> torch.Tensor:
    # the bf16 view of the weight, not the fp32 master: scales then agree with the trainer's fake-quantised forward
    # (vllm_weight_reload_dsv4.py:1156-1158).  The kernels read bf16 and compute in fp32, so the reference's
    # widening back to fp32 would only add a pass over the tensor.
    return t.bfloat16()


def iter_model_aware_quantized_weights(model: nn.Module, weights: Iterable[tuple[str, torch.Tensor]], *,
                                       expert_dtype: str) -> list[tuple[str, torch.Tensor]]:
    """[(key, tensor)] of one bf16 bucket -> the same keys with quantised payloads, each followed by its
    `<prefix>.scale` (e8m0).  A `.scale` key in the input is a RuntimeError: the bucket must be unquantised."""
    out: list[tuple[str, torch.Tensor]] = []
    for name, tensor in weights:
        if name.endswith(".scale"):
            raise RuntimeError(f"DSV4 worker-side quantization expects bf16 weight keys, got scale key {name!r}")
        is_expert = DSV4_EXPERT_WEIGHT_RE.match(name) is not None
        if is_expert:
            assert name.endswith(".weight"), name
        to_fp8 = False
        if not is_expert and name.endswith(".weight"):
            module = get_module_from_param_name(model, name)
            to_fp8 = _is_vllm_linear_module(module) and _module_weight_dtype(module) == torch.float8_e4m3fn
        if not (is_expert or to_fp8):
            out.append((name, tensor.contiguous()))
            continue
        if is_expert and expert_dtype == "fp4":
            codes, scale = quant_fp4_e2m1_scale_e8m0_packed(_as_bf16_values(tensor))
        else:
            codes, scale = quant_fp8_e4m3_scale_e8m0(_as_bf16_values(tensor))
        out.append((name, codes.contiguous()))
        out.append((name[: -len(".weight")] + ".scale", scale.contiguous()))
    return out
