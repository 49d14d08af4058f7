"""Validation and skip-list rules of the Qwen3 MTP post-processing step (CPU: every case fails or returns before a
kernel would run); cases of tools/convert_fp8/qwen3_5/tests/test_qwen3_mtp_fp8_postprocess.py:177-239."""
import json
import os

import pytest
import torch
from safetensors.torch import save_file

from gcore_lowp import qwen3_mtp_fp8_postprocess as P


def _config(path, layers=1, moe=True):
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump({"text_config": {"model_type": "qwen3_5_moe_text" if moe else "qwen3_5_text",
                                   "num_experts": 2 if moe else 0, "mtp_num_hidden_layers": layers}}, f)


def _dirs(tmp_path):
    src, dst = tmp_path / "in", tmp_path / "out"
    src.mkdir(), dst.mkdir()
    save_file({"model.weight": torch.ones(2, 2, dtype=torch.bfloat16)}, str(dst / "model.safetensors"))
    return str(src), str(dst)


def test_skip_list_rule():
    skip = ["mtp.fc", "mtp.layers.0.mlp.gate", "q_norm", r"mtp\.layers\.\d+\.input_layernorm"]
    assert not P._should_convert_module("mtp.fc", skip)
    assert not P._should_convert_module("mtp.layers.0.mlp.gate", skip)
    assert not P._should_convert_module("mtp.layers.0.self_attn.q_norm", skip)             # suffix
    assert not P._should_convert_module("mtp.layers.3.input_layernorm", skip)              # regex prefix
    assert P._should_convert_module("mtp.layers.0.mlp.shared_expert.gate_proj", skip)
    assert not P._should_convert_module("mtp.fc_extra", skip)                              # prefix match, as the reference
    assert P._should_convert_module("anything", None) and P._should_convert_module("anything", [])
    assert P._module_of("a.b.weight") == "a.b" and P._module_of("a.b.gate_up_proj") == "a.b.gate_up_proj"


def test_required_keys():
    req = P._required_moe_mtp_keys(1)
    assert len(req) == 4 + 15 and "mtp.layers.0.mlp.experts.gate_up_proj" in req and "mtp.fc.weight" in req


def test_missing_required_tensors(tmp_path):
    src, dst = _dirs(tmp_path)
    _config(src)
    save_file({"mtp.fc.weight": torch.ones(4, 8, dtype=torch.bfloat16)}, os.path.join(src, "bad.safetensors"))
    with pytest.raises(KeyError, match="Missing required MoE MTP tensors"):
        P.append_mtp_weights_to_fp8_checkpoint(src, dst, block_size=(2, 2), modules_to_not_convert=[], device="cpu")


def test_mtp_enabled_without_tensors(tmp_path):
    src, dst = _dirs(tmp_path)
    _config(src)
    with pytest.raises(ValueError, match="no top-level mtp"):
        P.append_mtp_weights_to_fp8_checkpoint(src, dst, block_size=(2, 2), modules_to_not_convert=[], device="cpu")


def test_several_mtp_layers(tmp_path):
    src, dst = _dirs(tmp_path)
    _config(src, layers=2)
    save_file({"mtp.fc.weight": torch.ones(4, 8, dtype=torch.bfloat16)}, os.path.join(src, "in.safetensors"))
    with pytest.raises(NotImplementedError):
        P.append_mtp_weights_to_fp8_checkpoint(src, dst, block_size=(2, 2), modules_to_not_convert=[], device="cpu")


def test_no_mtp_configured_and_none_present(tmp_path):
    src, dst = _dirs(tmp_path)
    _config(src, layers=0)
    save_file({"model.weight": torch.ones(2, 2, dtype=torch.bfloat16)}, os.path.join(src, "in.safetensors"))
    assert P.append_mtp_weights_to_fp8_checkpoint(src, dst, block_size=(2, 2), modules_to_not_convert=[]) == 0
    assert not os.path.exists(os.path.join(dst, "mtp.safetensors"))


def test_total_size_and_index_scan(tmp_path):
    d = tmp_path / "ck"
    d.mkdir()
    save_file({"a": torch.zeros(3, 5, dtype=torch.bfloat16), "b": torch.zeros(7, dtype=torch.float32)}, str(d / "x.safetensors"))
    save_file({"c": torch.zeros(4, 4).to(torch.float8_e4m3fn)}, str(d / "mtp.safetensors"))
    assert P._total_size(str(d)) == 30 + 28 + 16
    meta, wm = P._current_index(str(d))
    assert meta == {} and wm == {"a": "x.safetensors", "b": "x.safetensors"}            # the MTP shard is rebuilt, not scanned


def _qwen36_moe_vl_config():
    kinds = ["linear_attention" if (i + 1) % 4 else "full_attention" for i in range(40)]
    return {"architectures": ["Qwen3_5MoeForConditionalGeneration"],
            "text_config": {"model_type": "qwen3_5_moe_text", "num_hidden_layers": 40, "num_experts": 256, "layer_types": kinds},
            "vision_config": {"depth": 27, "deepstack_visual_indexes": []}}


def test_official_skip_list(tmp_path):
    """The cases of tools/convert_fp8/qwen3_5/tests/test_qwen3_official_fp8_skips.py: 648 entries for the
    Qwen3.6-35B-A3B structure, seven per linear-attention layer (never the large projections), q/k norms per
    full-attention layer, `model.` prefix for a text-only model, round trip of a reference list."""
    from gcore_lowp import qwen3_official_fp8_skips as S
    cfg = _qwen36_moe_vl_config()
    modules = S.build_qwen3_official_modules_to_not_convert(cfg)
    assert len(modules) == 648 and len(set(modules)) == 648
    kinds = cfg["text_config"]["layer_types"]
    for i, kind in enumerate(kinds):
        layer = f"model.language_model.layers.{i}."
        if kind == "linear_attention":
            hits = [m for m in modules if m.startswith(layer + "linear_attn.")]
            assert len(hits) == 7 and not any(x in m for m in hits for x in ("in_proj_qkv", "in_proj_z", "out_proj"))
        else:
            assert layer + "self_attn.q_norm" in modules and layer + "self_attn.k_norm" in modules
        assert layer + "mlp.gate" in modules and layer + "mlp.shared_expert_gate" in modules
    assert sum(k == "linear_attention" for k in kinds) == 30
    text_only = {"architectures": ["Qwen3_5ForCausalLM"], "model_type": "qwen3_5_text", "num_hidden_layers": 4,
                 "layer_types": ["linear_attention"] * 3 + ["full_attention"]}
    modules = S.build_qwen3_official_modules_to_not_convert(text_only, include_mtp=False, include_vision=False)
    assert any(m.startswith("model.layers.0.linear_attn.") for m in modules) and not any("language_model" in m for m in modules)
    assert not any(m.startswith("mtp.") for m in modules) and not any(".mlp.gate" in m for m in modules)
    # layer kinds from the interval when the config does not list them
    by_interval = S.build_qwen3_official_modules_to_not_convert({"num_hidden_layers": 8, "model_type": "qwen3_5_text"},
                                                                 include_mtp=False)
    assert "model.layers.3.self_attn.q_norm" in by_interval and "model.layers.7.self_attn.k_norm" in by_interval
    assert "model.layers.2.linear_attn.conv1d" in by_interval
    with pytest.raises(ValueError, match="Unknown layer_type"):
        S.build_qwen3_official_modules_to_not_convert({"num_hidden_layers": 1, "layer_types": ["mamba"]})
    ref = tmp_path / "ref.json"
    ref.write_text(json.dumps({"quantization_config": {"modules_to_not_convert": ["lm_head", "model.layers.0.mlp.gate"]}}))
    assert S.load_modules_to_not_convert_from_reference(str(ref)) == ["lm_head", "model.layers.0.mlp.gate"]
    ref.write_text(json.dumps({"quantization_config": {}}))
    with pytest.raises(ValueError):
        S.load_modules_to_not_convert_from_reference(str(ref))
    # the list drives the MTP step's decision
    assert not P._should_convert_module("mtp.fc", S.build_qwen3_official_modules_to_not_convert(cfg))
    assert P._should_convert_module("mtp.layers.0.self_attn.q_proj", S.build_qwen3_official_modules_to_not_convert(cfg))
