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
