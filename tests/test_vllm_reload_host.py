"""Host logic of the worker-side quantisation for vLLM weight reload (CPU only, the quantisers are stand-ins):
name variants, reflection of the live model and the routing of every key
(gpatch_v4/generation_backend/vllm_model_specific/vllm_weight_reload_dsv4.py:324-353,814-840,1082-1178)."""
from unittest.mock import patch

import pytest
import torch
from torch import nn

from gcore_lowp import vllm_weight_reload_dsv4 as R


class LinearBase(nn.Module):                     # stands in for vLLM's class of the same name (matched by name)
    def __init__(self, dtype):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(2, 2).to(dtype), requires_grad=False)


class FusedMoE(nn.Module):
    def __init__(self):
        super().__init__()
        self.w13_weight = nn.Parameter(torch.zeros(1, dtype=torch.uint8), requires_grad=False)


class _Attn(nn.Module):
    def __init__(self):
        super().__init__()
        self.fused_wqa_wkv = LinearBase(torch.float8_e4m3fn)     # fp8 linear reached through a rename
        self.wq_b = LinearBase(torch.float8_e4m3fn)
        self.wo_b = LinearBase(torch.bfloat16)                   # linear, but kept in bf16
        self.norm = nn.LayerNorm(2)                              # not a linear layer


class _Ffn(nn.Module):
    def __init__(self):
        super().__init__()
        self.experts = FusedMoE()
        self.shared_experts = nn.Module()
        self.shared_experts.gate_up_proj = LinearBase(torch.float8_e4m3fn)
        self.shared_experts.down_proj = LinearBase(torch.float8_e4m3fn)


class _Layer(nn.Module):
    def __init__(self):
        super().__init__()
        self.attn, self.ffn = _Attn(), _Ffn()


class _Model(nn.Module):
    def __init__(self):
        super().__init__()
        self.model = nn.Module()
        self.model.layers = nn.ModuleList([_Layer()])
        self.lm_head = LinearBase(torch.bfloat16)


def test_name_variants():
    m = _Model()
    assert R.apply_shared_expert_alias("layers.0.ffn.shared_experts.w1.scale", include_gate_up=True) == \
        "layers.0.ffn.shared_experts.gate_up_proj.weight_scale_inv"
    assert R.apply_shared_expert_alias("layers.0.ffn.shared_experts.w1.weight", include_gate_up=False) == \
        "layers.0.ffn.shared_experts.w1.weight"
    assert R.apply_shared_expert_alias("layers.0.ffn.shared_experts.w2.weight", include_gate_up=False) == \
        "layers.0.ffn.shared_experts.down_proj.weight"
    assert R.map_checkpoint_key_to_vllm_param_name(m, "head.weight") == "lm_head.weight"
    assert R.map_checkpoint_key_to_vllm_param_name(m, "embed.weight") == "model.embed.weight"
    assert R.map_checkpoint_key_to_vllm_param_name(m, "model.layers.1.attn.wq_b.weight") == "model.layers.1.attn.wq_b.weight"
    assert R.base_reload_name_variants("model.layers.3.attn.wkv.weight") == [
        "model.layers.3.attn.wkv.weight", "layers.3.attn.wkv.weight", "layers.3.attn.fused_wqa_wkv.weight"]
    assert R.base_reload_name_variants("layers.3.ffn.experts.7.w3.weight")[-1] == "layers.3.ffn.experts.w13_weight"
    assert R.base_reload_name_variants("layers.3.ffn.experts.7.w2.weight")[-1] == "layers.3.ffn.experts.w2_weight"
    assert R.base_reload_name_variants("layers.3.attn.wq_a.scale")[-1] == "layers.3.attn.fused_wqa_wkv.weight_scale_inv"
    assert R.with_model_prefix_variants(["a.b", "model.c", "a.b"]) == ["a.b", "model.a.b", "model.c"]
    cands = R.candidate_param_names_for_reflection(m, "layers.0.attn.wkv.weight")
    assert cands[0] == "layers.0.attn.wkv.weight" and "model.layers.0.attn.fused_wqa_wkv.weight" in cands
    assert len(cands) == len(set(cands))
    # a mapper on the model takes precedence
    m.hf_to_vllm_mapper = type("M", (), {"_map_name": staticmethod(lambda n: "mapped." + n)})()
    assert R.map_checkpoint_key_to_vllm_param_name(m, "head.weight") == "mapped.head.weight"


def test_module_reflection():
    m = _Model()
    layer = m.model.layers[0]
    assert R.get_module_from_param_name(m, "layers.0.attn.wq_b.weight") is layer.attn.wq_b
    assert R.get_module_from_param_name(m, "layers.0.attn.wkv.weight") is layer.attn.fused_wqa_wkv
    assert R.get_module_from_param_name(m, "layers.0.ffn.shared_experts.w3.weight") is layer.ffn.shared_experts.gate_up_proj
    assert R.get_module_from_param_name(m, "layers.0.ffn.shared_experts.w2.weight") is layer.ffn.shared_experts.down_proj
    assert R.get_module_from_param_name(m, "layers.0.ffn.experts.5.w1.weight") is layer.ffn.experts   # the MoE owns it
    assert R.get_module_from_param_name(m, "head.weight") is m.lm_head
    assert R.get_module_from_param_name(m, "layers.9.attn.wq_b.weight") is None
    assert R.module_from_param_name(m, "model.layers.x.attn.wq_b.weight") is None


@pytest.mark.parametrize("expert_dtype", ["fp4", "fp8"])
def test_routing(expert_dtype):
    m = _Model()
    calls = []

    def fake_fp8(t):
        calls.append(("fp8", t.dtype))
        return torch.full((1,), 8, dtype=torch.uint8), torch.full((1,), 1, dtype=torch.uint8)

    def fake_fp4(t):
        calls.append(("fp4", t.dtype))
        return torch.full((1,), 4, dtype=torch.uint8), torch.full((1,), 1, dtype=torch.uint8)

    w = torch.ones(4, 4)
    bucket = [("layers.0.ffn.experts.3.w1.weight", w), ("layers.0.attn.wq_b.weight", w), ("layers.0.attn.wkv.weight", w),
              ("layers.0.attn.wo_b.weight", w), ("layers.0.attn.norm.weight", w), ("layers.0.attn.attn_sink", w),
              ("head.weight", w), ("layers.0.ffn.shared_experts.w1.weight", w)]
    with patch.object(R, "quant_fp8_e4m3_scale_e8m0", fake_fp8), patch.object(R, "quant_fp4_e2m1_scale_e8m0_packed", fake_fp4):
        out = R.iter_model_aware_quantized_weights(m, bucket, expert_dtype=expert_dtype)
    names = [n for n, _ in out]
    assert names == ["layers.0.ffn.experts.3.w1.weight", "layers.0.ffn.experts.3.w1.scale",
                     "layers.0.attn.wq_b.weight", "layers.0.attn.wq_b.scale",
                     "layers.0.attn.wkv.weight", "layers.0.attn.wkv.scale",
                     "layers.0.attn.wo_b.weight", "layers.0.attn.norm.weight", "layers.0.attn.attn_sink", "head.weight",
                     "layers.0.ffn.shared_experts.w1.weight", "layers.0.ffn.shared_experts.w1.scale"]
    assert int(out[0][1][0]) == (4 if expert_dtype == "fp4" else 8)
    assert [c[0] for c in calls] == [expert_dtype, "fp8", "fp8", "fp8"]
    assert all(c[1] == torch.bfloat16 for c in calls)             # the bf16 view is what gets quantised
    assert out[6][1] is not None and out[6][1].dtype == torch.float32 and out[6][1].equal(w)


def test_scale_key_in_bucket_is_an_error():
    with pytest.raises(RuntimeError, match="expects bf16 weight keys"):
        R.iter_model_aware_quantized_weights(_Model(), [("layers.0.attn.wq_b.scale", torch.ones(1))], expert_dtype="fp8")


def test_reference_alias_cases():
    """The alias expectations of tests/test_gpatch_v4/test_vllm_weight_reload.py:217-339."""
    c = R.loaded_name_candidates("layers.0.attn.wq_b.scale")
    assert {"layers.0.attn.wq_b.weight_scale_inv", "model.layers.0.attn.wq_b.scale", "model.layers.0.attn.wq_b.weight_scale_inv"} <= c
    assert "model.embed_tokens.weight" in R.loaded_name_candidates("embed.weight")
    assert "model.lm_head.weight" in R.loaded_name_candidates("head.weight")
    c = R.loaded_name_candidates("model.layers.0.attn.wq_b.scale")
    assert {"layers.0.attn.wq_b.weight_scale_inv", "model.layers.0.attn.wq_b.weight_scale_inv"} <= c
    assert "model.model.layers.0.attn.wq_b.scale" not in c
    for key in ("layers.0.attn.wq_a.weight", "layers.0.attn.wkv.weight"):
        assert "model.layers.0.attn.fused_wqa_wkv.weight" in R.loaded_name_candidates(key)
    for key in ("layers.0.attn.wq_a.scale", "layers.0.attn.wkv.scale"):
        assert "model.layers.0.attn.fused_wqa_wkv.weight_scale_inv" in R.loaded_name_candidates(key)
    fused = "model.layers.2.attn.mla_attn.compressor.fused_wkv_wgate.weight"
    assert fused in R.loaded_name_candidates("layers.2.attn.compressor.wkv.weight")
    assert fused in R.loaded_name_candidates("layers.2.attn.compressor.wgate.weight")
    assert "model.layers.2.attn.mla_attn.compressor.norm.weight" in R.loaded_name_candidates("layers.2.attn.compressor.norm.weight")
    assert "model.layers.2.attn.mla_attn.compressor.ape" in R.loaded_name_candidates("layers.2.attn.compressor.ape")
    ifused = "model.layers.2.attn.indexer.compressor.fused_wkv_wgate.weight"
    assert ifused in R.loaded_name_candidates("layers.2.attn.indexer.compressor.wkv.weight")
    assert ifused in R.loaded_name_candidates("layers.2.attn.indexer.compressor.wgate.weight")
    m = nn.Module()
    assert "model.layers.0.ffn.experts.w13_weight" in R.candidate_param_names_for_reflection(m, "layers.0.ffn.experts.3.w1.weight")
    assert "model.layers.0.ffn.experts.w2_weight" in R.candidate_param_names_for_reflection(m, "layers.0.ffn.experts.3.w2.weight")
    assert "model.layers.0.ffn.experts.w13_weight" in R.candidate_param_names_for_reflection(m, "layers.0.ffn.experts.3.w3.weight")
    gate_up = "model.layers.0.ffn.shared_experts.gate_up_proj.weight"
    assert gate_up in R.candidate_param_names_for_reflection(m, "layers.0.ffn.shared_experts.w1.weight")
    assert gate_up in R.candidate_param_names_for_reflection(m, "layers.0.ffn.shared_experts.w3.weight")
    assert "model.layers.0.ffn.shared_experts.down_proj.weight" in R.candidate_param_names_for_reflection(m, "layers.0.ffn.shared_experts.w2.weight")
    assert gate_up + "_scale_inv" in R.candidate_param_names_for_reflection(m, "layers.0.ffn.shared_experts.w1.scale")
    # the loader mapping keeps the shard names of the fused gate_up projection
    assert R.map_checkpoint_key_to_vllm_param_name(m, "layers.0.ffn.shared_experts.w1.scale") == \
        "model.layers.0.ffn.shared_experts.w1.weight_scale_inv"
    assert R.map_checkpoint_key_to_vllm_param_name(m, "layers.0.ffn.shared_experts.w3.scale") == \
        "model.layers.0.ffn.shared_experts.w3.weight_scale_inv"
