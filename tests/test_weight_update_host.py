"""Host logic of the weight-export / SGLang weight-update path (CPU only, no kernel is launched): key renaming and
classification, atomic groups and buckets, and the routing of each key to its quantiser, checked the way the
reference's own unit tests check them (tests/test_gpatch_v4/test_sglang_weight_update_dsv4.py,
tests/test_gfused/test_deepseek_v4_weight_export.py) with the quantisers replaced by stand-ins."""
from unittest.mock import patch

import pytest
import torch

from gcore_lowp import sglang_weight_update_dsv4 as update
from gcore_lowp import weight_export as W

_EXPERT_KEY = "layers.0.ffn.experts.0.w1.weight"
_DENSE_KEY = "layers.0.attn.wq_b.weight"
_WO_A_KEY = "layers.0.attn.wo_a.weight"


def test_key_renaming_and_classes():
    cases = {
        "embed_tokens.weight": "embed.weight",
        "lm_head.weight": "head.weight",
        "hc_head.hc_fn": "hc_head_fn",
        "layers.3.attn_hc.base": "layers.3.hc_attn_base",
        "layers.3.input_layernorm.weight": "layers.3.attn_norm.weight",
        "layers.3.self_attn.q_a_proj.weight": "layers.3.attn.wq_a.weight",
        "layers.3.self_attn.o_a_proj.weight": "layers.3.attn.wo_a.weight",
        "layers.3.self_attn.q_a_norm.weight": "layers.3.attn.q_norm.weight",
        "layers.3.self_attn.compressor.kv_proj.weight": "layers.3.attn.compressor.wkv.weight",
        "layers.3.self_attn.compressor.indexer.q_b_proj.weight": "layers.3.attn.indexer.wq_b.weight",
        "layers.3.self_attn.compressor.indexer.kv_norm.weight": "layers.3.attn.indexer.compressor.norm.weight",
        "layers.3.self_attn.compressor.indexer._position_bias_holder.weight": "layers.3.attn.indexer.compressor.ape",
        "layers.3.self_attn.compressor._position_bias_holder.weight": "layers.3.attn.compressor.ape",
        "layers.3.self_attn._sink_holder.weight": "layers.3.attn.attn_sink",
        "layers.3.mlp.gate.e_score_correction_bias": "layers.3.ffn.gate.bias",
        "layers.3.mlp.shared_experts.up_proj.weight": "layers.3.ffn.shared_experts.w3.weight",
        "layers.3.mlp.gate.weight": "layers.3.ffn.gate.weight",
        "mtp.layers.1.self_attn.kv_proj.weight": "mtp.1.attn.wkv.weight",
        "mtp.layers.0.e_proj.weight": "mtp.0.e_proj.weight",
    }
    for src, dst in cases.items():
        assert W._model_to_disk_key(src) == dst, src
    f = torch.zeros(1)
    assert W._classify_for_save("layers.0.ffn.experts.7.w2.weight", f) == "fp4_expert"
    assert W._classify_for_save("layers.0.attn.wo_a.weight", f) == "fp8_e4m3"
    assert W._classify_for_save("layers.0.attn.wo_a.weight", f, is_sgl_ckpt_fmt=True) == "bf16_passthrough"
    assert W._classify_for_save("layers.0.attn.compressor.wkv.weight", f) == "bf16_passthrough"
    assert W._classify_for_save("layers.0.attn.indexer.wq_b.weight", f) == "fp8_e4m3"
    assert W._classify_for_save("mtp.0.main_proj.weight", f) == "fp8_e4m3"
    assert W._classify_for_save("layers.0.attn.attn_sink", f) == "f32_passthrough"
    assert W._classify_for_save("layers.0.attn.indexer.compressor.ape", f) == "f32_passthrough"
    assert W._classify_for_save("layers.0.hc_ffn_scale", f) == "f32_passthrough"
    assert W._classify_for_save("embed.weight", f) == "bf16_passthrough"
    assert W._classify_for_save("layers.0.ffn.gate.tid2eid", torch.zeros(1, dtype=torch.int32)) == "int_passthrough"

    class Cfg:
        pass

    c = Cfg()
    assert W.resolve_dsv4_export_dtypes(c) == ("fp4", False)
    c.is_sgl_ckpt_fmt = True
    assert W.resolve_dsv4_export_dtypes(c) == ("fp8", True)
    c.expert_dtype = "fp4"
    assert W.resolve_dsv4_export_dtypes(c) == ("fp4", True)
    c.expert_dtype = "int4"
    with pytest.raises(AssertionError):
        W.resolve_dsv4_export_dtypes(c)


def test_export_split_and_unquantised_paths():
    """test_deepseek_v4_weight_export.py:77-100 and the per-expert split, with stand-in quantisers"""
    dense = torch.randn(128, 128)
    out = dict(W.iter_disk_checkpoint_tensors("layers.0.mlp.gate.weight", dense, dtype_format="bf16"))
    assert list(out) == ["layers.0.ffn.gate.weight"] and out["layers.0.ffn.gate.weight"].dtype == torch.bfloat16
    assert list(W.iter_disk_checkpoint_tensors("mtp.layers.0.self_attn.q_a_proj.weight", dense, include_mtp=False)) == []
    gate_up = torch.randn(2, 256, 128)
    seen = []

    def fake_fp4(x):
        seen.append(("fp4", x))
        return torch.zeros(x.shape[0], x.shape[1] // 2, dtype=torch.int8), torch.zeros(x.shape[0], x.shape[1] // 32)

    def fake_fp8(x):
        seen.append(("fp8", x))
        return torch.zeros_like(x), torch.zeros(x.shape[0] // 128, x.shape[1] // 128)

    with patch.object(W, "quant_fp4_e2m1_scale_e8m0_packed", fake_fp4), patch.object(W, "quant_fp8_e4m3_scale_e8m0", fake_fp8):
        out = list(W.iter_disk_checkpoint_tensors("layers.0.mlp.experts.gate_up_proj", gate_up))
        names = [k for k, _ in out]
        assert names == ["layers.0.ffn.experts.0.w1.weight", "layers.0.ffn.experts.0.w1.scale",
                         "layers.0.ffn.experts.0.w3.weight", "layers.0.ffn.experts.0.w3.scale",
                         "layers.0.ffn.experts.1.w1.weight", "layers.0.ffn.experts.1.w1.scale",
                         "layers.0.ffn.experts.1.w3.weight", "layers.0.ffn.experts.1.w3.scale"]
        assert [k for k, _ in seen] == ["fp4"] * 4
        # the quantiser sees the bf16 view of the master, w1 = first half of dim 1, w3 = second half
        assert torch.equal(seen[0][1], gate_up[0, :128].bfloat16().float())
        assert torch.equal(seen[3][1], gate_up[1, 128:].bfloat16().float())
        seen.clear()
        out = list(W.iter_disk_checkpoint_tensors("layers.0.mlp.experts.down_proj", torch.randn(2, 128, 128), expert_dtype="fp8"))
        assert [k for k, _ in out] == ["layers.0.ffn.experts.0.w2.weight", "layers.0.ffn.experts.0.w2.scale",
                                       "layers.0.ffn.experts.1.w2.weight", "layers.0.ffn.experts.1.w2.scale"]
        assert [k for k, _ in seen] == ["fp8", "fp8"]
        seen.clear()
        out = list(W.iter_disk_checkpoint_tensors("layers.2.self_attn.o_b_proj.weight", dense))
        assert [k for k, _ in out] == ["layers.2.attn.wo_b.weight", "layers.2.attn.wo_b.scale"] and seen[0][0] == "fp8"
        out = list(W.iter_disk_checkpoint_tensors("layers.2.self_attn.o_b_proj.weight", dense, dtype_format="bf16"))
        assert len(out) == 1 and out[0][1] is dense
    with pytest.raises(AssertionError):
        W._split_per_expert("layers.0.mlp.experts.3.w1.weight", dense)


def test_atomic_units_and_buckets():
    groups = update.get_dsv4_sglang_atomic_update_groups()
    t = lambda n: torch.zeros(n, dtype=torch.uint8)
    items = [("layers.0.attn.wq_a.weight", t(10)), ("layers.0.attn.norm.weight", t(3)),
             ("layers.0.attn.wq_a.weight_scale_inv", t(1)), ("layers.1.attn.wkv.weight", t(7)),
             ("layers.0.attn.wkv.weight", t(20)), ("layers.0.attn.wkv.weight_scale_inv", t(2)),
             ("layers.1.attn.wq_a.weight", t(5)),
             ("layers.0.attn.indexer.compressor.wgate.weight", t(4)), ("layers.0.attn.indexer.compressor.wkv.weight", t(4)),
             ("layers.0.attn.compressor.wkv.weight", t(6)), ("layers.0.attn.compressor.wgate.weight", t(6))]
    units = list(update.stream_atomic_units(iter(items), groups))
    assert [[n for n, _ in u] for u in units] == [
        ["layers.0.attn.norm.weight"],
        ["layers.0.attn.wq_a.weight", "layers.0.attn.wkv.weight"],
        ["layers.0.attn.wq_a.weight_scale_inv", "layers.0.attn.wkv.weight_scale_inv"],
        ["layers.1.attn.wq_a.weight", "layers.1.attn.wkv.weight"],
        ["layers.0.attn.indexer.compressor.wkv.weight", "layers.0.attn.indexer.compressor.wgate.weight"],
        ["layers.0.attn.compressor.wkv.weight", "layers.0.attn.compressor.wgate.weight"]]
    with pytest.raises(RuntimeError, match="Incomplete"):
        list(update.stream_atomic_units(iter(items[:1]), groups))
    with pytest.raises(RuntimeError, match="Duplicate"):
        list(update.stream_atomic_units(iter([items[0], items[0]]), groups))
    buckets = list(update.chunk_atomic_units_by_size(iter(units), 32))
    sizes = [sum(x.numel() for _, x in b) for b in buckets]
    assert sizes == [3, 30, 23, 12]          # never split, flushed before the unit that reaches the limit
    assert sum(len(b) for b in buckets) == len(items)
    assert list(update.chunk_atomic_units_by_size(iter([]), 8)) == []


def test_routing_of_keys_to_quantisers():
    """test_sglang_weight_update_dsv4.py:66-264, the mock-based cases"""
    weight = torch.randn(128, 128)
    qweight, fp8_scale = torch.empty_like(weight), torch.ones(1, 1)
    with patch.object(update, "fp4_qat_then_to_fp8", return_value=(qweight, fp8_scale)) as kern, \
            patch.object(update, "quantize_fp8") as regular:
        out = list(update.iter_fp8_quantized_weights(iter([(_EXPERT_KEY, weight)]), fp4_qat=True))
    assert kern.call_count == 1 and not regular.called
    # the kernel receives the bf16 view of the master in an fp32 container
    passed = kern.call_args.args[0]
    assert passed.dtype == torch.float32 and torch.equal(passed, weight.bfloat16().float())
    assert not torch.equal(passed, weight)
    assert [n for n, _ in out] == [_EXPERT_KEY, "layers.0.ffn.experts.0.w1.weight_scale_inv"]
    assert out[0][1] is qweight and torch.equal(out[1][1], fp8_scale) and out[1][1].dtype == torch.float32

    sentinel = [(_DENSE_KEY, torch.empty(0)), ("layers.0.attn.wq_b.weight_scale_inv", torch.empty(0))]
    dense = torch.ones(128, 128, dtype=torch.bfloat16)
    with patch.object(update, "quantize_fp8", return_value=sentinel) as regular:
        out = list(update.iter_fp8_quantized_weights(iter([(_DENSE_KEY, dense)]), fp4_qat=True))
    regular.assert_called_once_with(_DENSE_KEY, dense, moe_deepgemm=False)
    assert out[0][1] is sentinel[0][1] and out[1][1] is sentinel[1][1]
    with patch.object(update, "quantize_fp8", return_value=sentinel) as regular:
        list(update.iter_fp8_quantized_weights(iter([(_EXPERT_KEY, dense)])))
    regular.assert_called_once_with(_EXPERT_KEY, dense, moe_deepgemm=False)

    transformed = torch.empty(1, 1, dtype=torch.uint8)
    with patch.object(update, "fp4_qat_then_to_fp8", return_value=(torch.empty(128, 128), fp8_scale)), \
            patch.object(update, "_init_fp8_quantizers") as init, \
            patch.object(update, "_use_ue8m0_scale", return_value=True) as use, \
            patch.object(update, "_transform_scale_ue8m0_fn", return_value=transformed) as tr:
        out = update.quantize_fp4_qat_expert(_EXPERT_KEY, weight, moe_deepgemm=True)
    init.assert_called_once_with()
    use.assert_called_once_with(_EXPERT_KEY, moe_deepgemm=True)
    tr.assert_called_once_with(fp8_scale, mn=128)
    assert out[1][0].endswith(".weight_scale_inv") and out[1][1] is transformed

    qdq = torch.full((128, 128), 0.5, dtype=torch.bfloat16)
    with patch.object(update, "simulate_fp8_wo_a", return_value=[(_WO_A_KEY, qdq)]) as sim, \
            patch.object(update, "quantize_fp8") as regular, patch.object(update, "quantize_fp4_qat_expert") as expert:
        out = list(update.iter_fp8_quantized_weights(iter([(_WO_A_KEY, dense)]), fp4_qat=True))
    sim.assert_called_once_with(_WO_A_KEY, dense)
    assert not regular.called and not expert.called and out == [(_WO_A_KEY, qdq)]
    with patch.object(update, "simulate_fp8_wo_a") as sim, patch.object(update, "quantize_fp8") as regular:
        out = list(update.iter_fp8_quantized_weights(iter([(_WO_A_KEY, dense)]), fp4_qat=False))
    assert not sim.called and not regular.called and out[0][1] is dense

    with pytest.raises(RuntimeError, match="scale key"):
        list(update.iter_fp8_quantized_weights(iter([("layers.0.attn.wq_b.scale", dense)])))
    assert update.should_fp8_quantize("mtp.0.h_proj.weight") and update.should_fp8_quantize("layers.9.ffn.shared_experts.w2.weight")
    assert not update.should_fp8_quantize("layers.9.ffn.gate.weight") and not update.should_fp8_quantize(_WO_A_KEY)
    assert not update._use_ue8m0_scale(_EXPERT_KEY, moe_deepgemm=True)       # SGLang has not asked for the DeepGEMM layout


def test_transform_scale_ue8m0_layout():
    """The DeepGEMM scale layout, restated element by element: row r of the result takes the scales of weight-row
    block r // 128, int32 j holds the exponent bytes of K blocks 4 j .. 4 j + 3 (low byte first, zero beyond the end),
    and rows are the fastest index in memory with a column pitch of mn rounded up to 4.  (Parity with the DeepGEMM
    helper itself is unpinned: the library is not in the reference tree.)"""
    g = torch.Generator().manual_seed(5)
    for lead, mn, kb in (((), 384, 7), ((), 130, 4), ((3,), 256, 9)):
        nblk = -(-mn // 128)
        expo = torch.randint(90, 140, (*lead, nblk, kb), generator=g)
        sf = torch.pow(2.0, (expo - 127).float())
        out = update.transform_scale_ue8m0(sf, mn=mn)
        kq = -(-kb // 4)
        assert out.dtype == torch.int32 and tuple(out.shape) == (*lead, mn, kq)
        assert out.stride(-2) == 1 and out.stride(-1) == -(-mn // 4) * 4
        flat_e = expo.reshape(-1, nblk, kb)
        flat_o = out.reshape(-1, mn, kq)
        for b in range(flat_e.shape[0]):
            for r in (0, 1, 127, 128, mn - 1):
                for j in range(kq):
                    want = 0
                    for i in range(4):
                        k = 4 * j + i
                        if k < kb:
                            want |= int(flat_e[b, r // 128, k]) << (8 * i)
                    got = int(flat_o[b, r, j]) & 0xFFFFFFFF
                    assert got == want, (lead, mn, kb, b, r, j, hex(got), hex(want))
