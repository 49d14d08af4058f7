"""The checkpoint converters (tools/convert_deepseek_v4_fp4_to_bf16.py, tools/dsv4_quant_and_dequant/convert.py
drop-ins) on a tiny synthetic DeepSeek-V4-style checkpoint: every written tensor equals the CPU oracle's,
key / shard / index / aux-file conventions follow the reference."""
import json
import os
import subprocess
import sys

import pytest
import torch
from safetensors import safe_open
from safetensors.torch import save_file

from oracle import torch_ref as T

pytestmark = pytest.mark.gpu

E4M3, E8M0 = torch.float8_e4m3fn, torch.float8_e8m0fnu


def say(*a):
    print("[case]", *a, flush=True)


def u8(t):
    return t.contiguous().view(torch.uint8)


def same(a, b):
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(u8(a), u8(b))


def make_official(root):
    """Two shards; the scale of expert 0 / w1 lives in the other shard than its weight."""
    g = torch.Generator().manual_seed(1)
    t = {}
    for layer in (0, 1):
        for e in (0, 1):
            for w, (o, i) in (("w1", (128, 256)), ("w2", (256, 128))):
                name = f"layers.{layer}.ffn.experts.{e}.{w}"
                t[name + ".weight"] = torch.randint(0, 256, (o, i // 2), generator=g, dtype=torch.int32).to(torch.uint8).view(torch.int8)
                t[name + ".scale"] = torch.randint(117, 128, (o, i // 32), generator=g, dtype=torch.int32).to(torch.uint8).view(E8M0)
        for nm, (o, i) in (("attn.wo_a", (128, 128)), ("attn.wq_a", (256, 128)), ("ffn.shared_experts.w1", (128, 256))):
            name = f"layers.{layer}.{nm}"
            t[name + ".weight"] = torch.randint(0, 0x7E, (o, i), generator=g, dtype=torch.int32).to(torch.uint8).view(E4M3)
            t[name + ".scale"] = torch.randint(115, 125, (o // 128, i // 128), generator=g, dtype=torch.int32).to(torch.uint8).view(E8M0)
        t[f"layers.{layer}.attn_norm.weight"] = torch.randn(128, generator=g).to(torch.bfloat16)
        t[f"layers.{layer}.ffn.gate.bias"] = torch.randn(4, generator=g)
    t["embed.weight"] = torch.randn(64, 128, generator=g).to(torch.bfloat16)
    shard_of = {k: ("model-00001-of-00002.safetensors" if (".experts.0." in k or "attn" in k or k == "embed.weight")
                    else "model-00002-of-00002.safetensors") for k in t}
    shard_of["layers.0.ffn.experts.0.w1.scale"] = "model-00002-of-00002.safetensors"
    os.makedirs(root, exist_ok=True)
    for shard in sorted(set(shard_of.values())):
        save_file({k: v for k, v in t.items() if shard_of[k] == shard}, os.path.join(root, shard))
    with open(os.path.join(root, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {"total_size": 0}, "weight_map": shard_of}, f)
    with open(os.path.join(root, "config.json"), "w") as f:
        json.dump({"model_type": "deepseek_v4", "expert_dtype": "fp4"}, f)
    with open(os.path.join(root, "tokenizer.json"), "w") as f:
        f.write("{}")
    return t, shard_of


def load_dir(root):
    out, where = {}, {}
    for fn in sorted(os.listdir(root)):
        if fn.endswith(".safetensors"):
            with safe_open(os.path.join(root, fn), framework="pt", device="cpu") as f:
                for k in f.keys():
                    out[k] = f.get_tensor(k)
                    where[k] = fn
    return out, where


def test_fp4_checkpoint_to_bf16(tmp_path):
    from gcore_lowp import convert_deepseek_v4_fp4_to_bf16 as C
    say("convert_deepseek_v4_fp4_to_bf16.main")
    src, dst = str(tmp_path / "official"), str(tmp_path / "bf16")
    t, shard_of = make_official(src)
    C.main(src, dst)
    out, where = load_dir(dst)
    assert not any(k.endswith(".scale") for k in out)
    assert set(out) == {k for k in t if not k.endswith(".scale")}
    for k, v in out.items():
        assert where[k] == shard_of[k], k                         # same file names as the source
        if t[k].dtype == torch.int8:
            assert same(v, T.cast_e2m1fn_to_bf16(t[k], t[k.replace(".weight", ".scale")])), k
        elif t[k].dtype == E4M3:
            assert same(v, T.cast_e4m3fn_to_bf16(t[k], t[k.replace(".weight", ".scale")])), k
        else:
            assert same(v, t[k]), k
    idx = json.load(open(os.path.join(dst, "model.safetensors.index.json")))
    assert idx["weight_map"] == where
    assert idx["metadata"]["total_size"] == sum(v.numel() * v.element_size() for v in out.values())
    assert os.path.isfile(os.path.join(dst, "tokenizer.json")) and os.path.isfile(os.path.join(dst, "config.json"))
    # --layers keeps layer-agnostic keys and the chosen layers only
    dst1 = str(tmp_path / "bf16_l1")
    C.main(src, dst1, layers=C._parse_layers("1"))
    out1, _ = load_dir(dst1)
    assert "embed.weight" in out1 and all(not k.startswith("layers.0.") for k in out1)
    assert any(k.startswith("layers.1.") for k in out1)
    assert C._parse_layers("0,1,3-5") == {0, 1, 3, 4, 5} and C._parse_layers(None) is None


def expected_official2sgl(t):
    want = {}
    for k, v in t.items():
        if k.endswith(".scale"):
            continue
        sk = k[:-len(".weight")] + ".scale" if k.endswith(".weight") else None
        s = t.get(sk) if sk else None
        if ".experts." in k and "shared_experts" not in k and k.endswith(".weight"):
            want[k], want[sk] = T.official_expert_to_sgl(v, s)
        elif k.endswith("attn.wo_a.weight"):
            want[k] = T.dequant_fp4_e2m1_fp8_scale_e8m0_packed(v, s).to(torch.bfloat16)
        elif s is not None and v.dtype == E4M3:
            want[k], want[sk] = v, s.float()
        else:
            want[k] = v
    return want


def test_official_to_sgl_and_back(tmp_path):
    from gcore_lowp import dsv4_convert as D
    say("dsv4_convert official2sgl")
    src, mid, back = str(tmp_path / "official"), str(tmp_path / "sgl"), str(tmp_path / "official2")
    t, shard_of = make_official(src)
    D.convert_checkpoint(src, mid, "official2sgl")
    out, where = load_dir(mid)
    want = expected_official2sgl(t)
    assert set(out) == set(want)
    for k in want:
        assert same(out[k], want[k]), k
        assert where[k] == shard_of[k[:-len(".scale")] + ".weight" if k.endswith(".scale") else k], k
    cfg = json.load(open(os.path.join(mid, "config.json")))
    assert "expert_dtype" not in cfg and cfg["model_type"] == "deepseek_v4"
    idx = json.load(open(os.path.join(mid, "model.safetensors.index.json")))
    assert idx["weight_map"] == where
    assert idx["metadata"]["total_size"] == sum(v.numel() * v.element_size() for v in out.values())

    say("dsv4_convert sgl2official (module CLI in a child process)")
    env = dict(os.environ)
    env["PYTHONPATH"] = os.pathsep.join(p for p in sys.path if p)
    r = subprocess.run([sys.executable, "-m", "gcore_lowp.dsv4_convert", "--direction", "sgl2official", "--src", mid,
                        "--dst", back], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    out2, _ = load_dir(back)
    for k, v in out.items():
        if k.endswith(".scale"):
            continue
        sk = k[:-len(".weight")] + ".scale" if k.endswith(".weight") else None
        s = out.get(sk) if sk else None
        if ".experts." in k and "shared_experts" not in k and k.endswith(".weight"):
            wq, ws = T.sgl_expert_to_official(v, s)
            assert same(out2[k], wq) and same(out2[sk], ws), k
        elif k.endswith("attn.wo_a.weight"):
            wq, ws = T.quant_fp8_e4m3_scale_e8m0(v.float(), (128, 128))
            assert same(out2[k], wq) and same(out2[sk], ws), k
        elif s is not None and v.dtype == E4M3:
            assert same(out2[k], v) and same(out2[sk], s.to(E8M0)), k
        else:
            assert same(out2[k], v), k
    assert json.load(open(os.path.join(back, "config.json")))["expert_dtype"] == "fp4"
    # dense weights and scales are back to the official bytes
    for k in t:
        if "wq_a" in k or "shared_experts" in k:
            assert same(out2[k], t[k]), k
    with pytest.raises(RuntimeError):
        D.convert_checkpoint(src, str(tmp_path / "x"), "official2sgl", device="cpu")


def test_compare_checkpoints(tmp_path, capsys):
    """tools/dsv4_quant_and_dequant/compare_hf_ckpts.py drop-in: a converted checkpoint equals its source after each
    side's dequantisation (the expert rebase is lossless), a planted difference and a missing key are reported."""
    from gcore_lowp import compare_hf_ckpts as V
    from gcore_lowp import dsv4_convert as D
    say("compare_hf_ckpts")
    src, mid, back = str(tmp_path / "official"), str(tmp_path / "sgl"), str(tmp_path / "official2")
    t, shard_of = make_official(src)
    D.convert_checkpoint(src, mid, "official2sgl")
    D.convert_checkpoint(mid, back, "sgl2official")
    # across the two layouts every shared tensor agrees in value; the keys differ by wo_a's scale (bf16 in the SGLang
    # layout), which the reference's verdict counts as a problem too
    assert V.main(["--a", src, "--b", mid, "--a-name", "official", "--b-name", "sgl"]) == 1
    text = capsys.readouterr().out
    assert "shared=%d" % (len(t) - 2) in text and "bad=0" in text and "expert/torch.int8" in text
    assert "only_official=2" in text and "layers.0.ffn.experts.E.w1.weight" in text      # experts folded into one line
    # same layout on both sides: the round trip of the converters
    assert V.main(["--a", src, "--b", back, "--a-name", "official", "--b-name", "roundtrip"]) == 0
    text = capsys.readouterr().out
    assert "shared=%d" % len(t) in text and "bad=0" in text and "ALL CONSISTENT" in text
    assert V.main(["--a", src, "--b", mid, "--dtype-only"]) == 1
    # plant a difference in one dense weight and drop one key from the index of the copy
    bad = str(tmp_path / "official_bad")
    os.makedirs(bad)
    out, where = load_dir(back)
    k = "layers.1.attn.wq_a.weight"
    out[k] = (-out[k].float()).to(E4M3)                           # cosine -1
    wm = dict(where)
    del out["embed.weight"], wm["embed.weight"]
    for shard in sorted(set(where.values())):
        save_file({kk: v for kk, v in out.items() if where[kk] == shard}, os.path.join(bad, shard))
    with open(os.path.join(bad, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": wm}, f)
    assert V.main(["--a", src, "--b", bad]) == 1
    text = capsys.readouterr().out
    assert "[DIFF] " + k in text and "only_A=1" in text and "[only in A] embed.weight" in text and "PROBLEMS FOUND" in text


def test_convert_json(tmp_path):
    """tools/convert_fp8/convert_json.py drop-in (no GPU work; kept with the other checkpoint tools)"""
    from gcore_lowp import convert_json as J
    src, dst = tmp_path / "in", tmp_path / "out"
    src.mkdir()
    dst.mkdir()
    (src / "config.json").write_text(json.dumps({"a": 1, "quantization_config": {"x": 1}, "num_nextn_predict_layers": 1}))
    (src / "model.safetensors.index.json").write_text(json.dumps({"metadata": {"total_size": 3}, "weight_map": {
        "model.layers.0.w.weight": "f1", "model.layers.0.w.weight_scale_inv": "f1", "model.layers.61.w.weight": "f2"}}))
    J.main(["--load_hf_dir", str(src), "--save_hf_dir", str(dst), "--remove_fp8", "--remove_mtp"])
    assert json.loads((dst / "config.json").read_text()) == {"a": 1}
    assert json.loads((dst / "model.safetensors.index.json").read_text()) == {
        "metadata": {"total_size": 3}, "weight_map": {"model.layers.0.w.weight": "f1"}}
    J.main(["--load_hf_dir", str(src), "--save_hf_dir", str(dst)])
    assert len(json.loads((dst / "model.safetensors.index.json").read_text())["weight_map"]) == 3


def test_pipeline_order_results_and_errors():
    """The converters' host <-> device pipeline: every job comes back once with the right payload, host-only jobs
    pass through, and an exception on the feeding thread or in the compute step surfaces in the caller."""
    from gcore_lowp._pipeline import run_pipelined
    say("run_pipelined")
    dev = torch.device("cuda", 0)
    src = [torch.full((257, 33), i, dtype=torch.float32) for i in range(40)]

    def jobs():
        for i, t in enumerate(src):
            yield i, (t, None), i % 5 != 0

    def compute(tag, tensors):
        t = tensors[0]
        assert t.is_cuda == (tag % 5 != 0)
        return {"double": t * 2, "meta": torch.tensor([tag])}

    got = dict(run_pipelined(dev, jobs(), compute))
    assert sorted(got) == list(range(40))
    for i, res in got.items():
        assert not res["double"].is_cuda and torch.equal(res["double"], src[i] * 2) and int(res["meta"]) == i

    def bad_jobs():
        yield 0, (src[0],), True
        raise OSError("shard unreadable")

    with pytest.raises(OSError, match="shard unreadable"):
        list(run_pipelined(dev, bad_jobs(), lambda tag, t: {"x": t[0]}))

    def bad_compute(tag, tensors):
        if tag == 3:
            raise ValueError("no rule for this weight")
        return {"x": tensors[0]}

    with pytest.raises(ValueError, match="no rule"):
        list(run_pipelined(dev, jobs(), bad_compute))


@pytest.mark.parametrize(("block", "hidden", "inter", "scale_dtype"),
                         [((2, 2), 4, 2, torch.bfloat16), ((128, 128), 256, 128, torch.float32), ((128, 128), 256, 192, torch.bfloat16)])
def test_qwen3_mtp_postprocess(tmp_path, block, hidden, inter, scale_dtype):
    """append_mtp_weights_to_fp8_checkpoint: stacked experts become per-expert gate / up / down weights, skipped
    modules stay bf16, the rest is FP8 + weight_scale_inv, stale mtp.* index entries go
    (tools/convert_fp8/qwen3_5/tests/test_qwen3_mtp_fp8_postprocess.py:77-175); every quantised tensor equals the
    CPU oracle's.  inter = 192 with 128-row blocks: the up / gate halves do not align with the stack's tiles, so the
    per-part path runs (and a down_proj of 192 columns is refused like in the reference)."""
    from gcore_lowp import qwen3_mtp_fp8_postprocess as P
    say("qwen3 mtp postprocess", block, hidden, inter, scale_dtype)
    g = torch.Generator().manual_seed(hidden + inter)
    src, dst = tmp_path / "in", tmp_path / "out"
    src.mkdir(), dst.mkdir()
    with open(src / "config.json", "w") as f:
        json.dump({"text_config": {"model_type": "qwen3_5_moe_text", "num_experts": 2, "mtp_num_hidden_layers": 1}}, f)
    bf = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16)
    down_cols = inter if inter % block[1] == 0 else 256
    t = {"mtp.fc.weight": bf(hidden, 2 * hidden), "mtp.norm.weight": bf(hidden), "mtp.pre_fc_norm_embedding.weight": bf(hidden),
         "mtp.pre_fc_norm_hidden.weight": bf(hidden)}
    L = "mtp.layers.0."
    for k in ("input_layernorm", "post_attention_layernorm", "self_attn.q_norm", "self_attn.k_norm"):
        t[L + k + ".weight"] = bf(hidden)
    for k in ("q_proj", "k_proj", "v_proj", "o_proj"):
        t[L + f"self_attn.{k}.weight"] = bf(hidden, hidden)
    t[L + "mlp.experts.gate_up_proj"] = bf(2, 2 * inter, hidden)
    t[L + "mlp.experts.down_proj"] = bf(2, hidden, down_cols)
    t[L + "mlp.gate.weight"] = bf(2, hidden)
    t[L + "mlp.shared_expert.gate_proj.weight"] = bf(hidden, hidden)
    t[L + "mlp.shared_expert.up_proj.weight"] = bf(hidden, hidden)
    t[L + "mlp.shared_expert.down_proj.weight"] = bf(hidden, hidden)
    t[L + "mlp.shared_expert_gate.weight"] = bf(1, hidden)
    save_file(t, str(src / "input.safetensors"))
    save_file({"model.language_model.embed_tokens.weight": torch.ones(2, 2, dtype=torch.bfloat16)}, str(dst / "model.safetensors"))
    with open(dst / "model.safetensors.index.json", "w") as f:
        json.dump({"metadata": {"format": "pt", "total_size": 123},
                   "weight_map": {"model.language_model.embed_tokens.weight": "model.safetensors",
                                  "mtp.stale.weight": "mtp.safetensors"}}, f)
    skip = ["mtp.fc", "mtp.norm", "mtp.pre_fc_norm_embedding", "mtp.pre_fc_norm_hidden", L + "input_layernorm",
            L + "post_attention_layernorm", L + "self_attn.q_norm", L + "self_attn.k_norm", L + "mlp.gate", L + "mlp.shared_expert_gate"]
    if inter % block[0]:
        with pytest.raises(ValueError, match="must be divisible"):
            P.append_mtp_weights_to_fp8_checkpoint(str(src), str(dst), block_size=block, modules_to_not_convert=skip,
                                                   device="cpu", scale_dtype=scale_dtype)
        return
    written = P.append_mtp_weights_to_fp8_checkpoint(str(src), str(dst), block_size=block, modules_to_not_convert=skip,
                                                     device="cpu", scale_dtype=scale_dtype)
    expected = {}
    for key, w in t.items():
        if key.endswith("gate_up_proj"):
            for e in range(2):
                expected[L + f"mlp.experts.{e}.gate_proj.weight"], expected[L + f"mlp.experts.{e}.up_proj.weight"] = w[e].chunk(2, dim=0)
        elif key.endswith("experts.down_proj"):
            for e in range(2):
                expected[L + f"mlp.experts.{e}.down_proj.weight"] = w[e]
        else:
            expected[key] = w
    n_quant = 0
    with safe_open(str(dst / "mtp.safetensors"), framework="pt", device="cpu") as f:
        keys = set(f.keys())
        assert L + "mlp.experts.gate_up_proj" not in keys and L + "mlp.experts.down_proj" not in keys
        for key, w in expected.items():
            module = key[:-len(".weight")]
            got = f.get_tensor(key)
            if any(module == s for s in skip):
                assert same(got, w) and module + ".weight_scale_inv" not in keys
                continue
            n_quant += 1
            q, s = T.quantize_fp8_blockwise(w, block, scale_dtype=scale_dtype)
            assert got.dtype == E4M3 and same(got, q), key
            gs = f.get_tensor(module + ".weight_scale_inv")
            assert gs.dtype == scale_dtype and tuple(gs.shape) == (w.shape[0] // block[0], w.shape[1] // block[1]) and same(gs, s), key
    assert written == len(keys) == len(expected) + n_quant
    with open(dst / "model.safetensors.index.json") as f:
        index = json.load(f)
    assert index["metadata"]["format"] == "pt" and index["metadata"]["total_size"] > 123
    wm = index["weight_map"]
    assert wm["model.language_model.embed_tokens.weight"] == "model.safetensors" and "mtp.stale.weight" not in wm
    assert all(wm[k] == "mtp.safetensors" for k in keys) and len(wm) == len(keys) + 1


def _bf16_ckpt(root):
    g = torch.Generator().manual_seed(9)
    bf = lambda *s: (torch.randn(*s, generator=g) * 0.05).to(torch.bfloat16)
    t = {"model.embed_tokens.weight": bf(64, 128), "lm_head.weight": bf(64, 128), "model.norm.weight": bf(128)}
    for layer in (0, 1):
        p = f"model.layers.{layer}."
        t[p + "self_attn.q_proj.weight"] = bf(256, 128)
        t[p + "self_attn.kv_a_proj_with_mqa.weight"] = bf(72, 128)          # 72 rows: an edge tile
        t[p + "self_attn.o_proj.weight"] = bf(128, 200)                      # 200 columns: an edge tile
        t[p + "input_layernorm.weight"] = bf(128)
        t[p + "mlp.gate.weight"] = bf(4, 128)
        t[p + "mlp.experts.0.down_proj.weight"] = torch.zeros(128, 256, dtype=torch.bfloat16)   # all-zero tiles
        t[p + "mlp.gate.e_score_correction_bias"] = torch.randn(4, generator=g)
    shard_of = {k: ("model-00001-of-00002.safetensors" if "layers.1." not in k else "model-00002-of-00002.safetensors") for k in t}
    os.makedirs(root, exist_ok=True)
    for shard in sorted(set(shard_of.values())):
        save_file({k: v for k, v in t.items() if shard_of[k] == shard}, os.path.join(root, shard))
    with open(os.path.join(root, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": shard_of}, f)
    with open(os.path.join(root, "config.json"), "w") as f:
        json.dump({"model_type": "deepseek_v3", "hidden_size": 128}, f)
    return t, shard_of


def _padded_quant(w):
    rows, cols = w.shape
    wp = torch.nn.functional.pad(w.float(), (0, -cols % 128, 0, -rows % 128))
    q, s = T.quant_block_fp32_scale(wp, (128, 128), amax_floor=None, zero_scale_to_one=True)
    return q[:rows, :cols].contiguous(), s


@pytest.mark.parametrize("with_reference", [False, True])
def test_bf16_cast_fp8_cli(tmp_path, with_reference):
    """tools/convert_fp8/bf16_cast_fp8.py drop-in: which tensors are quantised (by name rule, or by a reference FP8
    checkpoint's `_scale_inv` keys), `<weight>_scale_inv` fp32 next to the weight in the same shard, index and side
    files; codes and scales against the CPU oracle's divide form on zero-completed edge tiles."""
    say("bf16_cast_fp8 cli", with_reference)
    src, dst, ref = str(tmp_path / "bf16"), str(tmp_path / "fp8"), str(tmp_path / "ref")
    t, shard_of = _bf16_ckpt(src)
    cmd = [sys.executable, "-m", "gcore_lowp.bf16_cast_fp8", "--input-bf16-hf-path", src, "--output-fp8-hf-path", dst]
    if with_reference:
        # a reference FP8 checkpoint in which only q_proj (layers 0, 1) and layer 0's o_proj are FP8
        os.makedirs(ref)
        chosen = [k for k in t if k.endswith("q_proj.weight")] + ["model.layers.0.self_attn.o_proj.weight"]
        rt = {}
        for k, v in t.items():
            rt[k] = v.to(E4M3) if k in chosen else v
            if k in chosen:
                rt[k + "_scale_inv"] = torch.ones(-(-v.shape[0] // 128), -(-v.shape[1] // 128))
        rt["model.layers.1.self_attn.o_proj.weight"] = t["model.layers.1.self_attn.o_proj.weight"].to(E4M3)   # FP8, no scale: skipped
        save_file(rt, os.path.join(ref, "model.safetensors"))
        with open(os.path.join(ref, "model.safetensors.index.json"), "w") as f:
            json.dump({"metadata": {}, "weight_map": {k: "model.safetensors" for k in rt}}, f)
        with open(os.path.join(ref, "config.json"), "w") as f:
            json.dump({"model_type": "deepseek_v3", "from": "reference"}, f)
        cmd += ["--input-fp8-hf-path", ref]
    else:
        chosen = [k for k in t if k.endswith("_proj.weight")]
    env = dict(os.environ, PYTHONPATH=os.pathsep.join(p for p in sys.path if p))
    r = subprocess.run(cmd, env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]
    with open(os.path.join(dst, "model.safetensors.index.json")) as f:
        wm = json.load(f)["weight_map"]
    assert set(wm) == set(t) | {k + "_scale_inv" for k in chosen}
    for k in t:
        assert wm[k] == shard_of[k]
        with safe_open(os.path.join(dst, wm[k]), framework="pt", device="cpu") as f:
            got = f.get_tensor(k)
            if k in chosen:
                q, s = _padded_quant(t[k])
                assert wm[k + "_scale_inv"] == shard_of[k]
                gs = f.get_tensor(k + "_scale_inv")
                assert got.dtype == E4M3 and same(got, q), k
                assert gs.dtype == torch.float32 and same(gs, s), k
            else:
                assert same(got, t[k]), k
                assert k + "_scale_inv" not in f.keys()
    with open(os.path.join(dst, "config.json")) as f:
        cfg = json.load(f)
    if with_reference:
        assert cfg.get("from") == "reference" and "quantization_config" not in cfg
        with open(os.path.join(dst, "weight_with_scale_inv_map.index.json")) as f:
            assert set(json.load(f)["weight_with_scale_inv_map"]) == set(chosen)
    else:
        assert cfg["quantization_config"] == {"activation_scheme": "dynamic", "fmt": "e4m3", "quant_method": "fp8",
                                              "weight_block_size": [128, 128], "modules_to_not_convert": ["lm_head"]}
