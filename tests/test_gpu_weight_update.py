"""GPU parity of the weight-export / SGLang weight-update path: the kernel-backed quantisers behind
gcore_lowp.sglang_weight_update_dsv4 and gcore_lowp.weight_export against the CPU oracle, byte for byte
(tests/test_gpatch_v4/test_sglang_weight_update_dsv4.py:31-64,202-231, tests/test_gfused/test_deepseek_v4_weight_export.py:41-75)."""
import numpy as np
import pytest
import torch

from oracle import torch_ref as T

pytestmark = pytest.mark.gpu

_EXPERT_KEY = "layers.0.ffn.experts.0.w1.weight"
_WO_A_KEY = "layers.0.attn.wo_a.weight"


def say(*a):
    print("[case]", *a, flush=True)


def u8(t):
    return t.detach().cpu().contiguous().view(torch.uint8)


@pytest.mark.parametrize(("m", "n", "seed"), [(128, 128, 7), (128, 384, 11), (256, 256, 17), (384, 640, 23)])
def test_fp4_qat_expert_update(m, n, seed):
    from gcore_lowp import sglang_weight_update_dsv4 as update
    say("quantize_fp4_qat_expert", m, n)
    torch.manual_seed(seed)
    w = torch.randn(m, n)
    out = update.quantize_fp4_qat_expert(_EXPERT_KEY, w.cuda())
    wq, ws = T.fp4_qat_then_to_fp8(w.bfloat16().float())
    assert out[0][0] == _EXPERT_KEY and out[1][0] == "layers.0.ffn.experts.0.w1.weight_scale_inv"
    assert tuple(out[0][1].shape) == (m, n) and tuple(out[1][1].shape) == (m // 128, n // 128)
    assert torch.equal(u8(out[0][1]), u8(wq))
    assert out[1][1].dtype == torch.float32 and torch.equal(out[1][1].cpu(), ws.float())


@pytest.mark.parametrize(("m", "n", "seed"), [(128, 128, 9), (256, 128, 13), (128, 256, 19)])
def test_wo_a_update_is_qdq(m, n, seed):
    from gcore_lowp import sglang_weight_update_dsv4 as update
    say("wo_a update", m, n)
    torch.manual_seed(seed)
    w = torch.randn(m, n, dtype=torch.bfloat16)
    out = list(update.iter_fp8_quantized_weights(iter([(_WO_A_KEY, w.cuda())]), fp4_qat=True))
    assert len(out) == 1 and out[0][0] == _WO_A_KEY and out[0][1].dtype == torch.bfloat16 and out[0][1].shape == w.shape
    q, s = T.quant_fp8_e4m3_scale_e8m0(w.float(), (128, 128))
    want = T.dequant_fp4_e2m1_fp8_scale_e8m0_packed(q, s)
    assert torch.equal(out[0][1].cpu().view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("shape", [(128, 128), (256, 384), (200, 300), (2, 256, 128), (4096, 7168)])
def test_dense_update_is_per_block_cast(shape):
    """quantize_fp8 = the published per_block_cast_to_fp8 on the bf16 view; scales fp32 amax / 448"""
    from gcore_lowp import sglang_weight_update_dsv4 as update
    say("quantize_fp8", shape)
    torch.manual_seed(3)
    w = torch.randn(shape) * 0.05
    w.view(-1)[:40] = 0
    if len(shape) == 2 and shape[0] >= 256:
        w[128:256, :128] = 1e-6                              # a tile under the 1e-4 clamp
    name = "layers.0.attn.wq_b.weight"
    out = update.quantize_fp8(name, w.cuda())
    w2 = w.bfloat16().float().view(-1, shape[-1])
    wq, ws = T.per_block_cast_to_fp8(w2)
    assert out[0][0] == name and out[1][0] == "layers.0.attn.wq_b.weight_scale_inv"
    assert out[0][1].shape == w.shape and out[0][1].dtype == torch.float8_e4m3fn
    assert np.array_equal(out[1][1].cpu().numpy().view(np.uint32), ws.numpy().view(np.uint32))
    assert torch.equal(u8(out[0][1]).view(-1), u8(wq).view(-1))
    with pytest.raises(ValueError):
        update.quantize_fp8(name, torch.zeros(128, device="cuda"))


def test_bucket_stream_end_to_end():
    from gcore_lowp import sglang_weight_update_dsv4 as update
    say("iter_sglang_dsv4_weight_buckets")
    torch.manual_seed(5)
    names = ["embed.weight", "layers.0.attn.wq_a.weight", "layers.0.attn_norm.weight", "layers.0.attn.wkv.weight",
             "layers.0.ffn.experts.0.w1.weight", "layers.0.attn.wo_a.weight", "layers.0.ffn.gate.weight"]
    ws = {n: torch.randn(128, 256, dtype=torch.bfloat16, device="cuda") for n in names}
    buckets = list(update.iter_sglang_dsv4_weight_buckets(iter(ws.items()), 150_000, fp4_qat=True))
    flat = [n for b in buckets for n, _ in b]
    assert sorted(flat) == sorted(names + [n + "_scale_inv" for n in
                                           ("layers.0.attn.wq_a.weight", "layers.0.attn.wkv.weight", "layers.0.ffn.experts.0.w1.weight")])
    where = {n: i for i, b in enumerate(buckets) for n, _ in b}
    assert where["layers.0.attn.wq_a.weight"] == where["layers.0.attn.wkv.weight"]
    assert where["layers.0.attn.wq_a.weight_scale_inv"] == where["layers.0.attn.wkv.weight_scale_inv"]
    got = dict((n, t) for b in buckets for n, t in b)
    assert got["embed.weight"] is ws["embed.weight"] and got["layers.0.attn.wo_a.weight"].dtype == torch.bfloat16
    assert got["layers.0.attn.wq_a.weight"].dtype == torch.float8_e4m3fn
    assert got["layers.0.ffn.experts.0.w1.weight_scale_inv"].dtype == torch.float32


def test_export_quantised_tensors():
    """iter_disk_checkpoint_tensors, "quantized": experts to FP4 (or FP8), whitelist to FP8, from the bf16 view"""
    from gcore_lowp import weight_export as W
    say("iter_disk_checkpoint_tensors")
    torch.manual_seed(1)
    gate_up = torch.randn(2, 256, 128)
    out = dict(W.iter_disk_checkpoint_tensors("layers.0.mlp.experts.gate_up_proj", gate_up.cuda()))
    for e in range(2):
        for half, wname in ((0, "w1"), (1, "w3")):
            src = gate_up[e, 128 * half:128 * half + 128].bfloat16().float()
            wp, wsc = T.quant_fp4_e2m1_scale_e8m0_packed(src)
            k = f"layers.0.ffn.experts.{e}.{wname}"
            assert out[k + ".weight"].dtype == torch.int8 and out[k + ".scale"].dtype == torch.float8_e8m0fnu
            assert torch.equal(u8(out[k + ".weight"]), u8(wp)) and torch.equal(u8(out[k + ".scale"]), u8(wsc))
    down = torch.randn(2, 128, 128)
    out = dict(W.iter_disk_checkpoint_tensors("layers.0.mlp.experts.down_proj", down.cuda(), expert_dtype="fp8"))
    wq, wsc = T.quant_fp8_e4m3_scale_e8m0(down[1].bfloat16().float(), (128, 128))
    assert out["layers.0.ffn.experts.1.w2.weight"].dtype == torch.float8_e4m3fn
    assert torch.equal(u8(out["layers.0.ffn.experts.1.w2.weight"]), u8(wq))
    assert torch.equal(u8(out["layers.0.ffn.experts.1.w2.scale"]), u8(wsc))

    class Tiny(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.config = type("C", (), {"is_sgl_ckpt_fmt": True})()
            self.p = torch.nn.ParameterDict({"a": torch.nn.Parameter(torch.randn(128, 128))})

        def state_dict(self, *a, **k):
            return {"model.layers.0.self_attn.o_a_proj.weight": self.p["a"], "model.layers.0.self_attn.o_b_proj.weight": self.p["a"],
                    "mtp.layers.0.e_proj.weight": self.p["a"]}

    got = dict(W.export_deepseek_v4_quantized_weights(Tiny().cuda()))
    assert sorted(got) == ["layers.0.attn.wo_a.weight", "layers.0.attn.wo_b.scale", "layers.0.attn.wo_b.weight"]
    assert got["layers.0.attn.wo_a.weight"].dtype == torch.bfloat16 and got["layers.0.attn.wo_b.weight"].dtype == torch.float8_e4m3fn
    assert all(t.is_cuda for t in got.values())


@pytest.mark.parametrize("expert_dtype", ["fp4", "fp8"])
def test_vllm_reload_bucket_quantisation(expert_dtype):
    """iter_model_aware_quantized_weights (vllm_weight_reload_dsv4.py:1129-1178): experts by expert_dtype, a linear
    layer that the live model keeps in e4m3 to FP8, everything else untouched; bytes against the CPU oracle on the
    bf16 view of fp32 master weights."""
    from gcore_lowp import vllm_weight_reload_dsv4 as R
    say("iter_model_aware_quantized_weights", expert_dtype)

    class LinearBase(torch.nn.Module):
        def __init__(self, dtype):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.zeros(2, 2).to(dtype), requires_grad=False)

    model = torch.nn.Module()
    model.layers = torch.nn.ModuleList([torch.nn.Module()])
    model.layers[0].attn = torch.nn.Module()
    model.layers[0].attn.wq_b = LinearBase(torch.float8_e4m3fn)
    model.layers[0].attn.wo_b = LinearBase(torch.bfloat16)
    torch.manual_seed(3)
    expert, dense, kept = torch.randn(256, 384) * 0.1, torch.randn(128, 256) * 0.1, torch.randn(128, 128)
    bucket = [("layers.0.ffn.experts.1.w2.weight", expert.cuda()), ("layers.0.attn.wq_b.weight", dense.cuda()),
              ("layers.0.attn.wo_b.weight", kept.cuda())]
    out = R.iter_model_aware_quantized_weights(model, bucket, expert_dtype=expert_dtype)
    assert [n for n, _ in out] == ["layers.0.ffn.experts.1.w2.weight", "layers.0.ffn.experts.1.w2.scale",
                                   "layers.0.attn.wq_b.weight", "layers.0.attn.wq_b.scale", "layers.0.attn.wo_b.weight"]
    got = dict(out)
    assert all(t.is_cuda and t.is_contiguous() for t in got.values())
    src = expert.bfloat16().float()
    eq, es = T.quant_fp4_e2m1_scale_e8m0_packed(src) if expert_dtype == "fp4" else T.quant_fp8_e4m3_scale_e8m0(src, (128, 128))
    assert got["layers.0.ffn.experts.1.w2.weight"].dtype == (torch.int8 if expert_dtype == "fp4" else torch.float8_e4m3fn)
    assert got["layers.0.ffn.experts.1.w2.scale"].dtype == torch.float8_e8m0fnu
    assert torch.equal(u8(got["layers.0.ffn.experts.1.w2.weight"]), u8(eq))
    assert torch.equal(u8(got["layers.0.ffn.experts.1.w2.scale"]), u8(es))
    dq, ds = T.quant_fp8_e4m3_scale_e8m0(dense.bfloat16().float(), (128, 128))
    assert torch.equal(u8(got["layers.0.attn.wq_b.weight"]), u8(dq)) and torch.equal(u8(got["layers.0.attn.wq_b.scale"]), u8(ds))
    assert got["layers.0.attn.wo_b.weight"].dtype == torch.float32 and torch.equal(got["layers.0.attn.wo_b.weight"].cpu(), kept)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(256, 384), (3, 128, 256), (200, 320)])
def test_quant_weight_ue8m0_is_pow2_block_quant(shape):
    """quant_weight_ue8m0 == the power-of-two block quantiser with the 1e-4 amax floor (oracle), bit for bit, on whole
    and ragged shapes and with an all-zero block; scales are powers of two and survive the packed layout."""
    from gcore_lowp import sglang_weight_update_dsv4 as update
    g = torch.Generator().manual_seed(17)
    w = (torch.randn(*shape, generator=g) * 0.02).to(torch.bfloat16).float()
    w.view(-1, shape[-1])[:128, :128] = 0
    q, s = update.quant_weight_ue8m0(w.cuda(), weight_block_size=[128, 128])
    flat = w.view(-1, shape[-1])
    m, k = flat.shape
    mp, kp = -(-m // 128) * 128, -(-k // 128) * 128
    pad = torch.zeros(mp, kp)
    pad[:m, :k] = flat
    rq, rs = T.quant_block_pow2_scale(pad, (128, 128), amax_floor=1e-4)
    assert q.dtype == torch.float8_e4m3fn and tuple(q.shape) == tuple(shape)
    assert torch.equal(q.cpu().view(torch.uint8).view(m, k), rq.view(torch.uint8)[:m, :k])
    assert torch.equal(s.cpu().reshape(rs.shape), rs)
    mant = s.cpu().view(torch.int32) & 0x7FFFFF
    assert int(mant.abs().max()) == 0
    n = shape[-2]
    packed = update.transform_scale_ue8m0(s, mn=n)
    first = (packed[..., 0].cpu() & 0xFF)
    assert torch.equal(first, ((s.cpu().view(torch.int32) >> 23) & 0xFF)[..., 0].repeat_interleave(128, dim=-1)[..., :n])

