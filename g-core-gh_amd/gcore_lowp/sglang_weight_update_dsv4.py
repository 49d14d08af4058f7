"""MI355X drop-in for gpatch_v4/generation_backend/sglang_model_specific/sglang_weight_update_dsv4.py: the
quantise-before-push step of a DeepSeek-V4 weight update to an SGLang sampler running `--quantization fp8`.

A stream of bf16 disk-format `(name, tensor)` pairs goes in; routed / shared experts, the dense attention
projections and the MTP projections come out as e4m3fn + `weight_scale_inv` pairs (128 x 128 blocks), everything
else unchanged; pairs that SGLang fuses in one `load_weights` call stay in one bucket.  Under `fp4_qat` routed
experts are first put on the FP4 QAT grid (fp4_qat_then_to_fp8) and `wo_a` is pushed as bf16 values on the
trainer's 128 x 128 FP8 grid.  All arithmetic runs in the HIP kernels of this package.

The dense quantiser of the reference is SGLang's `per_block_cast_to_fp8`, imported at run time
(sglang_weight_update_dsv4.py:205-223).  SGLang is not part of the reference tree, so what is built in here is
that function as published (amax clamped at 1e-4, x * (448 / amax) -> e4m3fn, scale amax / 448, fp32): scale mode
LP_SCALE_MUL_FLOOR of lp_quant_fp8_block.  The DeepGEMM pair `quant_weight_ue8m0` / `transform_scale_ue8m0` is
restated the same way (power-of-two scales from LP_SCALE_POW2 with the 1e-4 amax floor; scale bytes expanded per weight
row, packed four K blocks to an int32 and laid out MN-major with the row count aligned to 4, as the published
DeepGEMM helper does) and installed as the default hooks.  Whether they are used is SGLang's decision
(`_should_ue8m0_fn`, None here as on any sampler that does not run DeepGEMM): by default every scale is float32.
"""
from __future__ import annotations

import re
from collections.abc import Iterator, Sequence
from dataclasses import dataclass

import torch

from . import _abi as A
from . import ops
from .fused_quant_kernels import fp4_qat_then_to_fp8

# ------------------------------------------------------------------------------------------------ classification
# (sglang_weight_update_dsv4.py:41-67)
_EXPERT_RE = re.compile(r"\.experts\.\d+\.w[123]\.weight$")
_WO_A_RE = re.compile(r"^(?:.*\.)?layers\.\d+\.attn\.wo_a\.weight$|^mtp\.\d+\.attn\.wo_a\.weight$")
_ATTN = r"attn\.(?:wq_a|wq_b|wkv|wo_b)\.weight$"
_INDEXER = r"attn\.indexer\.wq_b\.weight$"
_SHARED = r"ffn\.shared_experts\.w[123]\.weight$"
_FP8_DENSE_PATTERNS: tuple[str, ...] = tuple(
    [rf"^(?:.*\.)?layers\.\d+\.{tail}" for tail in (_ATTN, _INDEXER, _SHARED)]
    + [rf"^mtp\.\d+\.{tail}" for tail in (_ATTN, _INDEXER, _SHARED)]
    + [r"^mtp\.\d+\.(?:e_proj|h_proj)\.weight$"])
_FP8_DENSE_RE = re.compile("|".join(_FP8_DENSE_PATTERNS))
_WEIGHT_BLOCK_SIZE = [128, 128]


# ------------------------------------------------------------------------------------------------ atomic groups
@dataclass(frozen=True)
class AtomicUpdateGroup:
    """Disk-key suffixes that one `load_weights` call of SGLang must see together (:78-81)."""
    key: str
    suffixes: tuple[str, ...]


def get_dsv4_sglang_atomic_update_groups() -> list[AtomicUpdateGroup]:
    """(:84-107) wq_a + wkv fuse into wqkv_a (weights and scales separately: one dtype per pack); the
    compressor's and the indexer compressor's wkv + wgate fuse into wkv_gate."""
    table = {
        "wqkv_a_weight": (".attn.wq_a.weight", ".attn.wkv.weight"),
        "wqkv_a_scale": (".attn.wq_a.weight_scale_inv", ".attn.wkv.weight_scale_inv"),
        "compressor_wkv_gate": (".attn.compressor.wkv.weight", ".attn.compressor.wgate.weight"),
        "indexer_compressor_wkv_gate": (".attn.indexer.compressor.wkv.weight", ".attn.indexer.compressor.wgate.weight"),
    }
    return [AtomicUpdateGroup(k, v) for k, v in table.items()]


def stream_atomic_units(items: Iterator[tuple[str, torch.Tensor]],
                        atomic_update_groups: Sequence[AtomicUpdateGroup]) -> Iterator[list[tuple[str, torch.Tensor]]]:
    """(:110-143) Hold the members of a group back until all of them have arrived, then yield them as one
    unit in the group's suffix order; anything else is a unit of its own."""
    lookup = [(g, i, suf) for g in atomic_update_groups for i, suf in enumerate(g.suffixes)]
    waiting: dict[tuple[str, str], list] = {}
    for name, tensor in items:
        hit = next((h for h in lookup if name.endswith(h[2])), None)
        if hit is None:
            yield [(name, tensor)]
            continue
        group, idx, suffix = hit
        slot_key = (name[:-len(suffix)], group.key)
        slots = waiting.setdefault(slot_key, [None] * len(group.suffixes))
        if slots[idx] is not None:
            raise RuntimeError(f"Duplicate atomic update member {name!r} for group {slot_key[0]}:{group.key}")
        slots[idx] = (name, tensor)
        if all(s is not None for s in slots):
            yield list(slots)
            del waiting[slot_key]
    if waiting:
        raise RuntimeError(f"Incomplete atomic update groups at end of stream: {sorted(waiting)}")


def chunk_atomic_units_by_size(units: Iterator[list[tuple[str, torch.Tensor]]],
                               chunk_size: int) -> Iterator[list[tuple[str, torch.Tensor]]]:
    """(:146-166) Greedy buckets of about chunk_size bytes; a unit is never split, a bucket is flushed before
    the unit that would take it to chunk_size or beyond."""
    bucket: list[tuple[str, torch.Tensor]] = []
    filled = 0
    for unit in units:
        nbytes = sum(t.numel() * t.element_size() for _, t in unit)
        if bucket and filled + nbytes >= chunk_size:
            yield bucket
            bucket, filled = [], 0
        bucket.extend(unit)
        filled += nbytes
    if bucket:
        yield bucket


def iter_sglang_dsv4_weight_buckets(weights: Iterator[tuple[str, torch.Tensor]], max_bucket_bytes: int, *,
                                    moe_deepgemm: bool = False, fp4_qat: bool = False):
    """(:169-186) quantise, group, bucket."""
    quantized = iter_fp8_quantized_weights(weights, moe_deepgemm=moe_deepgemm, fp4_qat=fp4_qat)
    units = stream_atomic_units(quantized, get_dsv4_sglang_atomic_update_groups())
    yield from chunk_atomic_units_by_size(units, max_bucket_bytes)


# ------------------------------------------------------------------------------------------------ quantisers
def per_block_cast_to_fp8(x: torch.Tensor):
    """SGLang's / DeepGEMM's published per_block_cast_to_fp8 on the GPU: 2D x (any float dtype), 128 x 128 blocks
    with the ragged edge zero-padded; returns (e4m3fn [m, n], float32 scales [ceil(m/128), ceil(n/128)])."""
    assert x.dim() == 2
    m, n = x.shape
    mp, np_ = -(-m // 128) * 128, -(-n // 128) * 128
    xg, home = A.to_device(x)
    if (mp, np_) != (m, n):
        pad = torch.zeros(mp, np_, dtype=xg.dtype, device=xg.device)
        pad[:m, :n] = xg
        xg = pad
    q, s, _ = ops.quant_fp8_block(xg, (128, 128), scale_mode=A.SCALE_MUL_FLOOR, scale_dtype=torch.float32, amax_floor=1e-4)
    return q[:m, :n].contiguous().to(home), s.to(home)


def quant_weight_ue8m0(weight_dequant: torch.Tensor, weight_block_size=None):
    """SGLang's `quant_weight_ue8m0` as published: [..., n, k] -> e4m3fn codes of the same shape and fp32 scales
    [..., ceil(n / 128), ceil(k / 128)] that are powers of two, 2^ceil(log2(max(amax, 1e-4) / 448)), codes
    x * (1 / scale).  One launch of lp_quant_fp8_block (LP_SCALE_POW2) over the tensor viewed as (-1, k)."""
    assert weight_block_size is None or list(weight_block_size) == [128, 128], weight_block_size
    *lead, n, k = weight_dequant.shape
    assert not lead or n % 128 == 0, "stacked matrices must hold whole 128-row blocks each"
    flat = weight_dequant.reshape(-1, k)
    m = flat.shape[0]
    mp, kp = -(-m // 128) * 128, -(-k // 128) * 128
    xg, home = A.to_device(flat.contiguous())
    if (mp, kp) != (m, k):
        pad = torch.zeros(mp, kp, dtype=xg.dtype, device=xg.device)
        pad[:m, :k] = xg
        xg = pad
    q, s, _ = ops.quant_fp8_block(xg, (128, 128), scale_mode=A.SCALE_POW2, scale_dtype=torch.float32, amax_floor=1e-4)
    q = q[:m, :k].contiguous().to(home).view(weight_dequant.shape)
    return q, s.to(home).view(*lead, -(-n // 128), kp // 128)


def transform_scale_ue8m0(sf: torch.Tensor, mn: int, use_torch_impl: bool = False) -> torch.Tensor:
    """SGLang's `transform_scale_ue8m0` as published: power-of-two fp32 scales [..., ceil(mn / 128), kb] -> one scale row
    per weight row, the exponent bytes of four consecutive K blocks packed into an int32 (block 4 j in the low byte,
    kb padded with zero bytes), returned as [..., mn, ceil(kb / 4)] int32 whose mn index is the fastest in memory with
    the column pitch rounded up to 4 rows (DeepGEMM's `get_mn_major_tma_aligned_packed_ue8m0_tensor`).  Pure index
    arithmetic on a small tensor: torch ops on whatever device holds `sf`."""
    assert sf.dtype == torch.float32 and sf.dim() >= 2, (sf.dtype, sf.shape)
    rows = torch.arange(mn, device=sf.device) // 128
    exp = (sf.index_select(-2, rows).contiguous().view(torch.int32) >> 23) & 0xFF          # [..., mn, kb]
    kb = exp.shape[-1]
    kq = -(-kb // 4)
    if kq * 4 != kb:
        exp = torch.nn.functional.pad(exp, (0, kq * 4 - kb))
    e4 = exp.view(*exp.shape[:-1], kq, 4)
    packed = e4[..., 0] | (e4[..., 1] << 8) | (e4[..., 2] << 16) | (e4[..., 3] << 24)      # [..., mn, kq]
    pitch = -(-mn // 4) * 4
    store = torch.zeros(*packed.shape[:-2], kq, pitch, dtype=torch.int32, device=sf.device)
    store[..., :mn] = packed.transpose(-1, -2)
    return store.transpose(-1, -2)[..., :mn, :]


# Hooks with the reference's names (:193-197): the tests of the reference patch them, and a deployment that has
# SGLang's own functions can install them here.  `_should_ue8m0_fn` stays None unless the deployment sets it.
_per_block_cast_fn = None
_quant_weight_ue8m0_fn = None
_transform_scale_ue8m0_fn = None
_should_ue8m0_fn = None
_fp8_ready = False


def _init_fp8_quantizers():
    """(:200-238) Resolve the dense quantiser once: the kernel-backed per_block_cast_to_fp8 of this module."""
    global _per_block_cast_fn, _fp8_ready
    if _fp8_ready:
        return
    A.lib()                                               # fail loudly here if the HIP library is missing
    global _quant_weight_ue8m0_fn, _transform_scale_ue8m0_fn
    if _per_block_cast_fn is None:
        _per_block_cast_fn = per_block_cast_to_fp8
    if _quant_weight_ue8m0_fn is None:
        _quant_weight_ue8m0_fn = quant_weight_ue8m0
    if _transform_scale_ue8m0_fn is None:
        _transform_scale_ue8m0_fn = transform_scale_ue8m0
    _fp8_ready = True


def _use_ue8m0_scale(name: str, *, moe_deepgemm: bool = False) -> bool:
    """(:241-261) ue8m0 scales only when SGLang says DeepGEMM wants them, and for routed experts only when
    the MoE runner is DeepGEMM too."""
    if _should_ue8m0_fn is None:
        return False
    if not _should_ue8m0_fn(weight_block_size=_WEIGHT_BLOCK_SIZE):
        return False
    return moe_deepgemm if ".experts." in name else True


def should_fp8_quantize(name: str) -> bool:
    """(:269-271)"""
    return _EXPERT_RE.search(name) is not None or _FP8_DENSE_RE.search(name) is not None


def _scale_name(name: str) -> str:
    return name[:-len(".weight")] + ".weight_scale_inv"


def quantize_fp8(name: str, weight: torch.Tensor, *, moe_deepgemm: bool = False) -> list[tuple[str, torch.Tensor]]:
    """(:274-321) One weight -> [(name, e4m3fn weight), (name.weight_scale_inv, scale)], quantised from the bf16
    view of the master (what the QAT forward sees), 128 x 128 blocks over the tensor viewed as (-1, last)."""
    _init_fp8_quantizers()
    assert name.endswith(".weight"), f"Expected .weight suffix, got {name!r}"
    weight = weight.bfloat16().float().contiguous()
    if weight.dim() == 1:
        raise ValueError(f"Cannot FP8-quantize 1D weight {name!r}")
    w2 = weight.view(-1, weight.shape[-1])
    ue8m0 = _use_ue8m0_scale(name, moe_deepgemm=moe_deepgemm) and _quant_weight_ue8m0_fn is not None
    if ue8m0 or _per_block_cast_fn is None:
        qweight, scale = _quant_weight_ue8m0_fn(w2, weight_block_size=_WEIGHT_BLOCK_SIZE)
        scale = _transform_scale_ue8m0_fn(scale, mn=qweight.shape[-2])
    else:
        qweight, scale = _per_block_cast_fn(w2)
    return [(name, qweight.view_as(weight).contiguous()), (_scale_name(name), scale)]


def quantize_fp4_qat_expert(name: str, weight: torch.Tensor, *, moe_deepgemm: bool = False) -> list[tuple[str, torch.Tensor]]:
    """(:324-352) Routed expert under FP4 QAT: e2m1 1 x 32 on the bf16 view of the master, rebased to e4m3fn with
    one scale per 128 x 128 tile by the fused kernel; float32 scales unless the DeepGEMM layout is asked for."""
    assert _EXPERT_RE.search(name) is not None, f"Expected routed expert key, got {name!r}"
    assert name.endswith(".weight"), f"Expected .weight suffix, got {name!r}"
    qweight, fp8_scale = fp4_qat_then_to_fp8(weight.bfloat16().float())
    scale = fp8_scale.float()
    if moe_deepgemm:
        _init_fp8_quantizers()
        if _use_ue8m0_scale(name, moe_deepgemm=True):
            assert _transform_scale_ue8m0_fn is not None
            scale = _transform_scale_ue8m0_fn(fp8_scale, mn=qweight.shape[-2])
    return [(name, qweight), (_scale_name(name), scale.contiguous())]


def simulate_fp8_wo_a(name: str, weight: torch.Tensor) -> list[tuple[str, torch.Tensor]]:
    """(:355-372) wo_a stays bf16 in the sampler: push the values of the trainer's 128 x 128 FP8 fake-quantiser
    (e4m3 codes times a power of two are exact in bf16)."""
    assert _WO_A_RE.search(name) is not None, f"Expected wo_a key, got {name!r}"
    from .qat import fp8_simulate_qat_128x128

    return [(name, fp8_simulate_qat_128x128(weight.bfloat16()).contiguous())]


def iter_fp8_quantized_weights(weights: Iterator[tuple[str, torch.Tensor]], *, moe_deepgemm: bool = False,
                               fp4_qat: bool = False) -> Iterator[tuple[str, torch.Tensor]]:
    """(:375-418) The per-key rule: FP4-QAT experts and wo_a first (when fp4_qat), then the FP8 whitelist,
    everything else unchanged; a `.scale` key in the input is an error (the stream must be bf16)."""
    for name, tensor in weights:
        if name.endswith(".scale"):
            raise RuntimeError(f"FP8 sglang quantization expects bf16 weight keys, got scale key {name!r}")
        if fp4_qat and _EXPERT_RE.search(name) is not None:
            yield from quantize_fp4_qat_expert(name, tensor, moe_deepgemm=moe_deepgemm)
        elif fp4_qat and _WO_A_RE.search(name) is not None:
            yield from simulate_fp8_wo_a(name, tensor)
        elif should_fp8_quantize(name):
            yield from quantize_fp8(name, tensor, moe_deepgemm=moe_deepgemm)
        else:
            yield name, tensor
