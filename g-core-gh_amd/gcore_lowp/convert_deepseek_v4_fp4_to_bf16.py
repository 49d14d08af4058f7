"""MI355X drop-in for tools/convert_deepseek_v4_fp4_to_bf16.py: the two cast functions and the converter
around them (python -m gcore_lowp.convert_deepseek_v4_fp4_to_bf16 --hf-ckpt-path ... --save-path ...)."""
from __future__ import annotations

import torch

from . import ops

__all__ = ["cast_e2m1fn_to_bf16", "cast_e4m3fn_to_bf16", "main"]


def cast_e2m1fn_to_bf16(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """tools/convert_deepseek_v4_fp4_to_bf16.py:24-46: int8-packed e2m1 [out, in/2] with an
    e8m0 scale per 1 x 32 block -> bf16 [out, in]; code 8 decodes to +0.0."""
    assert x.dtype == torch.int8
    assert x.ndim == 2
    out_dim, in_dim = x.size()
    in_dim *= 2
    assert in_dim % 32 == 0
    assert scale.size(0) == out_dim and scale.size(1) == in_dim // 32
    sc = scale if scale.dtype in (torch.float32, torch.bfloat16, ops.E8M0) else scale.float()
    return ops.dequant_block(x.view(torch.uint8), sc, fp4=True, fp4_neg_zero=False, out_dtype=torch.bfloat16,
                             block=(1, 32))


def cast_e4m3fn_to_bf16(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """tools/convert_deepseek_v4_fp4_to_bf16.py:51-63: e4m3fn [out, in] with a 128 x 128 block
    scale -> bf16."""
    assert x.dtype == torch.float8_e4m3fn
    assert x.ndim == 2
    out_dim, in_dim = x.size()
    assert out_dim % 128 == 0 and in_dim % 128 == 0
    assert scale.size() == (out_dim // 128, in_dim // 128)
    sc = scale if scale.dtype in (torch.float32, torch.bfloat16, ops.E8M0) else scale.float()
    return ops.dequant_block(x.view(torch.uint8), sc, fp4=False, out_dtype=torch.bfloat16, block=(128, 128))


# ---------------------------------------------------------------------------------------------
# The converter around the two casts: tools/convert_deepseek_v4_fp4_to_bf16.py:71-164, same flags, same
# output (shard names, key names, HF index with total_size, aux files copied).  The reference holds the
# whole checkpoint in host memory before it converts; here one shard at a time is resident and a weight
# whose `.scale` lives in another shard is fetched from that shard when needed.

def _parse_layers(spec):
    """'0,1,3-5' -> {0, 1, 3, 4, 5}; None keeps every layer (:142-153)."""
    if spec is None:
        return None
    out = set()
    for part in spec.split(","):
        if "-" in part:
            lo, hi = part.split("-")
            out.update(range(int(lo), int(hi) + 1))
        else:
            out.add(int(part))
    return out


def _keep(name, layers):
    if layers is not None and name.startswith("layers."):
        return int(name.split(".")[1]) in layers
    return True


def main(hf_ckpt_path, save_path, layers=None):
    """Dequantise every quantised weight of a DeepSeek-V4-Flash safetensors directory to bf16 (:71-139)."""
    import json
    import os
    import shutil
    from glob import glob

    from safetensors import safe_open
    from safetensors.torch import save_file

    from . import _abi as A
    from ._pipeline import run_pipelined

    dev = A.require_gpu()
    os.makedirs(save_path, exist_ok=True)
    files = sorted(glob(os.path.join(hf_ckpt_path, "*.safetensors")))
    where = {}                                            # key -> shard file holding it
    for path in files:
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in f.keys():
                if _keep(name, layers):
                    where[name] = path
    handles = {}

    def fetch(name):
        path = where[name]
        if path not in handles:
            handles[path] = safe_open(path, framework="pt", device="cpu")
        return handles[path].get_tensor(name)

    weight_map, total_size = {}, 0
    for path in files:
        shard = os.path.basename(path)
        out = {}

        def jobs(path=path):
            with safe_open(path, framework="pt", device="cpu") as f:
                for name in f.keys():
                    if not _keep(name, layers) or name.endswith(".scale"):
                        continue                          # scales are consumed with their weight
                    w = f.get_tensor(name)
                    scale_name = name.replace(".weight", ".scale") if name.endswith(".weight") else name + ".scale"
                    if w.dtype in (torch.int8, torch.float8_e4m3fn) and scale_name in where:
                        yield name, (w, fetch(scale_name)), True
                    else:
                        yield name, (w, None), False

        def compute(name, tensors):
            w, scale = tensors
            if scale is None:
                return {name: w}
            return {name: cast_e2m1fn_to_bf16(w, scale) if w.dtype == torch.int8 else cast_e4m3fn_to_bf16(w, scale)}

        for _, conv in run_pipelined(dev, jobs(), compute):
            out.update({k: v.contiguous() for k, v in conv.items()})
        if not out:
            continue
        save_file(out, os.path.join(save_path, shard))
        for name, t in out.items():
            weight_map[name] = shard
            total_size += t.numel() * t.element_size()
    handles.clear()
    with open(os.path.join(save_path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {"total_size": total_size}, "weight_map": weight_map}, f, indent=2, sort_keys=True)
    for item in os.listdir(hf_ckpt_path):
        src = os.path.join(hf_ckpt_path, item)
        if not os.path.isfile(src) or item.endswith(".safetensors") or item == "model.safetensors.index.json":
            continue
        shutil.copy2(src, os.path.join(save_path, item))


if __name__ == "__main__":
    from argparse import ArgumentParser

    parser = ArgumentParser()
    parser.add_argument("--hf-ckpt-path", type=str, required=True)
    parser.add_argument("--save-path", type=str, required=True)
    parser.add_argument("--layers", type=str, default=None, help="restrict to a layer subset, e.g. '0,1' or '0-2'")
    args = parser.parse_args()
    main(args.hf_ckpt_path, args.save_path, layers=_parse_layers(args.layers))
