"""bf16 HF checkpoint -> block-wise FP8 (e4m3, 128 x 128, `<weight>_scale_inv` fp32) checkpoint; MI355X drop-in for
tools/convert_fp8/bf16_cast_fp8.py (same flags, shard names, `_scale_inv` keys, index and side files).

    python -m gcore_lowp.bf16_cast_fp8 --input-bf16-hf-path <dir> --output-fp8-hf-path <dir> [--input-fp8-hf-path <dir>]

With --input-fp8-hf-path the set of weights to quantise is read off a reference FP8 checkpoint (every 1-byte weight
that has a `_scale_inv` there; :171-221) and that checkpoint's *.json / *.py files are copied; without it the
bf16 checkpoint's side files are copied, `quantization_config` is written into config.json and `is_fp8_params`
decides per name.

The reference imports `is_fp8_params`, `FP8_BLOCK_QUANT_KWARGS` and `fp8_weight_block_wise_quant` from
`gpatch.core.fp8_utils.fp8`, which is not part of its tree.  What stands in for them here -- parity UNPINNED for
all three:
  * fp8_weight_block_wise_quant: scale_inv = amax / 448 per 128 x 128 tile (1.0 for an all-zero tile), codes =
    e4m3(clamp(w / scale_inv)); edge tiles of a matrix whose sides are not multiples of 128 are completed with
    zeros, so scale_inv has ceil(rows / 128) x ceil(cols / 128) entries (the layout of the published DeepSeek-V3
    FP8 checkpoints).
  * is_fp8_params: two-dimensional projection weights (`*_proj.weight`) outside `lm_head`, embeddings, norms and the
    router; override with --quant-regex.
  * FP8_BLOCK_QUANT_KWARGS: the `quantization_config` of the published DeepSeek-V3 config.json.
One shard is resident at a time; tensors go through the converters' host/device pipeline.
"""
from __future__ import annotations

import json
import os
import re
import shutil
from argparse import ArgumentParser
from glob import glob

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from . import _abi as A
from . import ops
from ._pipeline import run_pipelined

FP8_BLOCK_QUANT_KWARGS = {"activation_scheme": "dynamic", "fmt": "e4m3", "quant_method": "fp8", "weight_block_size": [128, 128]}
INDEX = "model.safetensors.index.json"
REF_MAP = "weight_with_scale_inv_map.index.json"
_DEFAULT_QUANT_RE = re.compile(r"_proj\.weight$")
_NEVER_QUANT_RE = re.compile(r"(^|\.)(lm_head|embed_tokens|embed)\.|norm|\.mlp\.gate\.weight$")


def is_fp8_params(name: str, pattern: re.Pattern | None = None) -> bool:
    if _NEVER_QUANT_RE.search(name):
        return False
    return (pattern or _DEFAULT_QUANT_RE).search(name) is not None


def fp8_weight_block_wise_quant(weight: torch.Tensor, block: int = 128):
    """[R, C] bf16/fp32 on the GPU -> (e4m3fn [R, C], fp32 scale_inv [ceil(R/block), ceil(C/block)])."""
    assert weight.dim() == 2, tuple(weight.shape)
    rows, cols = weight.shape
    pr, pc = -rows % block, -cols % block
    w = torch.nn.functional.pad(weight, (0, pc, 0, pr)) if pr or pc else weight
    q, s, _ = ops.quant_fp8_block(w, (block, block), scale_mode=A.SCALE_DIV, scale_dtype=torch.float32,
                                  amax_floor=0.0, zero_rule=A.ZERO_SCALE_TO_ONE)
    return (q[:rows, :cols].contiguous() if pr or pc else q), s


def _copy_side_files(src: str, dst: str) -> None:
    for item in os.listdir(src):
        if item.endswith((".json", ".py")):
            print(f"Copy {os.path.join(src, item)} to {os.path.join(dst, item)}.")
            shutil.copy(os.path.join(src, item), os.path.join(dst, item))


def _weight_map(path: str) -> dict[str, str]:
    index = os.path.join(path, INDEX)
    if os.path.exists(index):
        with open(index) as f:
            return json.load(f)["weight_map"]
    files = glob(os.path.join(path, "*.safetensors"))
    assert len(files) == 1, f"Expected 1 file, got {len(files)}"
    with safe_open(files[0], framework="pt", device="cpu") as f:
        return {key: os.path.basename(files[0]) for key in f.keys()}


def read_weight_inv_list(input_fp8_path: str, output_fp8_path: str) -> dict[str, str]:
    """Which weights of a reference FP8 checkpoint carry a `_scale_inv`: {weight: shard of its scale}, also written
    to weight_with_scale_inv_map.index.json in the output directory (:171-221).  Only headers are read."""
    weight_map = _weight_map(input_fp8_path)
    found: dict[str, str] = {}
    for shard in sorted(glob(os.path.join(input_fp8_path, "*.safetensors"))):
        with safe_open(shard, framework="pt", device="cpu") as f:
            for name in f.keys():
                if name.endswith("_scale_inv"):
                    continue
                if f.get_slice(name).get_dtype() not in ("F8_E4M3", "F8_E5M2", "I8", "U8", "BOOL"):
                    continue
                if f"{name}_scale_inv" in weight_map:
                    found[name] = weight_map[f"{name}_scale_inv"]
                else:
                    print(f"Warning: Missing scale_inv tensor for {name}, skipping conversion")
    with open(os.path.join(output_fp8_path, REF_MAP), "w") as f:
        json.dump({"metadata": {}, "weight_with_scale_inv_map": found}, f, indent=2)
    return found


def update_quant_model_config(fp8_path: str) -> None:
    """config.json gains quantization_config (lm_head excluded); plain JSON, no model classes are loaded (:161-168)."""
    path = os.path.join(fp8_path, "config.json")
    if not os.path.exists(path):
        return
    with open(path) as f:
        cfg = json.load(f)
    cfg["quantization_config"] = dict(FP8_BLOCK_QUANT_KWARGS, modules_to_not_convert=["lm_head"])
    with open(path, "w") as f:
        json.dump(cfg, f, indent=2, sort_keys=True)
        f.write("\n")


def main(bf16_path: str, fp8_path: str, ref_weights_scale_inv_map: dict | None = None, quant_regex: str | None = None):
    """:58-156.  A tensor of >= 2 bytes per element is quantised when the reference map lists it (map given) or
    is_fp8_params accepts it (no map); everything else is copied."""
    dev = A.require_gpu()
    os.makedirs(fp8_path, exist_ok=True)
    weight_map = dict(_weight_map(bf16_path))
    pattern = re.compile(quant_regex) if quant_regex else None
    scale_home: dict[str, str] = {}
    for shard in sorted(glob(os.path.join(bf16_path, "*.safetensors"))):
        shard_name = os.path.basename(shard)

        def wanted(name, itemsize, ndim):
            if itemsize < 2:
                print(f"[SKIP] non_fp8 {name} ...")
                return False
            if ref_weights_scale_inv_map is not None:
                return ndim == 2 and ref_weights_scale_inv_map.get(name) is not None
            if ndim == 2 and is_fp8_params(name, pattern):
                return True
            print(f"[SKIP] non_quant {name} ...")
            return False

        def jobs(shard=shard):
            with safe_open(shard, framework="pt", device="cpu") as f:
                for name in f.keys():
                    t = f.get_tensor(name)
                    q = wanted(name, t.element_size(), t.dim())
                    yield (name, q), (t,), q

        def compute(tag, tensors):
            name, q = tag
            if not q:
                return {name: tensors[0]}
            codes, scale_inv = fp8_weight_block_wise_quant(tensors[0])
            return {name: codes, f"{name}_scale_inv": scale_inv}

        out = {}
        for (name, q), res in run_pipelined(dev, jobs(), compute):
            out.update({k: v.contiguous() for k, v in res.items()})
            if q:
                scale_home[f"{name}_scale_inv"] = shard_name
        save_file(out, os.path.join(fp8_path, shard_name))
    weight_map.update(scale_home)
    with open(os.path.join(fp8_path, INDEX), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f, indent=2)


def cli(argv=None):
    parser = ArgumentParser(description=__doc__.split("\n\n")[0])
    parser.add_argument("--input-bf16-hf-path", type=str, required=False)
    parser.add_argument("--output-fp8-hf-path", type=str, required=False)
    parser.add_argument("--input-fp8-hf-path", type=str, required=False)
    parser.add_argument("--quant-regex", type=str, default=None,
                        help="which weight names to quantise when no reference FP8 checkpoint is given")
    args = parser.parse_args(argv)
    assert args.output_fp8_hf_path is not None, "output_fp8_hf_path is required"
    assert args.input_bf16_hf_path is not None, "input_bf16_hf_path is required"
    if not os.path.exists(args.output_fp8_hf_path):
        os.mkdir(args.output_fp8_hf_path)
        print(f"Creating output_fp8_hf_path: {args.output_fp8_hf_path}")
    ref_map = None
    if args.input_fp8_hf_path is not None:
        ref_map = read_weight_inv_list(args.input_fp8_hf_path, args.output_fp8_hf_path)
        _copy_side_files(args.input_fp8_hf_path, args.output_fp8_hf_path)
    else:
        _copy_side_files(args.input_bf16_hf_path, args.output_fp8_hf_path)
        update_quant_model_config(args.output_fp8_hf_path)
    main(args.input_bf16_hf_path, args.output_fp8_hf_path, ref_weights_scale_inv_map=ref_map, quant_regex=args.quant_regex)


if __name__ == "__main__":
    cli()
