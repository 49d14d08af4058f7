"""MI355X drop-in for tools/dsv4_quant_and_dequant/convert.py: DeepSeek-V4-Flash checkpoints between the official
layout (FP4 experts + e8m0 scales) and the SGLang FP8 layout (FP8 experts + fp32 scales).

    python -m gcore_lowp.dsv4_convert --direction official2sgl --src <dir> --dst <dir>

Same flags, same per-weight rules (convert.py:189-245), same outputs (shard names, `.scale` keys, HF index
with total_size, aux files, `expert_dtype` in config.json) as the reference driver.  What differs is the
machinery: the reference spreads shards over MPI ranks, one GPU each; this build runs on one GPU, so the
driver is a single process that walks the shards in the reference's deterministic size-balanced order
(convert.py:110-122 with world = 1) and keeps every weight on the GPU from upload to download.  The arithmetic
is the HIP kernels of this package; `--device cpu` is refused (there is no CPU path).
"""
from __future__ import annotations

import argparse
import json
import os
import re
import shutil
import time

import torch

from . import _abi as A
from ._pipeline import run_pipelined
from .dsv4_kernels import (is_expert_weight, is_wo_a_weight, official_dense_to_sgl, official_expert_to_sgl,
                           official_wo_a_to_sgl, scale_key, sgl_dense_to_official, sgl_expert_to_official,
                           sgl_wo_a_to_official)

DIRECTIONS = ("official2sgl", "sgl2official")
_LAYER_RE = re.compile(r"^(layers\.\d+|mtp\.\d+)")


def _partition_shards(shard_sizes, world):
    """Greedy longest-processing-time packing by shard size, deterministic (convert.py:110-122)."""
    buckets = [[] for _ in range(world)]
    loads = [0] * world
    for shard, size in sorted(shard_sizes, key=lambda x: (-x[1], x[0])):
        r = min(range(world), key=lambda i: (loads[i], i))
        buckets[r].append(shard)
        loads[r] += size
    return buckets


def _copy_aux_files(src, dst):
    for name in sorted(os.listdir(src)):
        if name.endswith(".safetensors") or name == "model.safetensors.index.json":
            continue
        s, d = os.path.join(src, name), os.path.join(dst, name)
        if os.path.isdir(s):
            if os.path.exists(d):
                shutil.rmtree(d)
            shutil.copytree(s, d)
        elif os.path.isfile(s):
            shutil.copy2(s, d)


def _update_config(src, dst, direction):
    cfg_path = os.path.join(src, "config.json")
    if not os.path.isfile(cfg_path):
        return
    with open(cfg_path) as f:
        cfg = json.load(f)
    if direction == "official2sgl":
        cfg.pop("expert_dtype", None)
    else:
        cfg["expert_dtype"] = "fp4"
    with open(os.path.join(dst, "config.json"), "w") as f:
        json.dump(cfg, f, indent=2, ensure_ascii=False)
        f.write("\n")


def convert_one_weight(name, weight, scale, direction):
    """One checkpoint weight (and its scale, if it has one) -> the tensors written for it (convert.py:189-245)."""
    out = {}
    if direction == "official2sgl":
        if is_expert_weight(name):
            assert scale is not None, f"missing scale for expert {name}"
            assert weight.dtype == torch.int8, (name, weight.dtype)
            out[name], out[scale_key(name)] = official_expert_to_sgl(weight, scale)
        elif is_wo_a_weight(name):
            assert scale is not None, f"missing scale for wo_a {name}"
            out[name] = official_wo_a_to_sgl(weight, scale)
        elif scale is not None and weight.dtype == torch.float8_e4m3fn:
            out[name], out[scale_key(name)] = official_dense_to_sgl(weight, scale)
        else:
            out[name] = weight
            if scale is not None:
                out[scale_key(name)] = scale
        return out
    if is_expert_weight(name):
        assert scale is not None, f"missing scale for expert {name}"
        assert weight.dtype == torch.float8_e4m3fn, (name, weight.dtype)
        out[name], out[scale_key(name)] = sgl_expert_to_official(weight, scale)
    elif is_wo_a_weight(name):
        if weight.dtype == torch.bfloat16:
            out[name], out[scale_key(name)] = sgl_wo_a_to_official(weight)
        elif scale is not None and weight.dtype == torch.float8_e4m3fn:
            out[name], out[scale_key(name)] = sgl_dense_to_official(weight, scale)
        else:
            raise TypeError(f"unexpected wo_a dtype {weight.dtype} for {name}")
    elif scale is not None and weight.dtype == torch.float8_e4m3fn:
        out[name], out[scale_key(name)] = sgl_dense_to_official(weight, scale)
    else:
        out[name] = weight
        if scale is not None:
            out[scale_key(name)] = scale.to(torch.float8_e8m0fnu) if scale.dtype == torch.float32 else scale
    return out


def _needs_gpu(name, weight, scale, direction):
    """True when the rule for this weight runs a kernel (convert.py:248-266)."""
    if direction == "official2sgl":
        return is_expert_weight(name) or is_wo_a_weight(name)
    if is_expert_weight(name):
        return True
    return is_wo_a_weight(name) and weight.dtype == torch.bfloat16


def _process_shard(src, dst, shard_name, direction, weight_map, dev):
    from safetensors import safe_open
    from safetensors.torch import save_file

    handles = {}

    def scale_of(sk):
        fname = weight_map.get(sk)
        if fname is None:
            return None
        if fname not in handles:
            handles[fname] = safe_open(os.path.join(src, fname), framework="pt", device="cpu")
        return handles[fname].get_tensor(sk) if sk in handles[fname].keys() else None

    out, n_conv, n_pass = {}, 0, 0

    def jobs():
        with safe_open(os.path.join(src, shard_name), framework="pt", device="cpu") as sf:
            for name in sf.keys():
                if name.endswith(".scale"):
                    continue
                tensor = sf.get_tensor(name)
                if not name.endswith(".weight"):
                    yield (name, False, False), (tensor,), False
                    continue
                scale = scale_of(scale_key(name))
                yield (name, True, scale is not None), (tensor, scale), _needs_gpu(name, tensor, scale, direction)

    def compute(tag, tensors):
        name, is_weight, _ = tag
        return convert_one_weight(name, tensors[0], tensors[1], direction) if is_weight else {name: tensors[0]}

    if os.environ.get("LP_CONVERT_PIPELINE", "1") != "0":
        stream = run_pipelined(dev, jobs(), compute)
    else:                                             # one tensor at a time, every copy synchronous (for comparison)
        stream = ((tag, {k: v.cpu() for k, v in compute(tag, [t.to(dev) if on_gpu and t is not None else t
                                                               for t in host]).items()})
                  for tag, host, on_gpu in jobs())
    for (name, is_weight, has_scale), conv in stream:
        out.update({k: v.contiguous() for k, v in conv.items()})
        if not is_weight or (list(conv.keys()) == [name] and not has_scale):
            n_pass += 1
        else:
            n_conv += 1
    handles.clear()
    if not out:
        return {}, 0, n_conv, n_pass
    save_file(out, os.path.join(dst, shard_name))
    return {k: shard_name for k in out}, sum(t.numel() * t.element_size() for t in out.values()), n_conv, n_pass


def convert_checkpoint(src, dst, direction, device="cuda"):
    assert direction in DIRECTIONS, direction
    if device != "cuda":
        raise RuntimeError("this build converts on the GPU only: --device cpu is not available")
    src, dst = os.path.abspath(src), os.path.abspath(dst)
    assert src != dst, "src and dst must differ"
    dev = A.require_gpu()
    t0 = time.time()
    with open(os.path.join(src, "model.safetensors.index.json")) as f:
        weight_map = json.load(f)["weight_map"]
    shards = sorted(set(weight_map.values()))
    order = _partition_shards([(s, os.path.getsize(os.path.join(src, s))) for s in shards], 1)[0]
    print(f"[convert] direction={direction}\n[convert] src={src}\n[convert] dst={dst}\n"
          f"[convert] shards={len(shards)} keys={len(weight_map)} world=1 device={dev}", flush=True)
    os.makedirs(dst, exist_ok=True)
    _copy_aux_files(src, dst)
    _update_config(src, dst, direction)
    out_map, total, n_conv, n_pass = {}, 0, 0, 0
    for shard in order:
        t1 = time.time()
        m, nbytes, c, p = _process_shard(src, dst, shard, direction, weight_map, dev)
        out_map.update(m)
        total += nbytes
        n_conv += c
        n_pass += p
        print(f"[convert][{direction}] shard={shard} done converted={c} passthrough={p} total={time.time() - t1:.1f}s",
              flush=True)
    with open(os.path.join(dst, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {"total_size": total}, "weight_map": out_map}, f, indent=2, sort_keys=True)
        f.write("\n")
    print(f"[convert] done: converted_weights={n_conv} passthrough={n_pass} wall={time.time() - t0:.1f}s", flush=True)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--direction", required=True, choices=DIRECTIONS, help="official2sgl | sgl2official")
    ap.add_argument("--src", required=True, help="source HF checkpoint directory")
    ap.add_argument("--dst", required=True, help="destination checkpoint directory")
    ap.add_argument("--device", default="cuda", choices=("cuda", "cpu"),
                    help="compute device; only cuda (the MI355X) is available in this build")
    args = ap.parse_args(argv)
    convert_checkpoint(args.src, args.dst, args.direction, device=args.device)


if __name__ == "__main__":
    main()
