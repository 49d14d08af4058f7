"""Drop-in for tools/convert_fp8/convert_json.py: rewrite config.json and the safetensors index of an HF checkpoint
directory when its FP8 quantisation (or its MTP layer) is removed.  No tensor data is touched.

    python -m gcore_lowp.convert_json --load_hf_dir <dir> --save_hf_dir <dir> [--remove_fp8] [--remove_mtp]
"""
from __future__ import annotations

import argparse
import json
import os


def convert_config_json(config_json, remove_fp8=False, remove_mtp=False):
    """(:15-20) drop `quantization_config` / `num_nextn_predict_layers`"""
    if remove_fp8:
        config_json.pop("quantization_config", None)
    if remove_mtp:
        config_json.pop("num_nextn_predict_layers", None)
    return config_json


def convert_index_json(index_json, remove_fp8=False, remove_mtp=False):
    """(:23-34) drop the `.weight_scale_inv` entries / the entries of layer 61 (the MTP layer) from the weight map"""
    keep = {}
    for key, fname in index_json["weight_map"].items():
        if remove_fp8 and key.endswith(".weight_scale_inv"):
            continue
        if remove_mtp and key.startswith("model.layers.61."):
            continue
        keep[key] = fname
    return {"metadata": index_json["metadata"], "weight_map": keep}


def _rewrite(load_dir, save_dir, name, fn, remove_fp8, remove_mtp):
    src, dst = os.path.join(load_dir, name), os.path.join(save_dir, name)
    assert os.path.exists(src), f"{src} does not exist"
    with open(src) as f:
        data = fn(json.load(f), remove_fp8, remove_mtp)
    with open(dst, "w") as f:
        json.dump(data, f, indent=2)
    print(f"Converted {src} to {dst} done.")


def convert_config_json_file(load_hf_dir, save_hf_dir, remove_fp8=False, remove_mtp=False):
    _rewrite(load_hf_dir, save_hf_dir, "config.json", convert_config_json, remove_fp8, remove_mtp)


def convert_index_json_file(load_hf_dir, save_hf_dir, remove_fp8=False, remove_mtp=False):
    _rewrite(load_hf_dir, save_hf_dir, "model.safetensors.index.json", convert_index_json, remove_fp8, remove_mtp)


def main(argv=None):
    ap = argparse.ArgumentParser(prog="convert_json.py", description="Convert JSON checkpoint from FP8 to FP16")
    ap.add_argument("--remove_fp8", action="store_true", help="Convert FP8 to FP16")
    ap.add_argument("--remove_mtp", action="store_true", help="Remove MTP from json")
    ap.add_argument("--load_hf_dir", required=True, help="Input hf_dir")
    ap.add_argument("--save_hf_dir", required=True, help="Output hf_dir")
    args = ap.parse_args(argv)
    convert_config_json_file(args.load_hf_dir, args.save_hf_dir, args.remove_fp8, args.remove_mtp)
    convert_index_json_file(args.load_hf_dir, args.save_hf_dir, args.remove_fp8, args.remove_mtp)


if __name__ == "__main__":
    main()
