"""MI355X drop-in for tools/dsv4_quant_and_dequant/compare_hf_ckpts.py: compare two DeepSeek-V4 HF checkpoints, dtypes
first, then values after each side's own dequantisation (FP4 / FP8 / `.scale` aware).

    python -m gcore_lowp.compare_hf_ckpts --a <dir> --b <dir> [--a-name A --b-name B] [--dtype-only]

Same report as the reference tool: key coverage (only in A / only in B / index entries whose shard lacks the key),
dtype-pair and role x dtype histograms, shape mismatches, and per normalised key (experts.N -> experts.E) the
count, raw-byte equality, worst max-abs-diff / cosine / relative error, with [DIFF] lines for tensors outside
--cos-tol / --abs-tol (quantised) or --plain-tol (plain).  The reference spreads the keys over MPI ranks, one GPU
each (compare_hf_ckpts.py:67-103,283-458); this build is one process on one GPU and walks the keys in order.  The
dequantisation runs on the HIP kernels (dsv4_kernels.dequant_fp8_block); the metrics are torch reductions.
The verdict follows the reference (:452-453): consistent when no compared tensor is out of tolerance and neither side
has keys the other lacks (raw shapes and dtypes may differ between the two layouts); it is also the exit status.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time
from collections import Counter, OrderedDict

import torch

from . import _abi as A
from .dsv4_kernels import dequant_fp8_block, is_expert_weight, is_wo_a_weight, scale_key

FP8 = torch.float8_e4m3fn


def _norm_key(k: str) -> str:
    return re.sub(r"experts\.\d+\.", "experts.E.", k)


def _role(k: str, dtype: torch.dtype) -> str:
    """(:109-118)"""
    if k.endswith(".scale"):
        return f"scale/{dtype}"
    if is_expert_weight(k):
        return f"expert/{dtype}"
    if is_wo_a_weight(k):
        return f"wo_a/{dtype}"
    return f"dense_fp8/{dtype}" if dtype == FP8 else f"other/{dtype}"


def _metrics(a: torch.Tensor, b: torch.Tensor):
    """(:149-158) max |a - b|, cosine, |a - b| / |a| on the flattened fp32 tensors"""
    a, b = a.float().reshape(-1), b.float().reshape(-1)
    if a.numel() != b.numel():
        return float("inf"), 0.0, float("inf")
    if a.numel() == 0:
        return 0.0, 1.0, 0.0
    d = a - b
    na, nb = a.norm(), b.norm()
    return d.abs().max().item(), float(torch.dot(a, b) / (na * nb + 1e-12)), float(d.norm() / (na + 1e-12))


class HF:
    """One checkpoint directory: index, lazily opened shards (:161-194)."""

    def __init__(self, d: str):
        from safetensors import safe_open
        self._open_fn = safe_open
        self.dir = d
        with open(os.path.join(d, "model.safetensors.index.json")) as f:
            self.wm = json.load(f)["weight_map"]
        self._shards, self._keys = {}, {}

    def _shard(self, fname):
        if fname not in self._shards:
            self._shards[fname] = self._open_fn(os.path.join(self.dir, fname), framework="pt", device="cpu")
            self._keys[fname] = set(self._shards[fname].keys())
        return self._shards[fname]

    def has(self, k: str) -> bool:
        if k not in self.wm:
            return False
        try:
            self._shard(self.wm[k])
            return k in self._keys[self.wm[k]]
        except Exception:                                   # noqa: BLE001 -- a broken shard counts as "not there"
            return False

    def raw(self, k: str) -> torch.Tensor:
        return self._shard(self.wm[k]).get_tensor(k)

    def scale_of(self, k: str):
        sk = scale_key(k)
        return self.raw(sk) if self.has(sk) else None

    def present(self):
        ok = {k for k in self.wm if self.has(k)}
        return ok, sorted(set(self.wm) - ok)


def _deq(k, w, scale, dev):
    """(:197-202) float32 value of a raw tensor: quantised weights through their scale, anything else cast"""
    w = w.to(dev)
    if k.endswith(".weight") and scale is not None and w.dtype in (FP8, torch.int8):
        return dequant_fp8_block(w, scale.to(dev)).float()
    return w.float()


def dtype_probe(keys, ca: HF, cb: HF):
    """(:219-236)"""
    pairs, roles, shapes = Counter(), Counter(), []
    for k in keys:
        try:
            a, b = ca.raw(k), cb.raw(k)
            pairs[(str(a.dtype), str(b.dtype))] += 1
            roles[(_role(k, a.dtype), str(a.dtype), str(b.dtype))] += 1
            if tuple(a.shape) != tuple(b.shape):
                shapes.append(f"{k}: {tuple(a.shape)} vs {tuple(b.shape)}")
        except Exception as ex:                             # noqa: BLE001
            shapes.append(f"{k}: {type(ex).__name__}: {ex}")
    return pairs, roles, shapes


def compare_values(keys, ca: HF, cb: HF, dev, cos_tol, abs_tol, plain_tol):
    """(:239-280) per normalised key: n, raw_equal, bad, max_abs_diff, min_cos, max_rel; plus report lines"""
    stats, reports = OrderedDict(), []
    for k in keys:
        if k.endswith(".scale"):
            continue
        st = stats.setdefault(_norm_key(k), {"n": 0, "raw_equal": 0, "bad": 0, "max_abs_diff": 0.0, "min_cos": 1.0,
                                             "max_rel": 0.0})
        try:
            ra, rb = ca.raw(k), cb.raw(k)
            wk = k.endswith(".weight")
            va = _deq(k, ra, ca.scale_of(k) if wk else None, dev)
            vb = _deq(k, rb, cb.scale_of(k) if wk else None, dev)
            quant = ra.dtype in (FP8, torch.int8) or rb.dtype in (FP8, torch.int8) or ra.dtype != rb.dtype
            mad, cos, rel = _metrics(va, vb)
            bad = (cos < cos_tol or mad > abs_tol) if quant else mad > plain_tol
            same = ra.dtype == rb.dtype and tuple(ra.shape) == tuple(rb.shape)
            raw_eq = same and bool(torch.equal(ra.view(torch.uint8), rb.view(torch.uint8)) if ra.dtype == FP8
                                   else torch.equal(ra, rb))
            st["n"] += 1
            st["raw_equal"] += int(raw_eq)
            st["bad"] += int(bad)
            st["max_abs_diff"] = max(st["max_abs_diff"], mad)
            st["min_cos"] = min(st["min_cos"], cos)
            st["max_rel"] = max(st["max_rel"], rel)
            if bad and len(reports) < 500:
                reports.append(f"[DIFF] {k} dtype=({ra.dtype},{rb.dtype}) shape=({tuple(ra.shape)},{tuple(rb.shape)}) "
                               f"mad={mad:.4g} cos={cos:.6f} rel={rel:.4g}")
        except Exception as ex:                             # noqa: BLE001
            st["bad"] += 1
            if len(reports) < 500:
                reports.append(f"[ERROR] {k}: {type(ex).__name__}: {ex}")
    return stats, reports


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--a", required=True, help="first HF ckpt dir")
    ap.add_argument("--b", required=True, help="second HF ckpt dir")
    ap.add_argument("--a-name", default="A")
    ap.add_argument("--b-name", default="B")
    ap.add_argument("--cos-tol", type=float, default=0.999)
    ap.add_argument("--abs-tol", type=float, default=1e-2)
    ap.add_argument("--plain-tol", type=float, default=1e-6)
    ap.add_argument("--jobs", "-j", type=int, default=8, help="accepted for compatibility; this build is one process")
    ap.add_argument("--dtype-only", action="store_true", help="coverage / dtype / shape report only")
    ap.add_argument("--max-report", type=int, default=50)
    ap.add_argument("--device", default="cuda", choices=("cuda", "cpu"), help="only cuda (the MI355X) is available")
    args = ap.parse_args(argv)
    if args.device != "cuda" and not args.dtype_only:
        raise RuntimeError("this build compares on the GPU only: --device cpu is not available")
    t0 = time.time()
    ca, cb = HF(args.a), HF(args.b)
    pa, miss_a = ca.present()
    pb, miss_b = cb.present()
    shared = sorted(pa & pb)
    print(f"[cmp] {args.a_name}={args.a}\n[cmp] {args.b_name}={args.b}")
    print(f"[cmp] keys: {args.a_name}={len(pa)} {args.b_name}={len(pb)} shared={len(shared)} "
          f"only_{args.a_name}={len(pa - pb)} only_{args.b_name}={len(pb - pa)} "
          f"phantom_{args.a_name}={len(miss_a)} phantom_{args.b_name}={len(miss_b)}")
    for tag, ks in ((f"only in {args.a_name}", sorted(pa - pb)), (f"only in {args.b_name}", sorted(pb - pa)),
                    (f"phantom in {args.a_name}", miss_a), (f"phantom in {args.b_name}", miss_b)):
        for k in ks[:args.max_report]:
            print(f"  [{tag}] {k}")
    pairs, roles, shapes = dtype_probe(shared, ca, cb)
    print("[cmp] dtype pairs:")
    for (da, db), n in sorted(pairs.items()):
        print(f"  {da:24s} {db:24s} {n}")
    print("[cmp] role x dtype pairs:")
    for (role, da, db), n in sorted(roles.items()):
        print(f"  {role:32s} {da:24s} {db:24s} {n}")
    for line in shapes[:args.max_report]:
        print(f"  [SHAPE] {line}")
    failed = bool(pa ^ pb)
    if not args.dtype_only:
        dev = A.require_gpu()
        stats, reports = compare_values(shared, ca, cb, dev, args.cos_tol, args.abs_tol, args.plain_tol)
        print("[cmp] values (per normalised key): n raw_equal bad max_abs_diff min_cos max_rel")
        for nk, st in stats.items():
            print(f"  {nk:64s} {st['n']:5d} {st['raw_equal']:5d} {st['bad']:5d} {st['max_abs_diff']:.4g} "
                  f"{st['min_cos']:.6f} {st['max_rel']:.4g}")
        for line in reports[:args.max_report]:
            print(line)
        n_bad = sum(st["bad"] for st in stats.values())
        print(f"[cmp] tensors compared={sum(st['n'] for st in stats.values())} bad={n_bad}")
        failed = failed or n_bad > 0
    print(f"[cmp] elapsed={time.time() - t0:.1f}s")
    print("VERDICT: PROBLEMS FOUND" if failed else "VERDICT: ALL CONSISTENT")
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main())
