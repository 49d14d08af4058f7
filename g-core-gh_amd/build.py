"""Builds the gfx950 C-ABI library in-tree: csrc/*.hip + api.cpp -> gcore_lowp/_lib/liblowp.so, and the
measurement / self-test aids of include/lowp_probe.h as a second library: csrc/probe/*.hip -> liblowp_probe.so.

Usage: python g-core-gh_amd/build.py [--force]
hipcc cross-compiles without a GPU.  The library links against the HIP runtime
by soname only, so that inside a PyTorch process it binds to the runtime torch
has already loaded.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIBDIR = os.path.join(HERE, "gcore_lowp", "_lib")
LIB = os.path.join(LIBDIR, "liblowp.so")
PROBE_LIB = os.path.join(LIBDIR, "liblowp_probe.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

COMMON = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off", "-fno-fast-math",
    "-Wall", "-Wno-unused-function",
    # packed-fp32 VALU ops are not trusted on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp")))


def probe_sources():
    return sorted(os.path.join("probe", f) for f in os.listdir(os.path.join(CSRC, "probe")) if f.endswith(".hip"))


def _headers_mtime():
    paths = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".h", ".inc"))]
    paths += [os.path.join(CSRC, "probe", f) for f in os.listdir(os.path.join(CSRC, "probe")) if f.endswith(".inc")]
    paths += [os.path.join(HERE, "..", "include", h) for h in ("lowp.h", "lowp_probe.h")]
    return max(os.path.getmtime(p) for p in paths)


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0].replace(os.sep, "_") + ".o")
    spath = os.path.join(CSRC, src)
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= max(os.path.getmtime(spath), _headers_mtime()):
        return obj
    audited = src in SPILL_AUDIT
    cmd = [HIPCC] + COMMON + (["-Rpass-analysis=kernel-resource-usage", "-fno-caret-diagnostics"] if audited else [])
    cmd += (["-x", "hip"] if src.endswith(".cpp") else []) + ["-c", spath, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and "kernel-resource-usage" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if audited:
        spilled = _kernels_with_scratch(r.stderr, SPILL_AUDIT[src])
        if spilled:
            os.remove(obj)
            raise RuntimeError(f"{src}: kernels that count their memory requests by hand must not spill registers "
                               f"(a spill's store and reload go through the same counter: they cost most of the rate, and "
                               f"a store that completes early can satisfy a wait meant for a request): "
                               + ", ".join(f"{n} ({b} bytes per lane)" for n, b in spilled))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


# Sources whose kernels are checked for register spills at build time (the compiler's own resource remarks), with the
# mangled-name pattern of the kernels that must have none.  gemm_thin.hip: every decode kernel (the variants that walk a
# long K in rounds are only instantiated where they need no scratch).
SPILL_AUDIT = {"gemm_thin.hip": re.compile(r"gemm_thin")}


def _kernels_with_scratch(remarks: str, pattern):
    out, name = [], None
    for line in remarks.splitlines():
        m = re.search(r"remark: Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            continue
        m = re.search(r"remark:\s+ScratchSize \[bytes/lane\]: (\d+)", line)
        if m and name and int(m.group(1)) > 0 and pattern.search(name):
            out.append((name, int(m.group(1))))
    return out


def _generate():
    """Run the generators of the hand-scheduled GEMM loops: they rewrite exactly those of its outputs (csrc/gemm_*_loop.inc)
    whose content differs from what it generates, so a stale or hand-edited file never reaches the compiler."""
    subprocess.check_call([sys.executable, os.path.join(CSRC, "gen_gemm_loop.py")])
    subprocess.check_call([sys.executable, os.path.join(CSRC, "gen_gemm_quad_loop.py")])


def _audit_asm_operands():
    """The hand-scheduled GEMM loops keep their addresses in asm operands: fail the build if the compiler placed
    one of them in a register a loop writes (csrc/check_asm_operands.py)."""
    sys.path.insert(0, CSRC)
    try:
        import check_asm_operands
    finally:
        sys.path.pop(0)
    if check_asm_operands.audit(quiet=True) != 0:
        raise RuntimeError("gemm_fp8_big.hip: an asm operand shares a register with the loop it feeds; not linking")


def build(force: bool = False) -> str:
    _generate()
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    srcs, psrcs = sources(), probe_sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs) + len(psrcs))) as ex:
        all_objs = list(ex.map(lambda s: _compile(s, force), srcs + psrcs))
    objs, pobjs = all_objs[:len(srcs)], all_objs[len(srcs):]
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        _audit_asm_operands()
        _link(LIB, objs)
    if force or not os.path.exists(PROBE_LIB) or any(os.path.getmtime(o) > os.path.getmtime(PROBE_LIB) for o in pobjs):
        _link(PROBE_LIB, pobjs)
    return LIB


def _link(lib, objs):
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link of {os.path.basename(lib)} failed:\n{r.stderr}")


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
