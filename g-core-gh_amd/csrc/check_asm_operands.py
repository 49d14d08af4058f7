"""Build-time audit of the hand-scheduled GEMM loops' register interface.

The generated loops (gemm_*_loop.inc) name their working registers literally (v30 .. v255, s40 .. s77) and take
addresses, offsets and counts as asm operands that stay live for the whole loop.  If the compiler ever assigns such an
operand to a register the loop also writes -- possible when an output is not marked early-clobber or a written
register is missing from the clobber list -- the loop overwrites its own addresses and the loads leave the buffers.
This script compiles gemm_fp8_big.hip to device assembly, finds every expansion of a loop, reads back which register
each operand received and fails when one of them is a register the loop names literally.  It also checks, in the
source, that every register a loop names is declared as an early-clobber output or a clobber of its asm statement.

Usage: python check_asm_operands.py [--quiet]     (exit status 1 on a violation)
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-fno-fast-math",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-S"]

_REG = re.compile(r"\b([vs])(?:(\d+)|\[(\d+):(\d+)\])")


def _regs(text: str) -> set[tuple[str, int]]:
    out = set()
    for m in _REG.finditer(text):
        lo = int(m.group(2) if m.group(2) is not None else m.group(3))
        hi = int(m.group(2) if m.group(2) is not None else m.group(4))
        out.update((m.group(1), r) for r in range(lo, hi + 1))
    return out


def load_template(path: str):
    """-> (list of per-line regexes with one named group per operand use, set of literally named registers)."""
    lines = []
    with open(path) as f:
        for raw in f:
            raw = raw.strip()
            if raw.startswith('"') and raw.endswith('\\n"'):
                lines.append(raw[1:-3])
    literal: set[tuple[str, int]] = set()
    patterns = []
    for text in lines:
        literal |= _regs(re.sub(r"%\[\w+\]", " ", text))
        if re.search(r"\bvcc", text) or re.search(r"\bv_(?:add_co|addc_co|sub_co|subb_co|div_scale|cmpx?_\w+(?<!_e64)\s)", text):
            raise RuntimeError(f"{path}: the loop uses vcc, which the compiler may assign to a scalar operand: {text}")
        parts = re.split(r"(%\[\w+\])", text)
        rx, n = "", 0
        for p in parts:
            if p.startswith("%["):
                # the compiler may hand a scalar operand vcc (a loop that names vcc fails in load_template)
                rx += rf"(?P<{p[2:-1]}__{n}>[vs](?:\d+|\[\d+:\d+\])|vcc(?:_lo|_hi)?)"
                n += 1
            else:
                rx += r"\s+".join(re.escape(w) for w in p.split(" ")).replace("%=", r"\d+") if p else ""
        patterns.append(re.compile(r"^\s*" + rx + r"\s*$"))
    return patterns, literal


def declared_registers(hip_path: str) -> dict[str, set[tuple[str, int]]]:
    """Per loop file: the registers its asm statement in the .hip source declares as outputs or clobbers."""
    with open(hip_path) as f:
        src = f.read()
    macros = {m.group(1): m.group(2) for m in re.finditer(r"#define (LP_ASM_CLOBBERS\w*)\b(.*?)(?=\n#define)", src, re.S)}
    out = {}
    for m in re.finditer(r'#include "(\w+_loop\.inc)"(.*?)\);', src, re.S):
        text = re.sub(r"LP_ASM_CLOBBERS\w*", lambda k: macros[k.group(0)], m.group(2))
        regs = set()
        for q in re.findall(r'"=&\{(v\[\d+:\d+\])\}"', text):
            regs |= _regs(q)
        for q in re.findall(r'"([vs]\d+)"', text):
            regs |= _regs(q)
        out[m.group(1)] = regs
    return out


def asm_blocks(asm_text: str):
    """-> list of (kernel symbol, body lines) for every inline-asm expansion."""
    kernel, body, out = None, None, []
    for line in asm_text.splitlines():
        m = re.match(r"^(\w+):", line)
        if m and body is None:
            kernel = m.group(1)
        if "ASMSTART" in line:
            body = []
        elif "ASMEND" in line:
            if body is not None:
                out.append((kernel, body))
            body = None
        elif body is not None and line.strip():
            body.append(line)
    return out


def accumulation_registers_outside_asm(asm_text: str, kernel_substr: str) -> list[str]:
    """Lines of the kernels whose symbol contains kernel_substr that name an accumulation register (a0 .. a255) outside the
    inline-asm expansions.  The four-wave loop keeps its accumulators there across two asm statements; the compiler is
    told they are clobbered, and must not put anything of its own (a spill, say) into them in between."""
    out, kernel, inside = [], "", False
    for line in asm_text.splitlines():
        m = re.match(r"^(\w+):", line)
        if m and not inside:
            kernel = m.group(1)
        if "ASMSTART" in line:
            inside = True
        elif "ASMEND" in line:
            inside = False
        elif not inside and kernel_substr in kernel:
            code = line.split(";")[0].strip()
            if code and not code.startswith(".") and re.search(r"\ba(?:\d+|\[\d+:\d+\])", code):
                out.append(f"{kernel}: {code}")
    return out


def audit(quiet: bool = False) -> int:
    templates = {f: load_template(os.path.join(HERE, f)) for f in sorted(os.listdir(HERE)) if f.endswith("_loop.inc")}
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "big.s")
        r = subprocess.run([HIPCC] + FLAGS + [os.path.join(HERE, "gemm_fp8_big.hip"), "-o", out], capture_output=True, text=True)
        if r.returncode != 0:
            sys.stderr.write(r.stderr)
            return 2
        with open(out) as f:
            asm_text = f.read()
        blocks = asm_blocks(asm_text)
    bad = checked = 0
    for line in accumulation_registers_outside_asm(asm_text, "gemm_asm_quad"):
        print(f"FAIL accumulation register used outside the asm statements: {line}")
        bad += 1
    declared = declared_registers(os.path.join(HERE, "gemm_fp8_big.hip"))
    for name, (_, literal) in templates.items():
        if name not in declared:
            print(f"FAIL {name}: no asm statement includes it")
            bad += 1
        elif literal - declared[name]:
            missing = sorted(f"{k}{n}" for k, n in literal - declared[name])
            print(f"FAIL {name}: the loop names registers that are neither early-clobber outputs nor clobbers: {' '.join(missing)}")
            bad += 1
    for kernel, body in blocks:
        if len(body) < 100:
            # Small statements: the compiler inserts the wait states a lane-crossing read of a vector register needs after
            # the instruction that writes it, but not across the border of an asm statement.  A statement whose first
            # instruction is such a read must bring its own (s_nop in front): without it v_readfirstlane has returned the
            # register's previous value whenever the scheduler put the producing v_mov right in front of the statement.
            first = next((l.strip() for l in body if l.strip() and not l.strip().startswith(";")), "")
            if re.match(r"v_(readfirstlane|readlane|permlane|writelane)", first) or " dpp" in first or "row_" in first:
                print(f"FAIL {kernel}: an asm statement starts with a lane-crossing instruction without wait states: {first}")
                bad += 1
            continue
        match = None
        for name, (patterns, literal) in templates.items():
            if len(patterns) != len(body):
                continue
            groups = []
            for p, line in zip(patterns, body):
                m = p.match(line)
                if m is None:
                    groups = None
                    break
                groups.append(m.groupdict())
            if groups is not None:
                match = (name, literal, groups)
                break
        if match is None:
            print(f"FAIL {kernel}: an asm block of {len(body)} lines matches no loop template")
            bad += 1
            continue
        name, literal, groups = match
        operands: dict[str, set[str]] = {}
        for g in groups:
            for key, reg in g.items():
                operands.setdefault(key.split("__")[0], set()).add(reg)
        checked += 1
        clash = {op: regs for op, regs in operands.items() if any(_regs(r) & literal for r in regs)}
        if clash:
            bad += 1
            print(f"FAIL {kernel} ({name}): operands in registers the loop writes: "
                  + ", ".join(f"{op}={'/'.join(sorted(regs))}" for op, regs in sorted(clash.items())))
        elif not quiet:
            print(f"ok   {kernel} ({name}): " + " ".join(f"{op}={'/'.join(sorted(regs))}" for op, regs in sorted(operands.items())))
    if checked == 0:
        print("FAIL: no loop expansion found in the device assembly")
        return 1
    print(f"{checked} loop expansions audited, {bad} failures")
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(audit(quiet="--quiet" in sys.argv))
