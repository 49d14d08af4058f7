#!/usr/bin/env python3
"""Turn rocprofv3 CSV output of `bench.py` runs into the short text summaries and the traffic table under profiles/.

Inputs (each a directory that one rocprofv3 run wrote with `--output-format csv -d <dir> -o run`):
  --kernel-trace DIR   a `--kernel-trace --stats` run of `python3 bench.py --no-cpu` (graph replays, as the bench times them)
  --bench-json FILE    the JSON line that same run printed
  --pmc DIR [DIR ...]  `--pmc` runs of `python3 bench.py --no-cpu --no-graph --steps 4 --warmup 1`, one counter set each;
                       the sets may be any of the ones named in COUNTER_SETS below (a missing set leaves its columns empty)
Outputs (under --out, default profiles/):
  bench_all_configs_kernel_trace.txt, gemm_kernels_mfma_lds_hbm_counters.txt   text tables
  traffic.json   {"kernels": [{"kernel", "grid_threads", "read_bytes", "write_bytes", "fetch_size_bytes"}, ...]}: HBM-side
                 bytes per launch, which bench.py puts into `roofline.traffic`
Whatever follows a line starting with "Reading the table" in an existing summary is hand-written commentary and is kept.

Every figure is an average per dispatch over the dispatches of one kernel at one grid size (workgroups x threads): the
grid separates the configs that share a kernel.  torch's own kernels are left out; the library's bare stream kernel
(stream_probe, which reads and writes byte counts the bench chooses) is the known-size kernel the memory counters are
checked against."""
import argparse
import collections
import csv
import glob
import json
import os
import statistics
import sys

COUNTER_SETS = {
    "pipes": "SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_WAIT_INST_ANY SQ_WAIT_INST_LDS SQ_ACTIVE_INST_LDS "
             "SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE GRBM_GUI_ACTIVE",
    "instructions": "SQ_INSTS_VALU_MFMA_MOPS_F8 SQ_ACTIVE_INST_VALU SQ_ACTIVE_INST_VMEM SQ_INSTS_LDS SQ_INSTS_VMEM_RD SQ_INSTS_VALU "
                    "SQ_WAIT_ANY SQ_INSTS_SALU GRBM_GUI_ACTIVE",
    "read requests": "TCC_EA0_RDREQ_32B_sum TCC_EA0_RDREQ_64B_sum TCC_EA0_RDREQ_128B_sum TCC_EA0_RDREQ_sum",
    "fetch": "FETCH_SIZE",
    "write": "WRITE_SIZE",
}
OURS = ("gemm", "quant", "fp4", "qdq", "dequant", "probe_", "stream_probe")
VENDOR = "Cijk_"


def short(name):
    """Kernel name without namespace, return type and argument list; the vendor GEMM keeps its tile description."""
    if VENDOR in name:
        parts = name.split("_")
        keep = [p for p in parts if p.startswith(("MT", "MI", "SK", "shortname")) or p in ("F8BS", "BH", "NTD")]
        return "hipBLASLt " + "_".join(keep)
    name = name.replace("(anonymous namespace)::", "").replace("void ", "")
    return name.split("(")[0]


def wanted(name):
    return VENDOR in name or any(k in name for k in OURS) and "at::native" not in name


def read_pmc(dirs):
    """{(kernel, grid): {counter: mean per dispatch, "_us": mean duration in the run that held GRBM_GUI_ACTIVE}}"""
    out = collections.defaultdict(dict)
    for d in dirs:
        acc, seen, dur = collections.defaultdict(float), collections.defaultdict(set), collections.defaultdict(dict)
        for f in glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True):
            with open(f, newline="") as fh:
                for r in csv.DictReader(fh):
                    n = r["Kernel_Name"]
                    if not wanted(n):
                        continue
                    key = (short(n), int(r["Grid_Size"]))
                    c = r["Counter_Name"]
                    acc[key, c] += float(r["Counter_Value"])
                    seen[key, c].add(r["Dispatch_Id"])
                    dur[key][r["Dispatch_Id"]] = (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3
        for (key, c), v in acc.items():
            out[key][c] = v / len(seen[key, c])
            if c == "GRBM_GUI_ACTIVE" and "_us" not in out[key]:
                out[key]["_us"] = statistics.fmean(dur[key].values())
    return out


def read_trace(d):
    per = collections.defaultdict(list)
    stats = []
    for f in glob.glob(os.path.join(d, "**", "*kernel_trace.csv"), recursive=True):
        with open(f, newline="") as fh:
            for r in csv.DictReader(fh):
                n = r["Kernel_Name"]
                if wanted(n):
                    per[short(n), int(r["Grid_Size_X"]) * int(r.get("Grid_Size_Y", 1) or 1) * int(r.get("Grid_Size_Z", 1) or 1)].append(
                        (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    for f in glob.glob(os.path.join(d, "**", "*kernel_stats.csv"), recursive=True):
        with open(f, newline="") as fh:
            for r in csv.DictReader(fh):
                if wanted(r["Name"]):
                    stats.append((short(r["Name"]), int(r["Calls"]), float(r["AverageNs"]) / 1e3, float(r["MinNs"]) / 1e3,
                                  float(r["MaxNs"]) / 1e3, float(r["Percentage"])))
    stats.sort(key=lambda x: -x[5])
    return per, stats


def commentary(path):
    try:
        text = open(path).read()
    except OSError:
        return ""
    at = text.find("\nReading the table")
    return text[at:] if at >= 0 else ""


def bench_lines(b):
    """What the profiled run itself reported, one line per config."""
    ex, roof = b.get("extras", {}), b["roofline"]
    L = [f"  config 2 headline ({b['config'].get('workload', '')}): {roof['launch_ms'] * 1e3:.1f} us per launch = {b['value']:.0f} TFLOP/s"
         f" = {roof['frac']:.3f} of 5 PFLOP/s"]

    def gemm(tag, label):
        if tag in ex:
            L.append(f"  {label}: {ex[tag]['ms'] * 1e3:.1f} us = {ex[tag]['tflops']:.0f} TFLOP/s ({ex[tag]['mfma_frac']:.3f})")

    def stream(tag, label, ms="ms"):
        if tag in ex:
            L.append(f"  {label}: {ex[tag][ms] * 1e3:.1f} us = {ex[tag]['GB/s']:.0f} GB/s ({ex[tag]['hbm_frac']:.3f} of 8 TB/s)")

    gemm("c2_gemm_e8m0_scales", "config 2 with e8m0 scales")
    gemm("deep_k_gemm_4096x7168x18432_fp32_scales", "deep K 4096 x 7168 x 18432, fp32 scales")
    gemm("deep_k_gemm_4096x7168x18432_e8m0_scales", "deep K 4096 x 7168 x 18432, e8m0 scales")
    for tag, v in ex.get("hipblaslt_fp8_tensorwise_scaled_mm", {}).items():
        if "ms" in v:
            L.append(f"  hipBLASLt, one scale per tensor, {tag}: {v['ms'] * 1e3:.1f} us = {v['tflops']:.0f} TFLOP/s ({v['mfma_frac']:.3f})")
    for tag in ("c3_skinny_gemm", "decode_gemm_64x18432x7168"):
        if tag in ex:
            L.append(f"  {tag}: {ex[tag]['ms'] * 1e3:.2f} us = {ex[tag]['weight_GB/s']:.0f} GB/s of weights")
    c4 = ex.get("c4_grouped_gemm", {})
    for proj in ("gate_up", "down", "gate_up_e8m0_scales", "down_e8m0_scales"):
        if proj in c4:
            L.append(f"  config 4 {proj}: {c4[proj]['ms']:.3f} ms = {c4[proj]['tflops']:.0f} TFLOP/s ({c4[proj]['mfma_frac']:.3f})")
    stream("c5_fp4_to_fp8_fused", "config 5 fused FP4 -> FP8, whole layer", "ms_total")
    stream("c1_quant_128x128", "config 1 quantise 4096 x 4096")
    stream("c1_dequant_128x128", "config 1 dequantise 4096 x 4096")
    bw = ex.get("grouped_linear_backward", {})
    for tag, v in bw.items():
        if isinstance(v, dict) and "ms" in v:
            L.append(f"  {tag}: {v['ms']:.3f} ms")
    return "\n".join(L)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--kernel-trace")
    ap.add_argument("--bench-json")
    ap.add_argument("--pmc", nargs="*", default=[])
    ap.add_argument("--out", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles"))
    args = ap.parse_args()
    os.makedirs(args.out, exist_ok=True)
    pmc = read_pmc(args.pmc)
    per, stats = read_trace(args.kernel_trace) if args.kernel_trace else ({}, [])

    # ---------------------------------------------------------------- counters
    keys = sorted(k for k in pmc if "GRBM_GUI_ACTIVE" in pmc[k] or "WRITE_SIZE" in pmc[k])
    T1 = ["%-46s %10s %6s %9s %9s %9s %8s %8s %8s %8s %8s %6s" % ("kernel", "grid", "calls", "trace us", "median", "pmc us", "MfmaUtil",
                                                                   "LdsBusy", "LdsConfl", "WaitAny", "WaitLds", "GHz")]
    for k in keys:
        c = pmc[k]
        g = c.get("GRBM_GUI_ACTIVE", 0) / 8                       # the counter is summed over the 8 XCDs
        if not g:
            continue
        d = per.get(k, [])
        wc = c.get("SQ_WAVE_CYCLES", 0) or float("nan")
        idx = c.get("SQ_LDS_IDX_ACTIVE", 0)
        T1.append("%-46s %10d %6d %9.1f %9.1f %9.1f %8.3f %8.3f %8.3f %8.3f %8.3f %6.2f" % (
            k[0][:46], k[1], len(d), statistics.fmean(d) if d else float("nan"), statistics.median(d) if d else float("nan"), c["_us"],
            c.get("SQ_VALU_MFMA_BUSY_CYCLES", 0) / (g * 1024), idx / (g * 256), (c.get("SQ_LDS_BANK_CONFLICT", 0) / idx) if idx else 0.0,
            c.get("SQ_WAIT_INST_ANY", 0) / wc, c.get("SQ_WAIT_INST_LDS", 0) / wc,
            g / (c["_us"] * 1e3) if c["_us"] >= 100 else float("nan")))
    T2 = ["%-46s %10s %10s %10s %12s %11s %11s %11s" % ("kernel", "grid", "read MB", "write MB", "FETCH_SIZE MB", "matrix ops", "LDS instr",
                                                        "VMEM reads")]
    traffic = []
    for k in keys:
        c = pmc[k]
        rd = 128 * c.get("TCC_EA0_RDREQ_128B_sum", 0) + 64 * c.get("TCC_EA0_RDREQ_64B_sum", 0) + 32 * c.get("TCC_EA0_RDREQ_32B_sum", 0)
        wr = c.get("WRITE_SIZE", 0) * 1024
        fs = c.get("FETCH_SIZE", 0) * 1024
        if not (rd or wr or fs):
            continue
        T2.append("%-46s %10d %10.1f %10.1f %12.1f %11.4g %11.4g %11.4g" % (k[0][:46], k[1], rd / 1e6, wr / 1e6, fs / 1e6,
                                                                            c.get("SQ_INSTS_VALU_MFMA_MOPS_F8", 0), c.get("SQ_INSTS_LDS", 0),
                                                                            c.get("SQ_INSTS_VMEM_RD", 0)))
        if "probe_" not in k[0]:
            traffic.append({"kernel": k[0], "grid_threads": k[1], "read_bytes": int(rd), "write_bytes": int(wr), "fetch_size_bytes": int(fs)})
    sets = "\n".join(f"  rocprofv3 --pmc {v} --output-format csv -d <out> -o run -- $B" for v in COUNTER_SETS.values())
    head = f"""Matrix-core, LDS and memory-side counters of the GEMM and streaming kernels and of hipBLASLt's fp8 GEMM, one MI355X
=================================================================================================================
Commands (from /tmp, TMPDIR=/tmp), one counter set per run, every run the same program on the same box:
  B="python3 /root/repo/bench.py --no-cpu --no-graph --steps 4 --warmup 1"
{sets}
  python3 profile_summary.py --kernel-trace <kt> --bench-json <kt>.json --pmc <out> <out> ...      (wrote this file)
Values are averages per dispatch over the dispatches of one kernel at one grid size (grid = workgroups x threads).
  trace us / median = mean and median launch duration in the kernel-trace run (graph replays; the mean takes in warm-up
             and clock-settling replays, the median does not); pmc us = mean duration in the counter run that held
             GRBM_GUI_ACTIVE (eager launches under counter collection: slower, and the run the ratios below belong to).
  GHz      = GRBM_GUI_ACTIVE / 8 / pmc us: the clock the chip held during the kernel (the counter is summed over the
             8 XCDs and ticks at the shader clock; left out under 100 us, where the counter's window is
             visibly longer than the kernel).
  MfmaUtil = SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE / 8 x 1024): busy matrix-pipe cycles over elapsed cycles of the
             1024 SIMDs.  The fp8 16x16x128 instruction is busy 32 cycles, so MfmaUtil x GHz / 2.4 is the fraction of the
             5 PFLOP/s peak; padded tiles of the grouped kernels count as busy.
  LdsBusy  = SQ_LDS_IDX_ACTIVE / (elapsed cycles x 256 CUs); LdsConfl = SQ_LDS_BANK_CONFLICT / SQ_LDS_IDX_ACTIVE.
  WaitAny / WaitLds = SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES, SQ_WAIT_INST_LDS / SQ_WAVE_CYCLES (share of wave time in s_waitcnt).
  read MB  = 128 n128 + 64 n64 + 32 n32 from the request-size counters; write MB = WRITE_SIZE KiB x 1024.  FETCH_SIZE
             prices the 128-byte requests of LDS-direct and non-temporal loads at 64 bytes, so it is shown but not used;
             the stream_probe rows (byte counts chosen by the bench) are the scale check of both.
  matrix ops = SQ_INSTS_VALU_MFMA_MOPS_F8 (512 per fp8 16x16x128 instruction); LDS instr, VMEM reads = instructions issued.

"""
    text = head + "\n".join(T1) + "\n\n" + "\n".join(T2) + "\n"
    path = os.path.join(args.out, "gemm_kernels_mfma_lds_hbm_counters.txt")
    keep = commentary(path)
    if args.pmc:
        open(path, "w").write(text + keep)
        json.dump({"source": "profile_summary.py over rocprofv3 --pmc runs of bench.py (request-size read counters, WRITE_SIZE)",
                   "kernels": traffic}, open(os.path.join(args.out, "traffic.json"), "w"), indent=1)

    # ---------------------------------------------------------------- kernel trace
    if args.kernel_trace:
        b = json.load(open(args.bench_json)) if args.bench_json else None
        kt = ["%-52s %7s %10s %10s %10s %6s" % ("kernel", "calls", "avg_us", "min_us", "max_us", "%")]
        kt += ["%-52s %7d %10.2f %10.2f %10.2f %6.2f" % ((r[0][:52],) + r[1:]) for r in stats]
        by = ["%-46s %10s %6s %10s %10s %10s %10s" % ("kernel", "grid", "calls", "avg_us", "median_us", "min_us", "max_us")]
        for k in sorted(per):
            d = per[k]
            by.append("%-46s %10d %6d %10.2f %10.2f %10.2f %10.2f" % (k[0][:46], k[1], len(d), statistics.fmean(d), statistics.median(d), min(d), max(d)))
        head = """Kernel trace of the whole benchmark (all configs), one MI355X
=============================================================
Command (from /tmp, TMPDIR=/tmp):
  rocprofv3 --kernel-trace --stats --output-format csv -d <out> -o run -- python3 /root/repo/bench.py --no-cpu > <out>.json
  python3 profile_summary.py --kernel-trace <out> --bench-json <out>.json      (wrote this file)
Durations are end - start of each dispatch (microseconds); launches are replayed from HIP graphs.  The averages take in
every dispatch of the run: the bench's untimed warm-up replays and the replays that settle the clock before each timed
region as well as the timed ones, so an average sits a few per cent above the figure the bench prints for the same
kernel; the median and the minimum are the figures to hold against it.  torch's own kernels (at::native::*, which build
the synthetic inputs) are left out; % is of all GPU time in the run.  The first table is rocprofv3's per-kernel summary
(a kernel used by several configs is one row); the second splits dispatches by grid size (workgroups x threads), which
separates the configs.
"""
        if b:
            head += "\nWhat bench.py reported in this same profiled run (tracing costs a few per cent):\n" + bench_lines(b) + "\n"
        path = os.path.join(args.out, "bench_all_configs_kernel_trace.txt")
        keep = commentary(path)
        open(path, "w").write(head + "\n" + "\n".join(kt) + "\n\nBy grid size:\n" + "\n".join(by) + "\n" + keep)
    return 0


if __name__ == "__main__":
    sys.exit(main())
