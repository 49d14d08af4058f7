#!/usr/bin/env python3
"""Turn rocprofv3 CSV output of `bench.py` runs into the short text summaries and the traffic table under profiles/.

Inputs (each a directory that one rocprofv3 run wrote with `--output-format csv -d <dir> -o run`):
  --kernel-trace DIR   a `--kernel-trace --stats` run of `python3 bench.py --no-cpu` (graph replays, as the bench times them)
  --bench-json FILE    the JSON line that same run printed
  --floor-json FILE    the JSON line of an untraced `python3 bench.py --no-cpu` run: its floor probes beside the kernels
                       they bound -> floor_probes_matrix_pipe_bare_stream_empty_launch.txt
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
    for tag in ("c3_skinny_gemm", "decode_gemm_64x18432x7168", "decode_gemm_64x7168x18432", "decode_gemm_1x7168x18432",
                "decode_gemm_1x129280x7168", "decode_gemm_16x129280x7168"):
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


def floor_summary(b):
    """The floor probes of one untraced bench run beside the kernels they bound."""
    ex = b["extras"]
    L = ["Floor probes: what the box gives with nothing of the kernels' own in the way, beside the kernels, one MI355X",
         "=" * 112,
         "Command: python3 bench.py --no-cpu > <out>.json ; python3 profile_summary.py --floor-json <out>.json      (one untraced run, one",
         "box; times are per launch, from HIP graph replays timed with events on the launching stream; the probes are the entry",
         "points lp_probe_mfma, lp_probe_stream and lp_probe_copy of the probe library)", ""]
    mp = ex.get("matrix_pipe_probe_registers_only")
    if mp:
        L.append("1. Matrix pipe, registers only (256 workgroups, the fp8 16x16x128 instruction into eight result buffers, no LDS and no")
        L.append("   memory traffic in the loop; TFLOP/s and fraction of 5 PFLOP/s)")
        L.append("   %-58s %12s %12s %12s" % ("into fresh registers, k fp32 FMAs behind each", "k = 0", "k = 4", "k = 8"))
        for tag, label in (("zero_operands", "zeros"), ("random_e4m3_operands", "random e4m3 codes")):
            L.append("   %-58s %12s %12s %12s" % (label, *["%.0f (%.2f)" % (mp[f"{tag}_{k}_fmas_per_instruction"]["tflops"],
                                                                        mp[f"{tag}_{k}_fmas_per_instruction"]["mfma_frac"]) for k in (0, 4, 8)]))
        for key, v in mp.items():
            if "in_place" in key:
                L.append("   %-58s %12s" % (key.replace("random_e4m3_operands_", "accumulating in place, ").replace("_", " "),
                                            "%.0f (%.2f)" % (v["tflops"], v["mfma_frac"])))
        d2 = ex.get("deep_k_gemm_4096x7168x18432_e8m0_scales", {})
        L.append("   In the same run: config 2 with fp32 scales (four FMAs per instruction) %.0f TFLOP/s = %.3f of peak; with e8m0 scales %.0f;"
                 % (b["value"], b["roofline"]["frac"], ex.get("c2_gemm_e8m0_scales", {}).get("tflops", float("nan"))))
        L.append("   deep K 4096 x 7168 x 18432: %.0f / %.0f." % (ex.get("deep_k_gemm_4096x7168x18432_fp32_scales", {}).get("tflops", float("nan")),
                                                                   d2.get("tflops", float("nan"))))
        L.append("")
    for n, tag, ptag, what in (("2", "c3_skinny_gemm", "c3_floor_probe", "config 3: M = 64, N = 4096, K = 7168"),
                               ("3", "decode_gemm_64x18432x7168", "decode_64x18432x7168_floor_probe", "M = 64, N = 18432, K = 7168"),
                               ("3b", "decode_gemm_64x7168x18432", "decode_64x7168x18432_floor_probe", "M = 64, N = 7168, K = 18432: three rounds of K"),
                               ("3c", "decode_gemm_1x7168x18432", "decode_1x7168x18432_floor_probe", "M = 1, N = 7168, K = 18432: three rounds of K"),
                               ("3d", "decode_gemm_1x129280x7168", "decode_1x129280x7168_floor_probe", "M = 1, N = 129280, K = 7168: the vocabulary projection"),
                               ("3e", "decode_gemm_16x129280x7168", "decode_16x129280x7168_floor_probe", "M = 16, N = 129280, K = 7168")):
        if tag in ex and ptag in ex:
            pr = ex[ptag]
            L.append(f"{n}. Decode GEMM ({what}) against an empty launch and a bare read of its weight bytes")
            L.append("   empty launch %37.2f us" % pr["empty_launch_us"])
            for k, v in pr.items():
                if k.startswith("read_"):
                    L.append("   bare %-44s %6.2f us" % (k[:-3].replace("_", " "), v))
            L.append("   the kernel %39.2f us = %.2f x the best bare read (%.0f GB/s)" % (ex[tag]["ms"] * 1e3, pr["gemm_over_bare_read"], pr["bare_read_best_GB/s"]))
            L.append("")
    if "c1_floor_probe" in ex:
        c1 = ex["c1_floor_probe"]
        L.append("4. 128 x 128 tile quantiser / dequantiser (config 1: 4096 x 4096, 32 MiB + 16 MiB) against a bare stream of the same bytes")
        for w in (512, 1024, 2048, 4096):
            L.append("   bare stream, %4d workgroups: read 32 MiB + write 16 MiB %6.2f us, read 16 MiB + write 32 MiB %6.2f us"
                     % (w, c1[f"read32MiB_write16MiB_{w}_workgroups_us"], c1[f"read16MiB_write32MiB_{w}_workgroups_us"]))
        L.append("   quant_tile128    %6.2f us = %.2f x the best bare stream (%.3f of 8 TB/s; the bare stream %.3f)"
                 % (ex["c1_quant_128x128"]["ms"] * 1e3, c1["quant_over_bare_stream"], ex["c1_quant_128x128"]["hbm_frac"], c1["bare_stream_hbm_frac"]["read32_write16"]))
        L.append("   dequant_fp8_fast %6.2f us = %.2f x the best bare stream (%.3f of 8 TB/s; the bare stream %.3f)"
                 % (ex["c1_dequant_128x128"]["ms"] * 1e3, c1["dequant_over_bare_stream"], ex["c1_dequant_128x128"]["hbm_frac"], c1["bare_stream_hbm_frac"]["read16_write32"]))
        L.append("")
    if "c5_floor_probe" in ex:
        c5 = ex["c5_floor_probe"]
        L.append("5. FP4 -> FP8 fused over a whole MoE layer (config 5) against a bare stream of the same mix (0.5 byte read, 1 byte")
        L.append("   written per element; the kernel also reads 1/32 byte of scales per element)")
        for k, v in c5.items():
            if k.endswith("_workgroups_ms"):
                L.append("   bare stream, %6s workgroups %8.3f ms" % (k.split("_")[-3], v))
        L.append("   fp4_amax (three launches)     %8.3f ms = %.3f x the best bare stream (%.3f of 8 TB/s; the bare stream %.3f)"
                 % (ex["c5_fp4_to_fp8_fused"]["ms_total"], c5["fused_over_bare_stream"], ex["c5_fp4_to_fp8_fused"]["hbm_frac"], c5["bare_stream_hbm_frac"]))
        L.append("")
    if "l2_to_cu_copy_probe" in ex:
        L.append("6. Operand copies out of the L2 alone (every wave issues eight 1 KB requests per step, 8 rows x 128 bytes with rows 7168")
        L.append("   bytes apart, one step in flight behind a wait and a workgroup barrier; 2 MB per region, L2-resident after the first pass)")
        for k, v in ex["l2_to_cu_copy_probe"].items():
            L.append("   %-46s %6.1f B/ns per CU = %5.1f TB/s over the chip" % (k.replace("_", " "), v["bytes_per_ns_per_cu"], v["TB/s"]))
        L.append("   What the GEMM loops ask of that path: the 256 x 288 tile 68 KB per %.2f us step = %.0f B/ns per CU (config 2)."
                 % (b["roofline"]["launch_ms"] * 1e3 / 112, 68 * 1024 / (b["roofline"]["launch_ms"] * 1e3 / 112) / 1e3))
    return "\n".join(L) + "\n"


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--kernel-trace")
    ap.add_argument("--bench-json")
    ap.add_argument("--floor-json")
    ap.add_argument("--pmc", nargs="*", default=[])
    ap.add_argument("--out", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles"))
    args = ap.parse_args()
    os.makedirs(args.out, exist_ok=True)
    if args.floor_json:
        open(os.path.join(args.out, "floor_probes_matrix_pipe_bare_stream_empty_launch.txt"), "w").write(floor_summary(json.load(open(args.floor_json))))
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
