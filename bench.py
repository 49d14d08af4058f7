#!/usr/bin/env python3
"""Benchmark of the MI355X low-precision weight / GEMM path (one GPU).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extras]

Headline (the JSON line's metric/value): the dense block-scaled FP8 GEMM of
benchmark config 2 -- A [2048,7168] (1x128 e4m3fn + fp32 scales) times
B [18432,7168] (128x128 e4m3fn + fp32 scales) -> bf16 [2048,18432] -- in TFLOP/s
with operands already quantised and resident in HBM.  One "step" is one GEMM.

The same line carries, under "extras", the bandwidth kernels (config 1 quantise
and dequantise, config 5 FP4 -> FP8 conversion), the skinny GEMM (config 3) and
the grouped MoE GEMM (config 4), each with its own roofline fraction, and under
"cpu_baseline" the eager-PyTorch CPU oracle timed on a bounded sample.

Kernel durations are measured with HIP events on the stream the kernels are
launched on (torch's current stream); launches are replayed from a HIP graph
where possible so that host launch cost does not leak into device time, and
bandwidth kernels rotate over buffer sets larger than the 256 MB Infinity Cache.
After the W warm-up launches every timed region is preceded by untimed replays
of its graph until the GPU has been busy for 40 ms, then exactly K launches are
timed in one region: the first tens of milliseconds after an idle stretch run
up to 15 % slower, which a short timed region would report as the kernel's time.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "g-core-gh_amd"))

SETTLE_MS = 40.0             # untimed graph replays before every timed region (see time_launches)
HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
FP8_PEAK_TFLOPS = 5000.0     # MI355X dense FP8 MFMA
# Bytes per launch between a kernel's L2s and the memory side (Infinity Cache / HBM) cannot be read from inside this
# process: `roofline.traffic` comes from profiles/traffic.json, which profile_summary.py writes from rocprofv3 --pmc
# runs of this script (reads from the request-size counters, 32 / 64 / 128-byte TCC->EA reads, exact -- the derived
# FETCH_SIZE prices the 128-byte requests of LDS-direct and non-temporal loads at 64 -- plus WRITE_SIZE).  A kernel the
# file does not list reports null.
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")


def measured_traffic(kernel, grid_threads):
    """read + write bytes per launch of `kernel` at that grid size from the committed counter summary, or None."""
    try:
        with open(TRAFFIC_JSON) as f:
            table = json.load(f)["kernels"]
    except (OSError, ValueError, KeyError):
        return None
    for row in table:
        if row["kernel"].startswith(kernel) and row["grid_threads"] == grid_threads:
            return row["read_bytes"] + row["write_bytes"]
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="only the headline GEMM")
    ap.add_argument("--only", default="", help="comma list of extra sections to run: deep,vendor,copy,c2q,c1,c3,c5,c4 (default: all)")
    ap.add_argument("--only-gemm", action="store_true", help="extras: only the skinny and the grouped GEMM (counter runs)")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches (for counter-collection runs)")
    ap.add_argument("--cpu-seconds", type=float, default=20.0, help="rough budget of the CPU baseline sample")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on ONE GPU (nothing on it communicates); use --gpus 1. "
                 "Across GPUs it would split by weight columns, experts or checkpoint shards without collectives.")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import gcore_lowp  # noqa: F401  (fails loudly if the HIP library is missing)
    from gcore_lowp import _abi as A
    from gcore_lowp import _probe_abi as PA            # bare-stream / matrix-pipe / copy-path probes (liblowp_probe.so)
    from tests._inputs import zipf_m_splits_with_idle_expert as zipf_m_splits   # the grouped problem's rows per expert: one recipe for tests and bench

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    L = A.lib()
    LP = PA.lib()
    E4M3, E8M0 = torch.float8_e4m3fn, torch.float8_e8m0fnu

    def stream():
        return torch.cuda.current_stream().cuda_stream

    def time_launches(fns, steps, warmup, graph=True):
        """Average device time (ms) of one call of fns[i % len(fns)], over `steps` calls."""
        for i in range(warmup):
            fns[i % len(fns)]()
        torch.cuda.synchronize()
        g = None
        if graph and not args.no_graph:
            try:
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    g = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(g, stream=side):
                        for i in range(steps):
                            fns[i % len(fns)]()
                torch.cuda.current_stream().wait_stream(side)
                torch.cuda.synchronize()
                # untimed replays until the GPU has worked for SETTLE_MS without a pause: after an idle stretch the
                # first ~30 ms of back-to-back GEMM launches run measurably slower (clocks still rising; six replays
                # of 5 ms went 288, 268, 257, 252, 249, 244 us per launch), and a timed region that short would
                # measure the ramp instead of the kernel
                spent, n_rep = 0.0, 0
                while n_rep < 1 or (spent < SETTLE_MS and n_rep < 64):
                    s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    s0.record()
                    g.replay()
                    s1.record()
                    torch.cuda.synchronize()
                    spent += s0.elapsed_time(s1)
                    n_rep += 1
            except Exception as e:             # capture unsupported: time eager launches
                print(f"[bench] graph capture failed ({e}); timing eager launches", file=sys.stderr)
                g = None
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        wall0 = time.perf_counter()
        t0.record()
        if g is not None:
            g.replay()
        else:
            for i in range(steps):
                fns[i % len(fns)]()
        t1.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - wall0) * 1e3
        return t0.elapsed_time(t1) / steps, wall / steps

    def chk(rc):
        A.check(rc)

    gen = torch.Generator(device=dev).manual_seed(1234)

    def randn(*shape, std=1.0):
        return (torch.randn(*shape, generator=gen, device=dev, dtype=torch.float32) * std).to(torch.bfloat16)

    def quant_into(x, bm, bn, q, s):
        chk(L.lp_quant_fp8_block(x.data_ptr(), A.BF16, x.shape[0], x.shape[1], bm, bn, A.SCALE_DIV, 1e-12, 0,
                                 q.data_ptr(), s.data_ptr(), A.F32, None, stream()))

    extras = {}
    only = set(filter(None, ("c3,c4" if args.only_gemm else args.only).split(",")))

    def want(section):
        return not args.no_extras and (not only or section in only)

    # ------------------------------------------------------------------ config 2: dense GEMM (headline)
    M, N, K = 2048, 18432, 7168
    a_bf = randn(M, K)
    aq = torch.empty(M, K, dtype=torch.uint8, device=dev)
    a_s = torch.empty(M, K // 128, dtype=torch.float32, device=dev)
    quant_into(a_bf, 1, 128, aq, a_s)
    n_sets = 2
    bq, b_s = [], []
    for _ in range(n_sets):
        w = randn(N, K, std=0.02)
        q = torch.empty(N, K, dtype=torch.uint8, device=dev)
        s = torch.empty(N // 128, K // 128, dtype=torch.float32, device=dev)
        quant_into(w, 128, 128, q, s)
        bq.append(q)
        b_s.append(s)
        del w
    c = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    torch.cuda.synchronize()

    def gemm_call(i):
        return lambda: chk(L.lp_gemm_fp8_block(aq.data_ptr(), a_s.data_ptr(), bq[i].data_ptr(), b_s[i].data_ptr(), A.F32,
                                                M, N, K, c.data_ptr(), A.BF16, None, 0, stream()))

    ms, wall_ms = time_launches([gemm_call(i) for i in range(n_sets)], args.steps, args.warmup)
    flops = 2.0 * M * N * K
    tflops = flops / (ms * 1e-3) / 1e12
    headline = {"ms": ms, "tflops": tflops}
    # The call above is one launch of gemm_asm_wide: 256 x 288 tiles, 8 x 64 = 512 of them, exactly two rounds on the 256
    # CUs.  Beside it, the 256 x 256-tile kernel on the 16384 weight rows that make two full rounds of its tiles:
    N_BIG = 16384
    c_big = torch.empty(M, N_BIG, dtype=torch.bfloat16, device=dev)

    def big_call(i):
        return lambda: chk(L.lp_gemm_fp8_block(aq.data_ptr(), a_s.data_ptr(), bq[i].data_ptr(), b_s[i].data_ptr(), A.F32,
                                                M, N_BIG, K, c_big.data_ptr(), A.BF16, None, 0, stream()))

    big_ms, _ = time_launches([big_call(i) for i in range(n_sets)], args.steps, args.warmup)
    big_flops = 2.0 * M * N_BIG * K
    big_tflops = big_flops / (big_ms * 1e-3) / 1e12
    del c_big
    # quantisation of the operands, timed separately (not part of `value`)
    qa_ms, _ = time_launches([lambda: quant_into(a_bf, 1, 128, aq, a_s)], 20, 3)
    extras["c2_act_quant_1x128"] = {"ms": qa_ms, "GB/s": (M * K * 3 + M * K // 32) / qa_ms / 1e6,
                                    "hbm_frac": (M * K * 3 + M * K // 32) / qa_ms / 1e6 / HBM_PEAK_GBS}
    # the same problem with power-of-two (e8m0) scales on both operands, the reference's default scale_dtype
    # (gfused/mygemm_fp8.py:55): the matrix instructions apply the scales themselves
    a_s8 = torch.empty(M, K // 128, dtype=torch.uint8, device=dev)
    chk(L.lp_quant_fp8_block(a_bf.data_ptr(), A.BF16, M, K, 1, 128, A.SCALE_POW2, 0.0, 0, aq.data_ptr(), a_s8.data_ptr(),
                             A.E8M0, None, stream()))
    b_s8 = [torch.randint(118, 124, (N // 128, K // 128), dtype=torch.uint8, device=dev) for _ in range(n_sets)]

    def gemm8_call(i):
        return lambda: chk(L.lp_gemm_fp8_block(aq.data_ptr(), a_s8.data_ptr(), bq[i].data_ptr(), b_s8[i].data_ptr(), A.E8M0,
                                                M, N, K, c.data_ptr(), A.BF16, None, 0, stream()))

    ms8, _ = time_launches([gemm8_call(i) for i in range(n_sets)], args.steps, args.warmup)
    extras["c2_gemm_e8m0_scales"] = {"ms": ms8, "tflops": flops / (ms8 * 1e-3) / 1e12,
                                     "mfma_frac": flops / (ms8 * 1e-3) / 1e12 / FP8_PEAK_TFLOPS}
    del bq, b_s, c, a_bf, a_s8, b_s8
    torch.cuda.empty_cache()

    if want("deep"):
        # -------------------------------------------------------------- a deep-K problem (K = 18432) on 256 x 256 tiles:
        # what the loop reaches when the K steps dominate; and the unscaled NT GEMM at the reference's benchmark shape
        # (tests/test_gfused/test_my_gemm_fp8.py:137: 4096^3, fp8 in, fp8 out, 0.575 ms on its hardware)
        Md, Nd, Kd = 4096, 7168, 18432
        ad = randn(Md, Kd)
        adq = torch.empty(Md, Kd, dtype=torch.uint8, device=dev)
        ads = torch.empty(Md, Kd // 128, dtype=torch.float32, device=dev)
        quant_into(ad, 1, 128, adq, ads)
        ads8 = torch.empty(Md, Kd // 128, dtype=torch.uint8, device=dev)
        chk(L.lp_quant_fp8_block(ad.data_ptr(), A.BF16, Md, Kd, 1, 128, A.SCALE_POW2, 0.0, 0, adq.data_ptr(), ads8.data_ptr(),
                                 A.E8M0, None, stream()))
        del ad
        wdq, wds, wds8 = [], [], []
        for _ in range(2):
            w = randn(Nd, Kd, std=0.02)
            q = torch.empty(Nd, Kd, dtype=torch.uint8, device=dev)
            sc = torch.empty(Nd // 128, Kd // 128, dtype=torch.float32, device=dev)
            quant_into(w, 128, 128, q, sc)
            wdq.append(q)
            wds.append(sc)
            wds8.append(torch.randint(118, 124, (Nd // 128, Kd // 128), dtype=torch.uint8, device=dev))
            del w
        cd = torch.empty(Md, Nd, dtype=torch.bfloat16, device=dev)
        fl_d = 2.0 * Md * Nd * Kd
        for label, sa, sbs, code in (("fp32_scales", ads, wds, A.F32), ("e8m0_scales", ads8, wds8, A.E8M0)):
            fns = [(lambda i=i: chk(L.lp_gemm_fp8_block(adq.data_ptr(), sa.data_ptr(), wdq[i].data_ptr(), sbs[i].data_ptr(), code,
                                                        Md, Nd, Kd, cd.data_ptr(), A.BF16, None, 0, stream()))) for i in range(2)]
            ms_d, _ = time_launches(fns, 10, 3)
            extras[f"deep_k_gemm_4096x7168x18432_{label}"] = {"ms": ms_d, "tflops": fl_d / ms_d / 1e9,
                                                              "mfma_frac": fl_d / ms_d / 1e9 / FP8_PEAK_TFLOPS}
        del adq, ads, ads8, wdq, wds, wds8, cd
        torch.cuda.empty_cache()
        n4 = 4096
        a_nt = torch.randint(-3, 4, (n4, n4), generator=gen, device=dev).float().to(E4M3)
        b_nt = [torch.randint(-3, 4, (n4, n4), generator=gen, device=dev).float().to(E4M3) for _ in range(4)]
        c_nt = torch.empty(n4, n4, dtype=torch.uint8, device=dev)
        fns = [(lambda i=i: chk(L.lp_gemm_nt(a_nt.data_ptr(), b_nt[i].data_ptr(), A.E4M3, n4, n4, n4, c_nt.data_ptr(), A.E4M3, stream())))
               for i in range(4)]
        ms_nt, _ = time_launches(fns, 12, 4)
        extras["gemm_impl_fp8_4096x4096x4096"] = {"ms": ms_nt, "tflops": 2.0 * n4 ** 3 / ms_nt / 1e9,
                                                  "mfma_frac": 2.0 * n4 ** 3 / ms_nt / 1e9 / FP8_PEAK_TFLOPS,
                                                  "reference_ms_on_its_hardware": 0.575}
        del a_nt, b_nt, c_nt
        # the reference's other published lines (gfused/test_my_gemm_fp8.py:267-269): quantise both operands (1 x 128 and
        # 128 x 128, fp32 scales) and multiply them, three launches on bf16 inputs that are resident, 4096^3 and 128 x 4096 x 4096
        # and 8096 x 129280 x 4096 (:280, a vocabulary projection: 2.1 GB of bf16 out, 38.959 ms in the reference's table)
        for (m_q, n_q, k_q), ref_ms, n_in, steps_q in (((4096, n4, n4), 0.675, 2, 12), ((128, n4, n4), 0.134, 2, 12), ((8096, 129280, 4096), 38.959, 1, 4)):
            xb = [randn(m_q, k_q) for _ in range(n_in)]
            wb = [randn(n_q, k_q, std=0.02) for _ in range(n_in)]
            xq_, xs_ = torch.empty(m_q, k_q, dtype=torch.uint8, device=dev), torch.empty(m_q, k_q // 128, dtype=torch.float32, device=dev)
            wq_, ws_ = torch.empty(n_q, k_q, dtype=torch.uint8, device=dev), torch.empty(n_q // 128, k_q // 128, dtype=torch.float32, device=dev)
            cq_ = torch.empty(m_q, n_q, dtype=torch.bfloat16, device=dev)

            def quant_and_multiply(i):
                quant_into(xb[i], 1, 128, xq_, xs_)
                quant_into(wb[i], 128, 128, wq_, ws_)
                chk(L.lp_gemm_fp8_block(xq_.data_ptr(), xs_.data_ptr(), wq_.data_ptr(), ws_.data_ptr(), A.F32, m_q, n_q, k_q, cq_.data_ptr(),
                                        A.BF16, None, 0, stream()))
            ms_q, _ = time_launches([(lambda i=i: quant_and_multiply(i)) for i in range(n_in)], steps_q, 2)
            extras[f"quant_x_w_then_gemm_{m_q}x{n_q}x{k_q}"] = {"ms": ms_q, "launches": 3, "gemm_flops_over_the_three_launches_TFLOP/s": 2.0 * m_q * n_q * k_q / ms_q / 1e9,
                                                                "reference_ms_on_its_hardware": ref_ms}
            del xb, wb, xq_, xs_, wq_, ws_, cq_
        torch.cuda.empty_cache()
        # the GEMM alone on pre-quantised operands at the reference's three shapes (test_my_gemm_fp8.py:411-424: its tile
        # compiler / TransformerEngine; tests/test_libs/test_deepgemm.py:230-249: DeepGEMM), workspace as the Python wrapper passes it
        ref_only = {(4096, n4, n4): {"tile_compiler": 0.625, "transformer_engine": 0.571, "deepgemm": 0.536},
                    (128, n4, n4): {"tile_compiler": 0.044, "transformer_engine": 0.217, "deepgemm": 0.023},
                    (8096, 129280, 4096): {"tile_compiler": 38.334, "transformer_engine": 30.667, "deepgemm": 31.097}}
        for (m_q, n_q, k_q), refs in ref_only.items():
            n_sets_q = 1 if n_q > 100000 else 4
            xb = randn(m_q, k_q)
            xq_, xs_ = torch.empty(m_q, k_q, dtype=torch.uint8, device=dev), torch.empty(m_q, k_q // 128, dtype=torch.float32, device=dev)
            quant_into(xb, 1, 128, xq_, xs_)
            wqs_, wss_ = [], []
            for _ in range(n_sets_q):
                wb = randn(n_q, k_q, std=0.02)
                wq_, ws_ = torch.empty(n_q, k_q, dtype=torch.uint8, device=dev), torch.empty(n_q // 128, k_q // 128, dtype=torch.float32, device=dev)
                quant_into(wb, 128, 128, wq_, ws_)
                wqs_.append(wq_)
                wss_.append(ws_)
                del wb
            cq_ = torch.empty(m_q, n_q, dtype=torch.bfloat16, device=dev)
            nws_q = L.lp_gemm_workspace_bytes(m_q, n_q, k_q)
            wsp_q = torch.empty(max(nws_q, 16), dtype=torch.uint8, device=dev)
            fns = [(lambda i=i: chk(L.lp_gemm_fp8_block(xq_.data_ptr(), xs_.data_ptr(), wqs_[i].data_ptr(), wss_[i].data_ptr(), A.F32, m_q, n_q, k_q,
                                                        cq_.data_ptr(), A.BF16, wsp_q.data_ptr(), nws_q, stream()))) for i in range(n_sets_q)]
            ms_o, _ = time_launches(fns, 4 if n_q > 100000 else 16, 4)
            extras[f"gemm_only_{m_q}x{n_q}x{k_q}_fp32_scales"] = {"ms": ms_o, "tflops": 2.0 * m_q * n_q * k_q / ms_o / 1e9,
                                                                  "mfma_frac": 2.0 * m_q * n_q * k_q / ms_o / 1e9 / FP8_PEAK_TFLOPS,
                                                                  "weight_GB/s": n_q * k_q / ms_o / 1e6,
                                                                  "reference_ms_on_its_hardware": refs}
            del xb, xq_, xs_, wqs_, wss_, cq_, wsp_q
        torch.cuda.empty_cache()
        # the same product on bf16 operands (the reference's benchmark quotes fp8 against bf16: 0.575 against 1.087 ms)
        a_bf = torch.randint(-3, 4, (n4, n4), generator=gen, device=dev).to(torch.bfloat16)
        b_bf = [torch.randint(-3, 4, (n4, n4), generator=gen, device=dev).to(torch.bfloat16) for _ in range(4)]
        c_bf = torch.empty(n4, n4, dtype=torch.bfloat16, device=dev)
        fns = [(lambda i=i: chk(L.lp_gemm_nt(a_bf.data_ptr(), b_bf[i].data_ptr(), A.BF16, n4, n4, n4, c_bf.data_ptr(), A.BF16, stream())))
               for i in range(4)]
        ms_bf, _ = time_launches(fns, 12, 4)
        extras["gemm_impl_bf16_4096x4096x4096"] = {"ms": ms_bf, "tflops": 2.0 * n4 ** 3 / ms_bf / 1e9,
                                                   "mfma_frac_of_bf16_peak": 2.0 * n4 ** 3 / ms_bf / 1e9 / 2500.0,
                                                   "fp8_speed_up": ms_bf / ms_nt, "reference_ms_on_its_hardware": 1.087,
                                                   "reference_fp8_speed_up": 1.89}
        del a_bf, b_bf, c_bf
        torch.cuda.empty_cache()
        # what the matrix cores hold with the loop's arithmetic and nothing else: the fp8 16x16x128 instruction on registers
        # only, two waves per SIMD, with 0 / 4 / 8 fp32 FMAs after each (the fp32-scaled loops fold with four), on zeros and
        # on random e4m3 operands -- the ceiling the GEMM figures above are to be read against (no LDS, no memory traffic)
        rnd = (torch.randint(0, 256, (4096,), generator=gen, device=dev, dtype=torch.int32).to(torch.uint8) & 0x77)
        iters, wgs = 2000, 256
        fl_p = 2.0 * 16 * 16 * 128 * 8 * iters * 8 * wgs
        probe = {}
        for tag, ptr in (("zero_operands", None), ("random_e4m3_operands", rnd.data_ptr())):
            for k in (0, 4, 8):
                ms_p, _ = time_launches([lambda k=k, ptr=ptr: PA.check(LP.lp_probe_mfma(k, iters, ptr, wgs, stream()))], 6, 2)
                probe[f"{tag}_{k}_fmas_per_instruction"] = {"ms": ms_p, "tflops": fl_p / ms_p / 1e9, "mfma_frac": fl_p / ms_p / 1e9 / FP8_PEAK_TFLOPS}
        # accumulating in place, as the e8m0 loops do: the hardware-scaled form and the plain one, with two waves and with one
        # wave per SIMD (flops follow the wave count)
        for k, waves, tag in ((-1, 8, "hardware_scaled_in_place_2_waves_per_simd"), (-2, 8, "unscaled_in_place_2_waves_per_simd"),
                              (-3, 4, "hardware_scaled_in_place_1_wave_per_simd"), (-4, 4, "unscaled_in_place_1_wave_per_simd")):
            ms_p, _ = time_launches([lambda k=k: PA.check(LP.lp_probe_mfma(k, iters, rnd.data_ptr(), wgs, stream()))], 6, 2)
            fl = fl_p * waves / 8
            probe[f"random_e4m3_operands_{tag}"] = {"ms": ms_p, "tflops": fl / ms_p / 1e9, "mfma_frac": fl / ms_p / 1e9 / FP8_PEAK_TFLOPS}
        extras["matrix_pipe_probe_registers_only"] = probe
        # what a CU's copy path out of the L2 delivers in the loops' request shape (1 KB per wave and request, rows 7168 bytes
        # apart, one step in flight behind a wait and a barrier; 2 MB per region, L2-resident): into LDS with one 8-wave
        # workgroup or two 4-wave workgroups per CU, and into registers.  A 128 x 128 tile needs 32 KB per 16 matrix
        # instructions of a SIMD (512 cycles), a 256 x 256 tile 64 KB per 64 (2048 cycles).
        cus = torch.cuda.get_device_properties(0).multi_processor_count
        rows_src = torch.zeros(4 * 512 * 7168, dtype=torch.uint8, device=dev)
        sink = torch.zeros(2048, dtype=torch.uint8, device=dev)
        cp = {}
        steps_c = 2048
        for tag, to_lds, waves, per_cu in (("to_lds_8_waves_1_wg_per_cu", 1, 8, 1), ("to_lds_4_waves_2_wg_per_cu", 1, 4, 2),
                                           ("to_registers_8_waves_1_wg_per_cu", 0, 8, 1)):
            wg = cus * per_cu
            ms_c, _ = time_launches([lambda to_lds=to_lds, waves=waves, wg=wg: PA.check(LP.lp_probe_copy(
                to_lds, waves, steps_c, rows_src.data_ptr(), rows_src.numel(), 7168, sink.data_ptr(), wg, stream()))], 6, 2)
            by = float(wg) * waves * steps_c * 8192
            cp[tag] = {"ms": ms_c, "TB/s": by / ms_c / 1e9, "bytes_per_ns_per_cu": by / ms_c / 1e6 / cus}
        extras["l2_to_cu_copy_probe"] = cp
        del rows_src, sink

    if want("vendor"):
        # -------------------------------------------------------------- the vendor library on the same silicon: hipBLASLt's
        # fp8 GEMM through torch._scaled_mm with one scale per tensor (no block scaling: what an unscaled or e8m0-scaled
        # loop is to be read against, not a replacement for the path) on config 2's shape and on the deep-K shape
        vend = {}
        for tag, (Mv, Nv, Kv) in (("c2_2048x18432x7168", (2048, 18432, 7168)), ("deep_k_4096x7168x18432", (4096, 7168, 18432))):
            try:
                av = [torch.randn(Mv, Kv, generator=gen, device=dev).to(E4M3) for _ in range(2)]
                bv = [(torch.randn(Nv, Kv, generator=gen, device=dev)).to(E4M3) for _ in range(2)]
                one = torch.ones((), device=dev)
                fns = [(lambda i=i: torch._scaled_mm(av[i], bv[i].t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)) for i in range(2)]
                msv, _ = time_launches(fns, 10, 3)
                vend[tag] = {"ms": msv, "tflops": 2.0 * Mv * Nv * Kv / msv / 1e9, "mfma_frac": 2.0 * Mv * Nv * Kv / msv / 1e9 / FP8_PEAK_TFLOPS}
                del av, bv
            except Exception as e:                  # a torch build without the fp8 path: reported, not fatal
                vend[tag] = {"error": repr(e)[:200]}
            torch.cuda.empty_cache()
        extras["hipblaslt_fp8_tensorwise_scaled_mm"] = vend

    if want("copy"):
        # -------------------------------------------------------------- calibration: a plain device copy of known size
        # (what a streaming read+write kernel reaches on this box; also the reference kernel for scaling the
        # FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run of this script)
        for mib in (32, 256):
            n = mib * 1024 * 1024 // 2
            sets = max(2, 768 // mib)
            src = [torch.empty(n, dtype=torch.bfloat16, device=dev).normal_() for _ in range(sets)]
            dst = [torch.empty(n, dtype=torch.bfloat16, device=dev) for _ in range(sets)]
            ms_c, _ = time_launches([(lambda i=i: dst[i].copy_(src[i])) for i in range(sets)], 24, 6)
            extras[f"copy_{mib}MiB_calibration"] = {"ms": ms_c, "GB/s": 4.0 * n / ms_c / 1e6, "hbm_frac": 4.0 * n / ms_c / 1e6 / HBM_PEAK_GBS,
                                                   "bytes": 4 * n, "kernel": "torch elementwise copy (bf16)"}
            del src, dst
            torch.cuda.empty_cache()
    if want("c2q"):
        # -------------------------------------------------------------- config 2 operand: weight quantisation at full size
        w_big = randn(N, K, std=0.02)
        wq_big = torch.empty(N, K, dtype=torch.uint8, device=dev)
        ws_big = torch.empty(N // 128, K // 128, dtype=torch.float32, device=dev)
        ms_wq, _ = time_launches([lambda: quant_into(w_big, 128, 128, wq_big, ws_big)], 10, 3)
        extras["c2_weight_quant_128x128"] = {"ms": ms_wq, "GB/s": N * K * 3 / ms_wq / 1e6, "hbm_frac": N * K * 3 / ms_wq / 1e6 / HBM_PEAK_GBS,
                                             "bytes": N * K * 3}
        del w_big, wq_big, ws_big
        torch.cuda.empty_cache()
    if want("c1"):
        # -------------------------------------------------------------- config 1: 128x128 quant / dequant
        R = C = 4096
        sets = 12                                   # 12 x (32 + 16 MiB) > 256 MB
        xs = [randn(R, C, std=0.02) for _ in range(sets)]
        for x in xs:
            m = torch.rand(R, C, generator=gen, device=dev) < 1e-3
            x[m] = 1.0
        qs = [torch.empty(R, C, dtype=torch.uint8, device=dev) for _ in range(sets)]
        ss = [torch.empty(R // 128, C // 128, dtype=torch.float32, device=dev) for _ in range(sets)]
        outs = [torch.empty(R, C, dtype=torch.bfloat16, device=dev) for _ in range(sets)]
        qfns = [(lambda i=i: quant_into(xs[i], 128, 128, qs[i], ss[i])) for i in range(sets)]
        ms_q, _ = time_launches(qfns, 48, 12)
        dfns = [(lambda i=i: chk(L.lp_dequant_fp8_block(qs[i].data_ptr(), ss[i].data_ptr(), A.F32, R, C, 128, 128,
                                                        outs[i].data_ptr(), A.BF16, stream()))) for i in range(sets)]
        ms_d, _ = time_launches(dfns, 48, 12)
        bytes_q = R * C * 3 + (R // 128) * (C // 128) * 4
        extras["c1_quant_128x128"] = {"ms": ms_q, "GB/s": bytes_q / ms_q / 1e6, "hbm_frac": bytes_q / ms_q / 1e6 / HBM_PEAK_GBS,
                                      "bytes": bytes_q}
        extras["c1_dequant_128x128"] = {"ms": ms_d, "GB/s": bytes_q / ms_d / 1e6,
                                        "hbm_frac": bytes_q / ms_d / 1e6 / HBM_PEAK_GBS, "bytes": bytes_q}
        # a bare stream of the same bytes: read 32 MiB + write 16 MiB (the quantiser's traffic) and the reverse
        probes = {}
        for wgs in (512, 1024, 2048, 4096):
            fq = [(lambda i=i: PA.check(LP.lp_probe_stream(xs[i].data_ptr(), R * C * 2, qs[i].data_ptr(), R * C, wgs, stream())))
                  for i in range(sets)]
            fd = [(lambda i=i: PA.check(LP.lp_probe_stream(qs[i].data_ptr(), R * C, outs[i].data_ptr(), R * C * 2, wgs, stream())))
                  for i in range(sets)]
            probes[f"read32MiB_write16MiB_{wgs}_workgroups_us"] = time_launches(fq, 48, 12)[0] * 1e3
            probes[f"read16MiB_write32MiB_{wgs}_workgroups_us"] = time_launches(fd, 48, 12)[0] * 1e3
        bq_ = min(v for k, v in probes.items() if k.startswith("read32"))
        bd_ = min(v for k, v in probes.items() if k.startswith("read16"))
        probes["quant_over_bare_stream"] = ms_q * 1e3 / bq_
        probes["dequant_over_bare_stream"] = ms_d * 1e3 / bd_
        probes["bare_stream_hbm_frac"] = {"read32_write16": bytes_q / bq_ / 1e3 / HBM_PEAK_GBS, "read16_write32": bytes_q / bd_ / 1e3 / HBM_PEAK_GBS}
        extras["c1_floor_probe"] = probes
        del xs, qs, ss, outs
        torch.cuda.empty_cache()

    if want("c3"):
        # -------------------------------------------------------------- config 3: skinny GEMM, and the same 64 tokens
        # against config 2's 18432 weight rows (a 132 MB weight stream, long enough to amortise launch and first bytes)
        # (and the transposed projection, K = 18432 against 7168 weight rows, which the decode kernels walk in three rounds
        # of K, with 64 tokens and with one)
        ms_empty, _ = time_launches([lambda: PA.check(LP.lp_probe_stream(None, 0, None, 0, 256, stream()))], 48, 12)
        sink = torch.empty(1 << 20, dtype=torch.uint8, device=dev)
        for tag, probe_tag, M3, N3, K3, sets in (("c3_skinny_gemm", "c3_floor_probe", 64, 4096, 7168, 12),
                                                 ("decode_gemm_64x18432x7168", "decode_64x18432x7168_floor_probe", 64, 18432, 7168, 4),
                                                 ("decode_gemm_64x7168x18432", "decode_64x7168x18432_floor_probe", 64, 7168, 18432, 4),
                                                 ("decode_gemm_1x7168x18432", "decode_1x7168x18432_floor_probe", 1, 7168, 18432, 4),
                                                 # the vocabulary projection as a decode step sees it: 927 MB of weights
                                                 ("decode_gemm_1x129280x7168", "decode_1x129280x7168_floor_probe", 1, 129280, 7168, 1),
                                                 ("decode_gemm_16x129280x7168", "decode_16x129280x7168_floor_probe", 16, 129280, 7168, 1)):
            a3 = randn(M3, K3)
            a3q = torch.empty(M3, K3, dtype=torch.uint8, device=dev)
            a3s = torch.empty(M3, K3 // 128, dtype=torch.float32, device=dev)
            quant_into(a3, 1, 128, a3q, a3s)
            w3q, w3s = [], []                           # sets x N3 x K3 bytes of weights > 256 MB
            for _ in range(sets):
                w = randn(N3, K3, std=0.02)
                q = torch.empty(N3, K3, dtype=torch.uint8, device=dev)
                sc = torch.empty(N3 // 128, K3 // 128, dtype=torch.float32, device=dev)
                quant_into(w, 128, 128, q, sc)
                w3q.append(q)
                w3s.append(sc)
                del w
            c3 = torch.empty(M3, N3, dtype=torch.bfloat16, device=dev)
            nws = L.lp_gemm_workspace_bytes(M3, N3, K3)
            ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=dev)
            fns = [(lambda i=i: chk(L.lp_gemm_fp8_block(a3q.data_ptr(), a3s.data_ptr(), w3q[i].data_ptr(), w3s[i].data_ptr(), A.F32,
                                                        M3, N3, K3, c3.data_ptr(), A.BF16, ws.data_ptr(), nws, stream())))
                   for i in range(sets)]
            ms3, _ = time_launches(fns, 48, 12)
            bytes3 = N3 * K3 + (N3 // 128) * (K3 // 128) * 4 + M3 * K3 + M3 * (K3 // 128) * 4 + M3 * N3 * 2
            extras[tag] = {"ms": ms3, "GB/s": bytes3 / ms3 / 1e6, "hbm_frac": bytes3 / ms3 / 1e6 / HBM_PEAK_GBS,
                           "weight_GB/s": N3 * K3 / ms3 / 1e6, "tflops": 2.0 * M3 * N3 * K3 / ms3 / 1e9, "bytes": bytes3}
            # what the box takes for an empty launch and for a bare stream of the same weight bytes (rotating buffers like above)
            wbytes = N3 * K3
            probes = {"empty_launch_us": ms_empty * 1e3}
            for wgs in (256, 512, 1024, 2048):
                fns = [(lambda i=i: PA.check(LP.lp_probe_stream(w3q[i].data_ptr(), wbytes, sink.data_ptr(), 4096 * wgs // 256, wgs, stream())))
                       for i in range(sets)]
                msp, _ = time_launches(fns, 48, 12)
                probes[f"read_{wbytes // 1000000}MB_{wgs}_workgroups_us"] = msp * 1e3
            best = min(v for k, v in probes.items() if k.startswith("read_"))
            probes["bare_read_best_GB/s"] = wbytes / best / 1e3
            probes["gemm_over_bare_read"] = ms3 * 1e3 / best
            extras[probe_tag] = probes
            del w3q, w3s, c3, ws, a3, a3q, a3s
            torch.cuda.empty_cache()
        del sink

    if want("c5"):
        # -------------------------------------------------------------- config 5: FP4 -> FP8 (fused), whole MoE layer
        E_total, chunk = 256, 256                    # experts per launch: the whole layer, one launch per tensor kind
        shapes = [(2048, 7168), (2048, 7168), (7168, 2048)]
        n_chunksets = 2                              # 2 x ~17.3 GB of buffers, far beyond the Infinity Cache
        bufs = []
        for _ in range(n_chunksets):
            per = []
            for (r, cc) in shapes:
                rows = chunk * r
                packed = torch.randint(0, 256, (rows, cc // 2), generator=gen, device=dev, dtype=torch.int32).to(torch.uint8)
                sc = torch.randint(117, 128, (rows, cc // 32), generator=gen, device=dev, dtype=torch.int32).to(torch.uint8)
                q = torch.empty(rows, cc, dtype=torch.uint8, device=dev)
                so = torch.empty(rows // 128, cc // 128, dtype=torch.float32, device=dev)
                per.append((packed, sc, q, so, rows, cc))
            bufs.append(per)

        def c5_chunk(i):
            def run():
                for (packed, sc, q, so, rows, cc) in bufs[i]:
                    chk(L.lp_fp4_to_fp8_amax(packed.data_ptr(), sc.data_ptr(), rows, cc, A.SCALE_DIV, 1e-12, 0,
                                             q.data_ptr(), so.data_ptr(), A.F32, None, stream()))
            return run

        n_chunks = E_total // chunk
        ms5, _ = time_launches([c5_chunk(i) for i in range(n_chunksets)], max(n_chunks, 4), 2)
        elems = sum(r * cc for r, cc in shapes) * E_total
        bytes5 = elems // 2 + elems // 32 + elems + (elems // 16384) * 4
        total_ms5 = ms5 * n_chunks
        extras["c5_fp4_to_fp8_fused"] = {"ms_total": total_ms5, "GB/s": bytes5 / total_ms5 / 1e6,
                                         "hbm_frac": bytes5 / total_ms5 / 1e6 / HBM_PEAK_GBS, "elements": elems,
                                         "bytes": bytes5, "variant": "fused, bf16 intermediate not written"}

        # a bare stream of the same mix: per tensor read its packed bytes and write its FP8 bytes (17/32 of the kernel's
        # reads: the 1 x 32 scale bytes are left out, so the probe moves slightly less than the kernel)
        probes5 = {}
        for wgs in (2048, 8192, 32768):
            def c5_stream(i, wgs=wgs):
                def run():
                    for (packed, sc, q, so, rows, cc) in bufs[i]:
                        PA.check(LP.lp_probe_stream(packed.data_ptr(), rows * cc // 2, q.data_ptr(), rows * cc, wgs, stream()))
                return run
            msb, _ = time_launches([c5_stream(i) for i in range(n_chunksets)], max(n_chunks, 4), 2)
            probes5[f"read_half_write_one_byte_per_element_{wgs}_workgroups_ms"] = msb * n_chunks
        best5 = min(probes5.values())
        probes5["bare_stream_hbm_frac"] = (elems // 2 + elems) / best5 / 1e6 / HBM_PEAK_GBS
        probes5["fused_over_bare_stream"] = total_ms5 / best5
        extras["c5_floor_probe"] = probes5

        def c5_rebase(i):
            def run():
                for (packed, sc, q, so, rows, cc) in bufs[i]:
                    chk(L.lp_fp4_to_fp8_rebase(packed.data_ptr(), sc.data_ptr(), rows, cc, q.data_ptr(), so.data_ptr(),
                                               A.F32, stream()))
            return run

        ms5r, _ = time_launches([c5_rebase(i) for i in range(n_chunksets)], max(n_chunks, 4), 2)
        extras["c5_fp4_to_fp8_rebase"] = {"ms_total": ms5r * n_chunks, "GB/s": bytes5 / (ms5r * n_chunks) / 1e6,
                                          "hbm_frac": bytes5 / (ms5r * n_chunks) / 1e6 / HBM_PEAK_GBS}
        # FP4 -> bf16 (the converter of tools/convert_deepseek_v4_fp4_to_bf16.py)
        bouts = [torch.empty(p[0][4], p[0][5], dtype=torch.bfloat16, device=dev) for p in bufs]

        def c5_bf16(i):
            packed, sc, q, so, rows, cc = bufs[i][0]
            return lambda: chk(L.lp_dequant_fp4_block(packed.data_ptr(), sc.data_ptr(), A.E8M0, rows, cc, 1, 32, A.FP4_POS_ZERO,
                                                      bouts[i].data_ptr(), A.BF16, stream()))

        ms5b, _ = time_launches([c5_bf16(i) for i in range(n_chunksets)], 6, 2)
        e1 = bufs[0][0][4] * bufs[0][0][5]
        b1 = e1 // 2 + e1 // 32 + e1 * 2
        extras["c5_fp4_to_bf16"] = {"ms": ms5b, "GB/s": b1 / ms5b / 1e6, "hbm_frac": b1 / ms5b / 1e6 / HBM_PEAK_GBS, "bytes": b1}
        # the way back: bf16 -> packed FP4 with 1 x 32 e8m0 scales (quant_fp4_e2m1_scale_e8m0_packed), on the tensors
        # the previous step wrote
        def c5_fp4q(i):
            packed, sc, q, so, rows, cc = bufs[i][0]
            return lambda: chk(L.lp_quant_fp4_block(bouts[i].data_ptr(), A.BF16, rows, cc, 1, 32, packed.data_ptr(),
                                                    sc.data_ptr(), None, stream()))

        ms5q, _ = time_launches([c5_fp4q(i) for i in range(n_chunksets)], 6, 2)
        extras["c5_bf16_to_fp4"] = {"ms": ms5q, "GB/s": b1 / ms5q / 1e6, "hbm_frac": b1 / ms5q / 1e6 / HBM_PEAK_GBS, "bytes": b1}
        # fused QAT conversions of the weight-export path on one expert-sized tensor set (rotating, > 256 MB)
        qs = 6
        wq32 = [torch.randn(2048, 7168, generator=gen, device=dev) * 0.02 for _ in range(qs)]
        wqb = [w.to(torch.bfloat16) for w in wq32]
        q8o = torch.empty(2048, 7168, dtype=torch.uint8, device=dev)
        s8o = torch.empty(16, 56, dtype=torch.uint8, device=dev)
        bo = torch.empty(2048, 7168, dtype=torch.bfloat16, device=dev)
        eq = 2048 * 7168
        msq, _ = time_launches([(lambda i=i: chk(L.lp_fp4_qat_to_fp8(wq32[i].data_ptr(), 2048, 7168, q8o.data_ptr(),
                                                                       s8o.data_ptr(), stream()))) for i in range(qs)], 18, 6)
        extras["fp4_qat_then_to_fp8_2048x7168"] = {"ms": msq, "GB/s": eq * 5 / msq / 1e6, "hbm_frac": eq * 5 / msq / 1e6 / HBM_PEAK_GBS,
                                                   "bytes": eq * 5}
        msq, _ = time_launches([(lambda i=i: chk(L.lp_qdq_fp8_tile128(wqb[i].data_ptr(), 2048, 7168, bo.data_ptr(), stream())))
                                for i in range(qs)], 18, 6)
        extras["fp_qat_128x128_2048x7168"] = {"ms": msq, "GB/s": eq * 4 / msq / 1e6, "hbm_frac": eq * 4 / msq / 1e6 / HBM_PEAK_GBS,
                                              "bytes": eq * 4}
        msq, _ = time_launches([(lambda i=i: chk(L.lp_fp4_qdq_row32(wqb[i].data_ptr(), eq, bo.data_ptr(), None, stream())))
                                for i in range(qs)], 18, 6)
        extras["fp4_simulate_qat_2048x7168"] = {"ms": msq, "GB/s": eq * 4 / msq / 1e6, "hbm_frac": eq * 4 / msq / 1e6 / HBM_PEAK_GBS,
                                                "bytes": eq * 4}
        msq, _ = time_launches([(lambda i=i: chk(L.lp_act_qdq_group(wqb[i].data_ptr(), eq, 64, 1, 0, bo.data_ptr(), None, stream())))
                                for i in range(qs)], 18, 6)
        extras["fp8_simulate_qat_1x64_2048x7168"] = {"ms": msq, "GB/s": eq * 4 / msq / 1e6,
                                                     "hbm_frac": eq * 4 / msq / 1e6 / HBM_PEAK_GBS, "bytes": eq * 4}
        del wq32, wqb, q8o, s8o, bo
        del bufs, bouts
        torch.cuda.empty_cache()

    if want("c4"):
        # -------------------------------------------------------------- config 4: grouped MoE GEMM
        E4, tokens, topk = 256, 8192, 8
        m_splits = zipf_m_splits(E4, tokens, topk, seed=4321)
        offs = torch.zeros(E4 + 1, dtype=torch.int32)
        offs[1:] = torch.cumsum(m_splits, 0)
        offs_d = offs.to(dev)
        Mt = int(offs[-1])
        res4 = {"m_splits_max": int(m_splits.max()), "m_splits_min": int(m_splits.min()),
                "m_splits_zero": int((m_splits == 0).sum()), "rows": Mt,
                "m_splits_histogram": {f"<={hi}": int(((m_splits > lo) & (m_splits <= hi)).sum())
                                       for lo, hi in ((-1, 0), (0, 64), (64, 128), (128, 256), (256, 512), (512, 1024),
                                                      (1024, 2048), (2048, 4096), (4096, 8192))}}
        # rows the launch multiplies over rows that exist: every 256 rows of an expert and a remainder above 128 rows
        # are 256-row tiles, a remainder of 1 .. 128 rows is a 128-row tile; waves whose 64 rows are all missing skip
        # their matrix instructions, so the matrix cores see the rows rounded up to 64
        ms_l = m_splits.tolist()
        tile_rows = sum((r >> 8) * 256 + (256 if (r & 255) > 128 else (128 if (r & 255) else 0)) for r in ms_l)
        mfma_rows = sum((r + 63) // 64 * 64 for r in ms_l)
        res4["padded_over_useful_flops"] = {"by_tile_rows": tile_rows / Mt, "after_idle_wave_rows_are_skipped": mfma_rows / Mt}
        for name, (N4, K4) in (("gate_up", (4096, 7168)), ("down", (7168, 2048))):
            x4 = randn(Mt, K4)
            x4q = torch.empty(Mt, K4, dtype=torch.uint8, device=dev)
            x4s = torch.empty(Mt, K4 // 128, dtype=torch.float32, device=dev)
            quant_into(x4, 1, 128, x4q, x4s)
            del x4
            w4q = torch.empty(E4 * N4, K4, dtype=torch.uint8, device=dev)
            w4s = torch.empty(E4 * N4 // 128, K4 // 128, dtype=torch.float32, device=dev)
            step_e = 32
            for e0 in range(0, E4, step_e):
                w = randn(step_e * N4, K4, std=0.02)
                quant_into(w, 128, 128, w4q[e0 * N4:(e0 + step_e) * N4], w4s[e0 * N4 // 128:(e0 + step_e) * N4 // 128])
                del w
            c4 = torch.empty(Mt, N4, dtype=torch.bfloat16, device=dev)
            fn = lambda: chk(L.lp_gemm_fp8_grouped(x4q.data_ptr(), x4s.data_ptr(), w4q.data_ptr(), w4s.data_ptr(), A.F32,  # noqa: E731
                                                   offs_d.data_ptr(), E4, Mt, N4, K4, c4.data_ptr(), A.BF16, stream()))
            ms4, _ = time_launches([fn], 5, 2)
            fl = 2.0 * Mt * N4 * K4
            touched = int((m_splits > 0).sum())
            by = touched * N4 * K4 + Mt * K4 + Mt * N4 * 2
            res4[name] = {"ms": ms4, "tflops": fl / ms4 / 1e9, "mfma_frac": fl / ms4 / 1e9 / FP8_PEAK_TFLOPS,
                          "hbm_floor_GB": by / 1e9, "hbm_frac_of_floor": by / ms4 / 1e6 / HBM_PEAK_GBS}
            # the same problem with power-of-two (e8m0) scales, which the matrix cores apply themselves: the codes
            # in place are kept (timing does not depend on their values), only the scale tables change type
            x4s8 = torch.randint(118, 128, (Mt, K4 // 128), generator=gen, device=dev, dtype=torch.int32).to(torch.uint8)
            w4s8 = torch.randint(110, 120, (E4 * N4 // 128, K4 // 128), generator=gen, device=dev, dtype=torch.int32).to(torch.uint8)
            fn8 = lambda: chk(L.lp_gemm_fp8_grouped(x4q.data_ptr(), x4s8.data_ptr(), w4q.data_ptr(), w4s8.data_ptr(), A.E8M0,  # noqa: E731
                                                    offs_d.data_ptr(), E4, Mt, N4, K4, c4.data_ptr(), A.BF16, stream()))
            ms48, _ = time_launches([fn8], 5, 2)
            res4[name + "_e8m0_scales"] = {"ms": ms48, "tflops": fl / ms48 / 1e9, "mfma_frac": fl / ms48 / 1e9 / FP8_PEAK_TFLOPS}
            # a decode-sized batch through the same weights: 64 tokens x top-8 = 512 rows over the 256 experts (same Zipf
            # recipe), where the launch is a stream of the weights of the experts that got a row
            m_dec = zipf_m_splits(E4, 64, topk, seed=99)
            offs_dec = torch.zeros(E4 + 1, dtype=torch.int32)
            offs_dec[1:] = torch.cumsum(m_dec, 0)
            offs_dec_d = offs_dec.to(dev)
            rows_dec = int(offs_dec[-1])
            fn_dec = lambda: chk(L.lp_gemm_fp8_grouped(x4q.data_ptr(), x4s.data_ptr(), w4q.data_ptr(), w4s.data_ptr(), A.F32,  # noqa: E731
                                                       offs_dec_d.data_ptr(), E4, rows_dec, N4, K4, c4.data_ptr(), A.BF16, stream()))
            ms_dec, _ = time_launches([fn_dec], 5, 2)
            hit = int((m_dec > 0).sum())
            res4[name + "_decode_sized_512_rows"] = {"ms": ms_dec, "experts_with_rows": hit, "max_rows": int(m_dec.max()),
                                                     "weight_GB/s": hit * N4 * K4 / ms_dec / 1e6,
                                                     "hbm_frac": hit * N4 * K4 / ms_dec / 1e6 / HBM_PEAK_GBS}
            if name == "gate_up":
                # the data gradient of the same layer, dX_e = dY_e W_e on the stored [N4, K4] weights (layout NN,
                # gpatch_v4/models/deepseek_v4/fp8.py:301-313): the kernel that turns the weight operand on its way out of
                # LDS, beside a transposed copy of all weights followed by the forward kernel (what the wrapper did before)
                dyq = torch.randint(0, 120, (Mt, N4), generator=gen, device=dev, dtype=torch.int32).to(torch.uint8)
                dys8 = torch.randint(118, 128, (Mt, N4 // 128), generator=gen, device=dev, dtype=torch.int32).to(torch.uint8)
                dx = torch.empty(Mt, K4, dtype=torch.bfloat16, device=dev)
                fnn = lambda: chk(L.lp_gemm_fp8_grouped_nn(dyq.data_ptr(), dys8.data_ptr(), w4q.data_ptr(), w4s8.data_ptr(), A.E8M0,  # noqa: E731
                                                           offs_d.data_ptr(), E4, Mt, K4, N4, dx.data_ptr(), A.BF16, stream()))
                ms_nn, _ = time_launches([fnn], 5, 2)
                wT = torch.empty(E4, K4, N4, dtype=torch.uint8, device=dev)
                wsT = torch.empty(E4, K4 // 128, N4 // 128, dtype=torch.uint8, device=dev)

                def f_transposed():
                    wT.copy_(w4q.view(E4, N4, K4).transpose(1, 2))
                    wsT.copy_(w4s8.view(E4, N4 // 128, K4 // 128).transpose(1, 2))
                    chk(L.lp_gemm_fp8_grouped(dyq.data_ptr(), dys8.data_ptr(), wT.data_ptr(), wsT.data_ptr(), A.E8M0,
                                              offs_d.data_ptr(), E4, Mt, K4, N4, dx.data_ptr(), A.BF16, stream()))
                ms_tr, _ = time_launches([f_transposed], 3, 1)
                fl_d = 2.0 * Mt * N4 * K4
                dgrad_res = {"ms": ms_nn, "tflops": fl_d / ms_nn / 1e9, "mfma_frac": fl_d / ms_nn / 1e9 / FP8_PEAK_TFLOPS,
                             "over_forward_gate_up_e8m0": ms_nn / ms48,
                             "with_a_transposed_copy_of_the_weights_ms": ms_tr,
                             "kernel": "gemm_asm_grouped_mixed<true, true>: weights read as stored [4096, 7168], operand turned by ds_read_b64_tr_b8"}
                del dyq, dys8, dx, wT, wsT
            del x4q, x4s, w4q, w4s, c4, x4s8, w4s8
            torch.cuda.empty_cache()
        extras["c4_grouped_gemm"] = res4

        # -------------------------------------------------------------- backward of the grouped linear (wgrad pair)
        # column-wise quantiser with transposed output on the gate_up gradient [rows, 4096], and one expert's
        # weight-gradient GEMM dW[4096, 7168] = dY^T[4096, P] X^T[7168, P]^T at P = 1024 rows
        nblk4 = [(int(m) + 127) // 128 for m in m_splits.tolist()]
        pb4 = sum(nblk4)
        dy = randn(Mt, 4096)
        qT = torch.empty(4096 * pb4 * 128, dtype=torch.uint8, device=dev)
        sT = torch.empty(4096 * pb4, dtype=torch.uint8, device=dev)
        fnq = lambda: chk(L.lp_quant_fp8_colwise_t(dy.data_ptr(), A.BF16, Mt, 4096, offs_d.data_ptr(), E4, pb4, 128,  # noqa: E731
                                                   qT.data_ptr(), sT.data_ptr(), A.E8M0, stream()))
        msq, _ = time_launches([fnq], 5, 2)
        byq = Mt * 4096 * 2 + 4096 * pb4 * 129
        Pw = 1024
        a_w = torch.randint(0, 120, (4096, Pw), dtype=torch.uint8, device=dev)
        b_w = torch.randint(0, 120, (7168, Pw), dtype=torch.uint8, device=dev)
        sa_w = torch.full((4096, Pw // 128), 120, dtype=torch.uint8, device=dev)
        sb_w = torch.full((7168, Pw // 128), 121, dtype=torch.uint8, device=dev)
        dw = torch.empty(4096, 7168, dtype=torch.bfloat16, device=dev)
        fnw = lambda: chk(L.lp_gemm_fp8_rowscale(a_w.data_ptr(), sa_w.data_ptr(), b_w.data_ptr(), sb_w.data_ptr(), A.E8M0,  # noqa: E731
                                                 4096, 7168, Pw, dw.data_ptr(), A.BF16, stream()))
        msw, _ = time_launches([fnw], 10, 3)
        # the whole layer's weight gradient, one launch per kind of problem (K a multiple of 512; one K block; two K blocks):
        # 256 problems [4096, 7168] x P_e, config 4's rows per expert padded as the wrapper pads them (experts of at most 256
        # rows to 128 or 256, the others to multiples of 512); operands are random codes (the time does not depend on the
        # values), 15 GB of bf16 out
        from gcore_lowp.grouped_gemm_fp8 import choose_colwise_pad, padded_blocks, rowscale_launches
        padw = choose_colwise_pad(m_splits.tolist())
        nblkw = [padded_blocks(int(m), padw) for m in m_splits.tolist()]
        pbw = sum(nblkw)
        launches_w, _ = rowscale_launches(nblkw)
        kinds_w = {"k_multiple_of_512": sum(1 for nb in nblkw if nb and nb % 4 == 0), "one_k_block": nblkw.count(1),
                   "two_k_blocks": nblkw.count(2), "other": sum(1 for nb in nblkw if nb > 2 and nb % 4)}
        aT = torch.randint(0, 120, (4096 * pbw * 128,), dtype=torch.uint8, device=dev)
        bT = torch.randint(0, 120, (7168 * pbw * 128,), dtype=torch.uint8, device=dev)
        saT = torch.full((4096 * pbw,), 120, dtype=torch.uint8, device=dev)
        sbT = torch.full((7168 * pbw,), 121, dtype=torch.uint8, device=dev)
        dW = torch.empty(E4, 4096, 7168, dtype=torch.bfloat16, device=dev)
        tabs = [(torch.tensor(g, dtype=torch.int32, device=dev), len(g), max(x[1] for x in g), mult)
                for g, mult in launches_w]

        def fng():
            for tab, n, mx, mult in tabs:
                chk(L.lp_gemm_fp8_rowscale_grouped(aT.data_ptr(), saT.data_ptr(), bT.data_ptr(), sbT.data_ptr(), A.E8M0, tab.data_ptr(), n, mx,
                                                   mult, 4096, 7168, dW.data_ptr(), A.BF16, stream()))
        msg, _ = time_launches([fng], 3, 1)
        flg = 2.0 * 4096 * 7168 * pbw * 128
        n_launches_w = len(tabs)
        del aT, bT, saT, sbT, dW, tabs
        extras["grouped_linear_backward"] = {
            "dgrad_grouped_256_experts_65536x4096_to_7168": dgrad_res,
            "wgrad_grouped_256_experts_4096x7168": {"ms": msg, "rows_padded_to": "128 up to 256 rows, 512 beyond" if padw == 0 else padw,
                                                    "problems_by_kernel": kinds_w,
                                                    "tflops_on_padded_rows": flg / msg / 1e9,
                                                    "mfma_frac": flg / msg / 1e9 / FP8_PEAK_TFLOPS,
                                                    "output_GB": E4 * 4096 * 7168 * 2 / 1e9,
                                                    "output_write_GB/s": E4 * 4096 * 7168 * 2 / msg / 1e6, "launches": n_launches_w},
            "quant_colwise_t_65536x4096": {"ms": msq, "GB/s": byq / msq / 1e6, "hbm_frac": byq / msq / 1e6 / HBM_PEAK_GBS, "bytes": byq},
            "wgrad_gemm_rowscale_4096x7168xP1024": {"ms": msw, "tflops": 2.0 * 4096 * 7168 * Pw / msw / 1e9,
                                                    "mfma_frac": 2.0 * 4096 * 7168 * Pw / msw / 1e9 / FP8_PEAK_TFLOPS}}
        del dy, qT, sT, a_w, b_w, sa_w, sb_w, dw
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ CPU baseline (oracle, bounded sample)
    # The eager-PyTorch restatement of the reference's CPU path (oracle/torch_ref.py), on the host cores this job may
    # use: configs 1 to 3 at full size, configs 4 and 5 on a stated subset of the experts and scaled up linearly.
    # One warm-up and three runs each, median.  A reported baseline, not a target.
    cpu = None
    if not args.no_cpu:
        from oracle import torch_ref as T
        threads = torch.get_num_threads()               # the box allots OMP_NUM_THREADS per GPU job; not raised beyond it
        print(f"[bench] CPU baseline on {threads} threads (host shows {os.cpu_count()} cores)\n{torch.__config__.parallel_info()}",
              file=sys.stderr)
        g = torch.Generator().manual_seed(7)

        def med3(fn):
            fn()
            ts = []
            for _ in range(3):
                t0 = time.perf_counter()
                fn()
                ts.append(time.perf_counter() - t0)
            return sorted(ts)[1]

        # config 2, whole problem: fp32 dequantise then fp32 matmul on pre-quantised operands, as the GPU side is timed
        a = torch.randn(M, K, generator=g).to(torch.bfloat16)
        w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
        xq, xs_ = T.quant_block_fp32_scale(a, (1, 128))
        wq, ws_ = T.quant_block_fp32_scale(w, (128, 128))
        t_c2 = med3(lambda: T.gemm_fp8_block_scaling_ref(xq, xs_, wq, ws_))
        cpu = {"value": 2.0 * M * N * K / t_c2 / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
               "host_cores_visible": os.cpu_count(),
               "sample": f"config 2 at full size (M={M}, N={N}, K={K}): fp32 dequantise then fp32 matmul in eager torch on "
                         f"pre-quantised operands, 1 warm-up + 3 runs, median {t_c2 * 1e3:.0f} ms"}
        if not args.no_extras:
            ex = {}
            # config 1 at full size
            x1 = (torch.randn(4096, 4096, generator=g) * 0.02).to(torch.bfloat16)
            q1, s1 = T.quant_block_fp32_scale(x1, (128, 128))
            b1 = 4096 * 4096 * 3 + 32 * 32 * 4
            ex["c1_quant_GB/s"] = b1 / med3(lambda: T.quant_block_fp32_scale(x1, (128, 128))) / 1e9
            ex["c1_dequant_GB/s"] = b1 / med3(lambda: T.dequant_fp4_e2m1_fp8_scale_e8m0_packed(q1, s1.to(torch.bfloat16))) / 1e9
            # config 3 at full size: weight stream of the skinny GEMM
            a3c = torch.randn(64, K, generator=g).to(torch.bfloat16)
            x3q, x3s = T.quant_block_fp32_scale(a3c, (1, 128))
            t3 = med3(lambda: T.gemm_fp8_block_scaling_ref(x3q, x3s, wq[:4096], ws_[:32]))
            ex["c3_skinny_gemm_weight_GB/s"] = 4096 * K / t3 / 1e9
            # config 4 on 4 experts (ranks 9 .. 12 by rows, about 1000 rows each; gate_up; their weights are the first
            # 4 x 4096 rows of the config-2 weight), scaled to the whole problem by flops
            ms4 = zipf_m_splits(256, 8192, 8, seed=4321).tolist()        # (one of the 256 experts has no rows)
            sub = sorted(range(256), key=lambda e: -ms4[e])[8:12]
            rows_sub = [ms4[e] for e in sub]
            x4c = torch.randn(sum(rows_sub), K, generator=g).to(torch.bfloat16)
            x4cq, x4cs = T.quant_block_fp32_scale(x4c, (1, 128), amax_floor=None, zero_scale_to_one=True)
            w4cq = wq[:4 * 4096].view(4, 4096, K)
            w4cs = ws_[:4 * 32].view(4, 32, K // 128)
            t4 = med3(lambda: T.grouped_gemm_fp8_ref(x4cq, x4cs, w4cq, w4cs, rows_sub))
            ex["c4_gate_up_TFLOP/s (4 experts of 256, %d of 65536 rows; extrapolated by flops: whole problem %.1f s)"
               % (sum(rows_sub), t4 * 65536 / sum(rows_sub))] = 2.0 * sum(rows_sub) * 4096 * K / t4 / 1e12
            # config 5 on one expert's three tensors, scaled to 256 experts
            t5 = 0.0
            for (r5, c5) in ((2048, 7168), (2048, 7168), (7168, 2048)):
                pk = torch.randint(0, 256, (r5, c5 // 2), generator=g, dtype=torch.int32).to(torch.uint8).view(torch.int8)
                sc = torch.randint(117, 128, (r5, c5 // 32), generator=g, dtype=torch.int32).to(torch.uint8).view(torch.float8_e8m0fnu)
                t5 += med3(lambda: T.fp4_to_fp8_amax(pk, sc))
            e5 = 3 * 2048 * 7168
            ex["c5_fp4_to_fp8_GB/s (one expert of 256, algorithmic fused bytes; extrapolated: whole layer %.0f s)" % (t5 * 256)] = \
                e5 * (0.5 + 1 / 32 + 1) / t5 / 1e9
            cpu["extras"] = ex

    line = {
        "metric": "block-FP8 GEMM TFLOP/s & %MFMA peak; quant/dequant GB/s & %HBM peak",
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3 x fp8_e4m3 -> f32 accumulate -> bf16", "data": "synthetic",
        "config": {"workload": "C2 dense block-FP8 GEMM: A[2048,7168] 1x128 e4m3 x B[18432,7168] 128x128 e4m3, fp32 scales -> bf16 [2048,18432]",
                   "M": M, "N": N, "K": K, "operands": "pre-quantised, resident in HBM"},
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / FP8_PEAK_TFLOPS, "traffic": measured_traffic("gemm_asm_wide<false, 288>", 512 * 512),
                     "traffic_source": "profiles/traffic.json (rocprofv3 --pmc runs of this script, summarised by profile_summary.py)",
                     "kernel": "gemm_asm_wide<false>: the whole problem in one launch, 512 tiles of 256x288 (two full rounds of 256 CUs)",
                     "launch_ms": ms, "flops_per_launch": flops, "wall_ms_per_step": wall_ms,
                     "tiles_256x256_alone": {"kernel": "gemm_asm<256,256,1>: M=2048, weight rows 0..16383 of 18432, K=7168 (512 tiles)",
                                         "launch_ms": big_ms, "flops_per_launch": big_flops, "tflops": big_tflops,
                                         "frac": big_tflops / FP8_PEAK_TFLOPS, "traffic": measured_traffic("gemm_asm<256, 256, 1, false, 2>", 512 * 512)}},
        "cpu_baseline": cpu,
        "extras": extras,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
