#!/usr/bin/env python3
"""Benchmark of the Hadamard hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--sweep] [--no-cpu]
                    [--only-gemm | --only-fwht | --only-rht | --only-gemv | --only-gemm-f32]

The reference's compound metric has two halves and both are printed at the top level of the one
JSON line:

  value / roofline / cpu_baseline       the fused HT->GEMM  C = W.H(X)/32  at K=1024, M=N=4096 in
                                        bf16 (fp32 accumulate, C in bf16) against the dense bf16
                                        MFMA peak.  A *step* is one call of fused_ht_gemm.
  fwht.value / .roofline / .cpu_baseline  the stand-alone in-place normalised FWHT of a bf16
                                        X[16384, 4096] against the 8 TB/s HBM peak, plus
                                        fwht.dram_bound: the same kernel on 2^30 elements (the
                                        reference harness's size, bench/bench.py:138), which does
                                        not fit the 256 MiB Infinity Cache.

Timing protocol (the reference's, bench/bench.py:112-127): warm-up launches, then K back-to-back
launches inside one event window on the launch stream, inputs resident in HBM.  The matrix-core
bound kernels are warmed for at least 60 ms first (clock ramp).  `others` carries the remaining
configurations (the 15 (K, N, M) shapes of the reference's sweep, fused_ht/benchmark_sweep.py:20-45,
in bf16 and in fp32, each beside transform + vendor GEMM; HT+GEMV with its unfused comparator;
RHT+FP8 quantize; FP8 GEMM).  `fwht.sweep_128MiB` is the bf16 n = 2^4..2^15 sweep of configs[1];
--sweep adds fp16 and fp32.
"""
from __future__ import annotations

import argparse
import hashlib
import importlib
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PKG = "6s894_project_2025_amd"
HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2516.6, "f16": 2516.6, "f32": 157.3, "fp8": 5033.2}
RAMP_MS = 60.0  # untimed device time before a matrix-core-bound kernel is timed (clock ramp)
BASELINE_METRIC = "fused HT+GEMM TFLOP/s (K=1024,M=N=4096) + standalone FWHT HBM GB/s vs peak"


_SHARED_HEADERS = ("common.hpp", "fwht_device.hpp")
_XREG_HEADERS = _SHARED_HEADERS + ("xreg_common.hpp", "lds_layout.hpp")
# which HIP sources each measured kernel is built from: a traffic figure is reported only while
# these are what they were when it was measured
TRAFFIC_SOURCES = {
    "fused_ht_gemm_bf16": _XREG_HEADERS + ("xreg_mfma16.hpp", "fused_gemm_xreg.hip"),
    "fused_ht_gemm_bf16_K2048_M4096_N4096": _XREG_HEADERS + ("xreg_mfma16.hpp", "fused_gemm_xreg_k2048.hip"),
    "fused_ht_gemm_bf16_K4096_M4096_N4096": _XREG_HEADERS + ("xreg_mfma16.hpp", "fused_gemm_xreg_k2048.hip"),
    "fused_ht_gemm_f32": _XREG_HEADERS + ("fused_gemm_xreg_f32.hip",),
    "fwht_bf16_16384x4096": _SHARED_HEADERS + ("hadamard_device.hpp", "fwht.hip"),
    "fwht_bf16_2^30_n4096": _SHARED_HEADERS + ("hadamard_device.hpp", "fwht.hip"),
    "fwht_bf16_2^30_n32768": _SHARED_HEADERS + ("hadamard_device.hpp", "fwht.hip"),
    "rht_quant_fp8_8192x4096": _SHARED_HEADERS + ("rht_fp8.hip",),
    "fp8_gemm_8192x14336x4096_l2_fill_plus_write": ("common.hpp", "fp8_gemm.hip"),
}


def kernel_sources_digest(names) -> str:
    """sha256 over the named HIP sources (names and contents)."""
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, PKG, "csrc")
    for name in sorted(names):
        h.update(name.encode())
        with open(os.path.join(csrc, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def load_traffic() -> dict:
    """HBM bytes per launch recorded from `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` runs
    (profiles/hbm_traffic.json, figures taken from the summaries beside it).  Every entry names the
    digest of the kernel sources it was measured on (TRAFFIC_SOURCES); an entry whose sources have
    changed since is dropped, i.e. reported as null rather than as a stale number."""
    p = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if not os.path.exists(p):
        return {}
    with open(p) as f:
        rec = json.load(f)
    out = {}
    for key, entry in rec.get("entries", {}).items():
        if key in TRAFFIC_SOURCES and entry.get("sources_sha256") == kernel_sources_digest(TRAFFIC_SOURCES[key]):
            out[key] = entry.get("bytes_per_launch")
    return out


def roofline(bound, achieved, peak, unit, traffic, **extra):
    r = {"bound": bound, "achieved": round(achieved, 1), "peak": peak, "unit": unit,
         "frac": round(achieved / peak, 4), "traffic": traffic}
    r.update(extra)
    return r


def fwht_sweep(hada, events_ms, torch, dev, dtypes, calls=50):
    """In-place transform of a 128 MiB tensor for every n = 2^4 .. 2^15: 3 warm-up launches, then
    `calls` back-to-back launches in one event window; bytes = one read + one write."""
    sweep = {}
    for dname, dt, es in dtypes:
        for p in range(4, 16):
            nn = 1 << p
            numel = (128 << 20) // es
            t = torch.randn(numel // nn, nn, device=dev).to(dt)
            ms, _ = events_ms(lambda: hada.hadamard_transform(t, inplace=True), calls, 3)
            gbs = 2 * numel * es / ms / 1e6
            sweep[f"{dname}_n{nn}"] = {"us": round(ms * 1e3, 2), "GB/s": round(gbs, 1),
                                       "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
            del t
    return sweep


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--sweep", action="store_true", help="also time n = 2^4..2^15 (128 MiB each)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--only-gemm-large-k", action="store_true",
                    help="fused bf16 GEMM at K = 2048 and 4096, M = N = 4096, nothing else (profiling)")
    for flag, what in (("fwht", "stand-alone transform"), ("gemm", "fused bf16 GEMM"),
                       ("gemm-f32", "fused fp32 GEMM"), ("gemv", "fused HT+GEMV"),
                       ("rht", "RHT + FP8 quantize and FP8 GEMM")):
        ap.add_argument(f"--only-{flag}", action="store_true", help=f"{what} only (profiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.stderr.write("bench.py: this build runs on exactly one GPU; --gpus must be 1 "
                         "(rows are independent, so several GPUs would each take a row slab with no exchange)\n")
        return 2

    import torch

    if not torch.cuda.is_available():
        sys.stderr.write("bench.py: no GPU visible\n")
        return 2
    hada = importlib.import_module(PKG)
    timing = importlib.import_module(PKG + ".timing")
    events_ms, steady_ms = timing.event_window_ms, timing.steady_window_ms
    dev = torch.device("cuda:0")
    traffic = load_traffic()
    steps, warmup = args.steps, args.warmup
    only = [k for k in ("fwht", "gemm", "gemm_f32", "gemv", "rht") if getattr(args, "only_" + k)]
    want = (lambda k: not only or k in only)

    result: dict = {}
    others: dict = {}

    if args.only_gemm_large_k:
        out = {}
        for Kx in (2048, 4096):
            Wx = torch.randn(4096, Kx, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(dev)
            Xx = torch.randn(4096, Kx, generator=torch.Generator().manual_seed(0)).to(torch.bfloat16).to(dev)
            f_ms, _ = steady_ms(lambda: hada.fused_ht_gemm(Wx, Xx), max(10, min(steps, 50)), 30.0)
            out[f"fused_ht_gemm_bf16_K{Kx}_M4096_N4096"] = {"us": round(f_ms * 1e3, 2)}
        print(json.dumps(out))
        return 0

    # ---- fused HT -> GEMM, bf16 (config 4): the first half of the metric -----------------------------
    M = N = 4096
    K = 1024
    flops = 2 * M * N * K
    if want("gemm"):
        W = torch.randn(M, K, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(dev)
        Xt = torch.randn(N, K, generator=torch.Generator().manual_seed(0)).to(torch.bfloat16).to(dev)
        C = hada.fused_ht_gemm(W, Xt)
        # whole-output check against the unfused product of the library's own transform
        ref = torch.matmul(W.float(), hada.hadamard_transform(Xt).float().t())
        err = ((C.float() - ref).abs().max() / ref.abs().max()).item()
        del ref
        gsteps = max(10, steps)
        steady_ms(lambda: hada.fused_ht_gemm(W, Xt), 4, RAMP_MS)  # clock ramp, untimed
        ms, wall_ms = events_ms(lambda: hada.fused_ht_gemm(W, Xt), gsteps, warmup)
        tf = flops / ms / 1e9
        mm_ms, _ = steady_ms(lambda: torch.matmul(W, Xt.t()), gsteps, RAMP_MS)
        # the reference's "Baseline (Unfused)" (fusion_pipelined.cu:640-656): transform kernel, H(X)
        # through HBM, then the GEMM (here the vendor library's)
        un_ms, _ = steady_ms(lambda: torch.matmul(W, hada.hadamard_transform(Xt).t()), gsteps, RAMP_MS)
        # what this box sustains with nothing but MFMAs (random bf16 operands, one wavefront per
        # SIMD with four LDS fragment reads per step, the regime of the fused kernel), and the
        # launch-to-launch time of a kernel that does next to nothing
        harness = importlib.import_module("6s894_project_2025_amd.harness")
        probe = harness.mfma_probe(16, 4, 1, Xt.reshape(-1)[:32768], 4096, 20, 30.0)
        floor = harness.mfma_probe(16, 0, 1, Xt.reshape(-1)[:32768], 4, 200, 0.0)
        result.update({
            "metric": BASELINE_METRIC,
            "value": round(tf, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": gsteps, "warmup": warmup,
            "warmup_protocol": {
                "clock_ramp_ms": RAMP_MS, "calls_after_ramp": warmup,
                "note": "every matrix-core-bound timing (this one, the vendor GEMM, the unfused path, the "
                        "`others` GEMM rows) is preceded by at least clock_ramp_ms of untimed back-to-back "
                        "launches of the same call (the clocks keep settling for ~30 ms of sustained load); "
                        "the headline then runs `warmup` more untimed calls before the timed window, the "
                        "comparators go straight into theirs; `others` rows ramp for 30 ms"},
            "ms_per_step": round(ms, 6), "wall_ms_per_step": round(wall_ms, 6),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "BASELINE configs[3]: fused C = W.(H_1024 X)/32, W[4096,1024] seed 1, "
                                   "Xt[4096,1024] seed 0, iid N(0,1), bf16 in, fp32 accumulate, bf16 out; "
                                   "`value` is this half of the metric, `fwht` the other",
                       "M": M, "N": N, "K": K, "algorithmic_flops_per_step": flops},
            "roofline": roofline("mfma", tf, PEAK_TFLOPS["bf16"], "TFLOP/s",
                                 traffic.get("fused_ht_gemm_bf16"),
                                 kernel="fused_ht_gemm_xreg_kernel<BF16,1024,false>"),
            "checks": {"fused_vs_unfused_max_rel_diff": err},
            "library_gemm_without_transform_tflops": round(flops / mm_ms / 1e9, 1),
            "unfused_transform_then_library_gemm_ms": round(un_ms, 6),
            "fused_over_unfused_speedup": round(un_ms / ms, 3),
            "matrix_core_probe": {
                "sustained_tflops": round(probe["tflops"], 1), "shader_ghz": round(probe["ghz"], 3),
                "frac_of_peak": round(probe["tflops"] / PEAK_TFLOPS["bf16"], 4),
                "note": "back-to-back v_mfma_f32_16x16x32_bf16 on every SIMD from registers, random bf16 "
                        "operands (mi_probe_mfma_rate, libmi_probe.so): the rate this box sustains under full matrix-core "
                        "load; value / sustained_tflops = " + str(round(tf / probe["tflops"], 3))},
            "launch_floor_us": round(floor["us_per_launch"], 2),
        })
        del W, Xt, C

    # ---- stand-alone FWHT (config 2): the second half ------------------------------------------------
    rows, n = 16384, 4096
    x_cpu = None
    if want("fwht"):
        g = torch.Generator().manual_seed(0)
        x_cpu = torch.randn(rows, n, generator=g, dtype=torch.float32).to(torch.bfloat16)
        x = x_cpu.to(dev)
        ms, wall_ms = events_ms(lambda: hada.hadamard_transform(x, inplace=True), steps, warmup)
        alg_bytes = 2 * rows * n * 2
        gbs = alg_bytes / ms / 1e6
        # size-independent sanity on the timed buffer: an even number of normalised transforms
        # returns the input (up to bf16 rounding drift)
        if (steps + warmup) % 2 == 1:
            hada.hadamard_transform(x, inplace=True)
        drift = (x.float() - x_cpu.to(dev).float()).abs().max().item()
        add_ms, _ = events_ms(lambda: x.add_(1), min(steps, 50), 3)
        fw = {
            "metric": "standalone FWHT HBM GB/s (bf16 [16384,4096], in place)",
            "value": round(gbs, 1), "unit": "GB/s", "steps": steps, "warmup": warmup,
            "ms_per_step": round(ms, 6), "wall_ms_per_step": round(wall_ms, 6),
            "config": {"workload": "BASELINE configs[1]: in-place normalised FWHT over the last dim, "
                                   "bf16 X[16384,4096] iid N(0,1) seed 0, scale 1/64",
                       "rows": rows, "n": n, "algorithmic_bytes_per_step": alg_bytes},
            "roofline": roofline("hbm", gbs, HBM_PEAK_GBS, "GB/s", traffic.get("fwht_bf16_16384x4096"),
                                 kernel="fwht_reg_kernel<Io16<BF16>,8,3>",
                                 add_one_proxy_gbs=round(alg_bytes / add_ms / 1e6, 1),
                                 note="the 128 MiB buffer is re-run in place and fits the 256 MiB "
                                      "Infinity Cache: this figure is cache-assisted; dram_bound below "
                                      "is the same kernel on a tensor that does not fit"),
            "checks": {"max_abs_drift_after_even_number_of_transforms": drift},
        }
        del x
        # DRAM-bound rows: 2^30 bf16 elements (2 GiB), the reference harness's size
        dram = {}
        for nn in (4096, 32768):
            big = torch.empty((1 << 30) // nn, nn, dtype=torch.bfloat16, device=dev).normal_()
            bsteps = max(5, min(steps, 20))
            bms, _ = events_ms(lambda: hada.hadamard_transform(big, inplace=True), bsteps, 2)
            ams, _ = events_ms(lambda: big.add_(1), bsteps, 2)
            bb = 2 * big.numel() * 2
            dram[f"bf16_2^30_elements_n{nn}"] = {
                "ms_per_step": round(bms, 5), "algorithmic_bytes_per_step": bb,
                "roofline": roofline("hbm", bb / bms / 1e6, HBM_PEAK_GBS, "GB/s",
                                     traffic.get(f"fwht_bf16_2^30_n{nn}"),
                                     add_one_proxy_gbs=round(bb / ams / 1e6, 1))}
            del big
        fw["dram_bound"] = dram
        # configs[1]'s sweep: last dim 2^4 .. 2^15, row count chosen so that each tensor is 128 MiB
        # (bench/bench.py:133,138 of the reference sweeps the same sizes); bf16 here, --sweep adds
        # fp16 and fp32
        fw["sweep_128MiB"] = fwht_sweep(hada, events_ms, torch, dev, (("bf16", torch.bfloat16, 2),))
        if result:
            result["fwht"] = fw
        else:
            result = fw
    if only == ["fwht"] or only == ["gemm"]:
        print(json.dumps(result))
        return 0

    # ---- the same kernel at other sizes: larger N and M amortise the prologue, K = 512 halves the LDS
    # traffic per flop; K = 2048 and 4096 run the kernel that splits K over wavefront pairs (bf16,
    # fused / vendor GEMM without transform / transform + vendor GEMM) --------------------------------
    if not only:
        # the reference's 15 sweep shapes (fused_ht/benchmark_sweep.py:20-45) but the headline one,
        # which is the top-level record, and two larger ones
        shapes = [(k, sz, sz) for k in (256, 512, 1024, 2048, 4096) for sz in (1024, 2048, 4096)
                  if (k, sz) != (K, M)] + [(1024, 8192, 8192), (512, 8192, 8192)]
        for (Kx, Mx, Nx) in shapes:
            Wx = torch.randn(Mx, Kx, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(dev)
            Xx = torch.randn(Nx, Kx, generator=torch.Generator().manual_seed(0)).to(torch.bfloat16).to(dev)
            fx = 2 * Mx * Nx * Kx
            f_ms, _ = steady_ms(lambda: hada.fused_ht_gemm(Wx, Xx), 30, 30.0)
            v_ms, _ = steady_ms(lambda: torch.matmul(Wx, Xx.t()), 30, 30.0)
            u_ms, _ = steady_ms(lambda: torch.matmul(Wx, hada.hadamard_transform(Xx).t()), 30, 30.0)
            others[f"fused_ht_gemm_bf16_K{Kx}_M{Mx}_N{Nx}"] = {
                "us": round(f_ms * 1e3, 2), "algorithmic_flops": fx,
                "roofline": roofline("mfma", fx / f_ms / 1e9, PEAK_TFLOPS["bf16"], "TFLOP/s",
                                     traffic.get(f"fused_ht_gemm_bf16_K{Kx}_M{Mx}_N{Nx}")),
                "library_gemm_without_transform_us": round(v_ms * 1e3, 2),
                "unfused_transform_then_library_gemm_us": round(u_ms * 1e3, 2),
                "fused_over_unfused_speedup": round(u_ms / f_ms, 3)}
            del Wx, Xx

    # ---- fp32 fused GEMM -------------------------------------------------------------------------------
    if want("gemm_f32"):
        W = torch.randn(M, K, generator=torch.Generator().manual_seed(1)).to(dev)
        Xt = torch.randn(N, K, generator=torch.Generator().manual_seed(0)).to(dev)
        gsteps = max(10, min(steps, 50))
        ms, _ = steady_ms(lambda: hada.fused_ht_gemm(W, Xt), gsteps)
        tf = flops / ms / 1e9
        others["fused_ht_gemm_f32"] = {
            "metric": "fused HT+GEMM TFLOP/s (K=1024, M=N=4096, f32 in/out, fp32 MFMA)",
            "value": round(tf, 1), "unit": "TFLOP/s", "ms_per_step": round(ms, 6), "steps": gsteps,
            "algorithmic_flops_per_step": flops,
            "roofline": roofline("mfma", tf, PEAK_TFLOPS["f32"], "TFLOP/s",
                                 traffic.get("fused_ht_gemm_f32"))}
        u_ms, _ = steady_ms(lambda: torch.matmul(W, hada.hadamard_transform(Xt).t()), 10, 30.0)
        others["fused_ht_gemm_f32"]["unfused_transform_then_library_gemm_us"] = round(u_ms * 1e3, 2)
        others["fused_ht_gemm_f32"]["fused_over_unfused_speedup"] = round(u_ms / ms, 3)
        del W, Xt
        # the other K of the reference's sweep at the same M = N (fp32 is the reference's precision)
        if not only:
            for Kx, Sx in [(k, sz) for k in (256, 512, 1024, 2048, 4096) for sz in (1024, 2048, 4096)
                           if (k, sz) != (K, M)]:
                Wx = torch.randn(Sx, Kx, generator=torch.Generator().manual_seed(1)).to(dev)
                Xx = torch.randn(Sx, Kx, generator=torch.Generator().manual_seed(0)).to(dev)
                fx = 2 * Sx * Sx * Kx
                f_ms, _ = steady_ms(lambda: hada.fused_ht_gemm(Wx, Xx), 10, 30.0)
                u_ms, _ = steady_ms(lambda: torch.matmul(Wx, hada.hadamard_transform(Xx).t()), 10, 30.0)
                others[f"fused_ht_gemm_f32_K{Kx}_M{Sx}_N{Sx}"] = {
                    "us": round(f_ms * 1e3, 2), "algorithmic_flops": fx,
                    "roofline": roofline("mfma", fx / f_ms / 1e9, PEAK_TFLOPS["f32"], "TFLOP/s", None),
                    "unfused_transform_then_library_gemm_us": round(u_ms * 1e3, 2),
                    "fused_over_unfused_speedup": round(u_ms / f_ms, 3)}
                del Wx, Xx

    # ---- fused HT+GEMV and its unfused comparator (fwht_gemv_fusion.cu:323-363) ----------------------
    if want("gemv"):
        # config 3 (M = N = 256, B = 512; M = N = 1024, B = 8 .. 512) and the two large shapes of the
        # reference's own benchmark list (fwht_gemv_fusion.cu:643-653)
        for (m, nn, b) in ((256, 256, 512), (1024, 1024, 8), (1024, 1024, 64), (1024, 1024, 256),
                           (1024, 1024, 512), (1024, 1024, 2048), (2048, 2048, 512)):
            Wg = torch.randn(m, nn, device=dev) / math.sqrt(nn)
            X = torch.randn(nn, b, device=dev)
            Xcols = X.t().contiguous()  # untimed layout change for the unfused leg's transform

            def unfused():
                return torch.matmul(Wg, hada.hadamard_transform(Xcols).t())

            Y = hada.fused_ht_gemv(Wg, X)
            ref = unfused()
            gerr = ((Y - ref).abs().max() / ref.abs().max()).item()
            # both legs past the clock ramp, like every other figure of this file: on a chip that has
            # just left idle the leg that is timed first runs at a lower clock than the second
            ms, _ = steady_ms(lambda: hada.fused_ht_gemv(Wg, X), 50)
            ums, _ = steady_ms(unfused, 50)
            byt = 4 * (m * nn + nn * b + m * b)
            flo = 2 * m * nn * b + int(nn * math.log2(nn) * b)
            others[f"fused_ht_gemv_M{m}_N{nn}_B{b}"] = {
                "us": round(ms * 1e3, 2), "unfused_transform_then_library_gemm_us": round(ums * 1e3, 2),
                "fused_over_unfused_speedup": round(ums / ms, 2),
                "fused_vs_unfused_max_rel_diff": gerr,
                "algorithmic_bytes": byt, "algorithmic_flops": flo,
                "GB/s": round(byt / ms / 1e6, 1), "TFLOP/s": round(flo / ms / 1e9, 3)}
            del Wg, X, Xcols

    # ---- RHT + FP8 quantize, FP8 GEMM (config 5) -------------------------------------------------------
    if want("rht"):
        T, nq, Nw = 8192, 4096, 14336
        xa = torch.randn(T, nq, generator=torch.Generator().manual_seed(0))
        outl = torch.randperm(nq, generator=torch.Generator().manual_seed(3))[:41]  # 1 % outlier channels
        xa[:, outl] *= 50.0
        xa = xa.to(torch.bfloat16).to(dev)
        sign = (1 - 2 * torch.randint(0, 2, (nq,), generator=torch.Generator().manual_seed(2))
                ).to(torch.int8).to(dev)
        ms, _ = steady_ms(lambda: hada.rht_quant_fp8(xa, sign), 50)
        qbytes = T * nq * 3 + T * 4
        others["rht_quant_fp8_8192x4096"] = {
            "us": round(ms * 1e3, 2), "algorithmic_bytes": qbytes,
            "roofline": roofline("hbm", qbytes / ms / 1e6, HBM_PEAK_GBS, "GB/s",
                                 traffic.get("rht_quant_fp8_8192x4096"))}
        qx, sx = hada.rht_quant_fp8(xa, sign)
        w = (torch.randn(Nw, nq, device=dev) * 0.02).to(torch.bfloat16)
        qw, sw = hada.rht_quant_fp8(w, sign)
        ms, _ = steady_ms(lambda: hada.fp8_gemm_rowscale(qx, sx, qw, sw), 20)
        fl = 2 * T * Nw * nq
        entry = {"us": round(ms * 1e3, 1), "algorithmic_flops": fl,
                 "roofline": roofline("mfma", fl / ms / 1e9, PEAK_TFLOPS["fp8"], "TFLOP/s",
                                      traffic.get("fp8_gemm_8192x14336x4096_l2_fill_plus_write"))}
        try:  # the vendor library's row-scaled FP8 GEMM on the same operands, for comparison only
            lib_ms, _ = steady_ms(lambda: torch._scaled_mm(
                qx, qw.t(), scale_a=sx.view(-1, 1), scale_b=sw.view(1, -1), out_dtype=torch.bfloat16), 20)
            entry["library_scaled_mm_rowwise_us"] = round(lib_ms * 1e3, 1)
            entry["library_scaled_mm_rowwise_tflops"] = round(fl / lib_ms / 1e9, 1)
        except Exception as ex:  # not every torch build exposes it
            entry["library_scaled_mm_rowwise_us"] = f"unavailable: {str(ex)[:80]}"
        others["fp8_gemm_8192x14336x4096"] = entry
        del xa, w, qx, qw
    if only:
        print(json.dumps(result if result else others))
        return 0

    if args.sweep:
        others["fwht_sweep_128MiB"] = fwht_sweep(hada, events_ms, torch, dev,
                                                 (("f16", torch.float16, 2), ("f32", torch.float32, 4)))
    result["others"] = others

    # ---- CPU baselines: the reference's truth path on the host cores ----------------------------------
    if not args.no_cpu:
        import scipy.linalg

        import oracle  # CPU restatement: only this leg uses it

        nthreads = torch.get_num_threads()

        def cpu_median_s(fn, warm, reps):
            for _ in range(warm):
                fn()
            ts = []
            for _ in range(reps):
                t0 = time.perf_counter()
                fn()
                ts.append(time.perf_counter() - t0)
            return sorted(ts)[len(ts) // 2]

        # fused configuration: W @ (H_K @ X) in fp32, whole configuration
        Wc = torch.randn(M, K, generator=torch.Generator().manual_seed(1))
        Xc = torch.randn(N, K, generator=torch.Generator().manual_seed(0)).t().contiguous()
        Hk = torch.tensor(scipy.linalg.hadamard(K), dtype=torch.float32) / math.sqrt(K)
        fdt = cpu_median_s(lambda: Wc @ (Hk @ Xc), 2, 5)
        result["cpu_baseline"] = {
            "value": round(flops / fdt / 1e12, 4), "unit": "TFLOP/s", "cores": nthreads, "kind": "port",
            "ms": round(fdt * 1e3, 2),
            "sample": "torch CPU fp32 W @ (H_1024 @ X), whole configuration, matrices built once "
                      f"(untimed), median of 5 after 2 warm-up calls; flops counted as 2MNK; os.cpu_count()={os.cpu_count()}"}
        del Wc, Xc, Hk

        # transform: x @ (hadamard(4096)/64) in bf16 on a bounded row sample (~10 s of host work)
        sample = 64
        xs = x_cpu[:sample].clone()
        oracle.hadamard_matrix_ref(xs)  # builds the matrix, warms the thread pool
        t0 = time.perf_counter()
        oracle.hadamard_matrix_ref(xs)
        est = time.perf_counter() - t0
        sample = int(max(64, min(rows, 64 * (10.0 / max(est, 1e-3)) / 13)))
        xs = x_cpu[:sample].clone()
        H = (torch.tensor(scipy.linalg.hadamard(n), dtype=torch.float32) / math.sqrt(n)).to(torch.bfloat16)
        dt_s = cpu_median_s(lambda: xs @ H, 3, 10)
        # the C restatement's O(n log n) butterfly on one core, over the whole batch (under a second)
        xb = x_cpu.float().numpy()
        oracle.fwht_f32(xb[:64])
        t0 = time.perf_counter()
        oracle.fwht_f32(xb)
        bdt = time.perf_counter() - t0
        result["fwht"]["cpu_baseline"] = {
            "value": round(2 * sample * n * 2 / dt_s / 1e9, 4), "unit": "GB/s", "cores": nthreads,
            "kind": "port",
            "sample": f"torch CPU x @ (hadamard(4096)/64).to(bf16) on the first {sample} of 16384 rows "
                      "(matrix built once, untimed), median of 10 calls after 3 warm-up calls",
            "ms_for_sample": round(dt_s * 1e3, 3),
            "ms_extrapolated_full_batch": round(dt_s * 1e3 * rows / sample, 1),
            "butterfly_port": {"value": round(2 * rows * n * 2 / bdt / 1e9, 4), "unit": "GB/s", "cores": 1,
                               "sample": f"oracle_fwht_f32 (plain C butterfly, fp32) on all {rows} rows; "
                                         "bytes counted at the workload's 2 B per element",
                               "ms_for_sample": round(bdt * 1e3, 3)}}

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
