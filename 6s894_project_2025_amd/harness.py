"""Benchmark / check harness around the ops, following the reference's protocols.

Sub-commands (run from the repository root)::

    python -m 6s894_project_2025_amd.harness fwht  [--check] [--runs-per-size 400] [--sizes ...]
    python -m 6s894_project_2025_amd.harness fused [--dtype bf16|f32] [--runs 8] [--out-prefix P]
    python -m 6s894_project_2025_amd.harness plot P.csv [--out-dir plots]
    python -m 6s894_project_2025_amd.harness gemv  [--iters 100] [--out-prefix P]
    python -m 6s894_project_2025_amd.harness mfma  [--steps 4096]
    python -m 6s894_project_2025_amd.harness issue
    python -m 6s894_project_2025_amd.harness power [--seconds 1.5]

``fwht`` follows the protocol of the reference's bench/bench.py: a registry of in-place cases
(add-one roofline proxies around the transform, :96-103), a correctness pass of every case with
``allclose(atol=1e-2 fp16 / 5e-2 bf16, rtol=0)`` (:159-203), timing as "3 warm-up calls, then N
back-to-back calls on the same buffer inside one event window" (:112-127), and a JSON dump with
the same fields (:226-237, :291-300).  The reference checks its own kernel against HadaCore; here
the truth is the matrix path ``t @ (hadamard(n) * n**-0.5)`` evaluated with torch on the GPU
(bench/bench.py:49-59).  The check runs each case on the full-size buffer, because the launcher
picks its kernel variant by tensor size, and compares row slices of the result.

``fused`` covers the 15 (K, N, M) shapes of fused_ht/benchmark_sweep.py:20-45 with its FLOP and
byte models (:123-140), but with run-time shapes (no regex edit + recompile), and times the
unfused baseline next to the fused kernel the way fused_ht/fusion_pipelined.cu:640-683 does:
"transform kernel, then GEMM" (here: ``hadamard_transform`` + ``torch.matmul``, i.e. the vendor
GEMM) versus ``fused_ht_gemm``; min over runs after 2 warm-ups (:631-683), max-abs difference
between the two reported like :694-703.

``gemv`` is the benchmark half of fused_ht/fwht_gemv_fusion.cu's main() (:643-653): its seven
(M, N, B) shapes, fused HT+GEMV against transform-then-GEMM, with its FLOP count and its
memory-traffic model (:576-588).

``mfma``, ``issue`` and ``power`` are measurement aids with no counterpart in the reference: the
matrix-core rate and clock the chip sustains, what a SIMD can issue beside its MFMAs and per vector
instruction kind, and package power and shader clock while each kernel runs (read from the amdgpu
sysfs files).
"""
from __future__ import annotations

import argparse
import csv
import functools
import json
import math
import sys
import time
from dataclasses import dataclass, field
from datetime import datetime
from typing import Any, Callable

import torch

from .ops import fused_ht_gemm, fused_ht_gemv, hadamard_transform
from .timing import best_single_call_ms, event_window_ms, steady_window_ms

ATOL = {torch.float16: 1e-2, torch.bfloat16: 5e-2, torch.float32: 1e-4}
DTYPES = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}


@functools.lru_cache(maxsize=None)
def _normalised_sylvester(n: int) -> torch.Tensor:
    """H_n / sqrt(n) on the GPU in fp32, H[i][j] = (-1)**popcount(i & j)."""
    idx = torch.arange(n, device="cuda")
    bits = idx[:, None] & idx[None, :]
    parity = torch.zeros_like(bits)
    for b in range(max(1, n.bit_length())):
        parity ^= (bits >> b) & 1
    return (1.0 - 2.0 * parity.to(torch.float32)) / math.sqrt(n)


@dataclass(frozen=True)
class Case:
    """One in-place benchmark case: ``run`` is what gets timed, ``truth`` returns what ``run``
    must leave in a buffer that held ``t``.  The registry below keeps the reference's order
    (bench/bench.py:96-103): add-one roofline proxies before and after the transform."""
    run: Callable[[torch.Tensor], Any]
    truth: Callable[[torch.Tensor], torch.Tensor]


def _matrix_truth(t: torch.Tensor) -> torch.Tensor:
    # the reference's definition of correct: t @ (hadamard(n) * n**-0.5) in t's dtype
    # (HadaCore/test.py:27,40; bench/bench.py:49-59)
    return t @ _normalised_sylvester(int(t.shape[-1])).to(t.dtype)


_ADD_ONE = Case(run=lambda t: t.add_(1), truth=lambda t: t + 1)
CASES: dict[str, Case] = {
    "AddOne1": _ADD_ONE,
    "AddOne2": _ADD_ONE,
    "Ours": Case(run=lambda t: hadamard_transform(t, inplace=True), truth=_matrix_truth),
    "AddOne3": _ADD_ONE,
}


@dataclass
class TestConfig:
    check: bool = False
    runs_per_size: int = 400
    json_output_file: str | None = None
    benchmark_cases: list[str] = field(default_factory=lambda: list(CASES))
    test_sizes: list[int] = field(default_factory=lambda: [1 << x for x in range(8, 16)])
    elem_counts: list[int] = field(default_factory=lambda: [1 << 30])
    dtypes: tuple[torch.dtype, ...] = (torch.float16, torch.bfloat16)


def _check_case(name: str, case: Case, full: torch.Tensor) -> None:
    """Runs the case on the *full-size* buffer (so the launch path that gets timed is the one that
    gets checked) and compares bounded row slices of the result with the truth path, which costs
    O(rows * n^2) and is therefore evaluated on slices only.  Only those slices are put back to
    their input values; the caller resets the whole buffer between cases."""
    rows, n = full.shape
    take = min(rows, max(1, (1 << 21) // n))
    starts = sorted({0, max(0, rows // 2 - take // 2), rows - take})
    before = [full[s:s + take].clone() for s in starts]
    case.run(full)
    for s, src in zip(starts, before):
        got, want = full[s:s + take], case.truth(src)
        if not torch.allclose(want, got, atol=ATOL.get(full.dtype, 1e-2), rtol=0):
            worst = (want.float() - got.float()).abs().max().item()
            print(f"Failed test: {name} {n}x{rows} {full.dtype} rows {s}..{s + take}; max diff {worst}")
            raise SystemExit(1)
        got.copy_(src)


def run_fwht(cfg: TestConfig) -> list[dict[str, Any]]:
    print("test_sizes_m: ", cfg.test_sizes)
    print("test_elem_counts: ", cfg.elem_counts)
    print("cases: ", cfg.benchmark_cases)
    torch.manual_seed(0)
    device_name = torch.cuda.get_device_name(0)
    print(f"running on {device_name}\n")
    results: list[dict[str, Any]] = []
    for m in cfg.test_sizes:
        for elem_c in cfg.elem_counts:
            if elem_c < m:
                continue
            rows = elem_c // m
            print(f"Testing size {m}x{rows}")
            base = torch.randn((rows, m), device="cuda", dtype=torch.float32)
            for dtype in cfg.dtypes:
                buf = base.to(dtype).contiguous()
                dname = str(dtype).replace("torch.", "")
                for name in cfg.benchmark_cases:
                    case = CASES[name]
                    _check_case(name, case, buf)
                    if cfg.check:
                        continue
                    ms, _ = event_window_ms(lambda: case.run(buf), cfg.runs_per_size)
                    gbs = 2 * buf.numel() * buf.element_size() / ms / 1e6
                    print(f"{name} m={m} n={rows} {dname} | {ms:.4f} ms/iter over "
                          f"{cfg.runs_per_size} iters ({gbs:.0f} GB/s)")
                    results.append({"device": device_name, "case": name, "m": m, "n": rows,
                                    "dtype": dname, "runs": cfg.runs_per_size, "per_iter_ms": ms,
                                    "total_ms": ms * cfg.runs_per_size, "GB/s": gbs})
                    buf.copy_(base)  # add-one and repeated transforms drift; start each case alike
                del buf
            del base
    if not cfg.check and cfg.json_output_file:
        with open(cfg.json_output_file, "w") as f:
            json.dump({"device": device_name, "cases": cfg.benchmark_cases,
                       "pytorch": torch.__version__, "results": results}, f, indent=2)
        print(f"Wrote {cfg.json_output_file}")
    return results


# (KDIM, NDIM, MDIM) of fused_ht/benchmark_sweep.py:20-45
FUSED_CONFIGS = [(k, s, s) for k in (256, 512, 1024, 2048, 4096) for s in (1024, 2048, 4096)]


def sweep_metrics(K: int, N: int, M: int, ms: float, esize: int = 4) -> tuple[float, float]:
    """(GFLOP/s, GB/s) of one (K, N, M) shape under the reference's accounting
    (fused_ht/benchmark_sweep.py:123-140): two flops per butterfly output and per multiply-add,
    each of X, W and C moved once."""
    seconds = ms / 1e3
    flops = 2 * K * (K.bit_length() - 1) * N + 2 * M * N * K
    moved = esize * (K * N + M * K + M * N)
    return flops / 1e9 / seconds, moved / 1e9 / seconds


def run_fused(dtype: torch.dtype, runs: int = 8, configs=None, out_prefix: str | None = None):
    rows = []
    g = torch.Generator().manual_seed(123)
    for (K, N, M) in configs or FUSED_CONFIGS:
        W = torch.rand(M, K, generator=g).to(dtype).cuda()      # uniform [0,1) like drand48
        Xt = torch.rand(N, K, generator=g).to(dtype).cuda()
        scale = 1.0 / math.sqrt(K)
        fused = lambda: fused_ht_gemm(W, Xt, scale)
        unfused = lambda: torch.matmul(W, hadamard_transform(Xt, scale).t())
        t_f = best_single_call_ms(fused, runs)
        t_u = best_single_call_ms(unfused, runs)
        diff = (fused().float() - unfused().float()).abs().max().item()
        ref_scale = unfused().float().abs().max().item()
        esize = W.element_size()
        gf, bw = sweep_metrics(K, N, M, t_f, esize)
        gu, _ = sweep_metrics(K, N, M, t_u, esize)
        print(f"K={K:5d} N={N:5d} M={M:5d} {str(dtype).replace('torch.', ''):9s} "
              f"unfused {t_u * 1e3:9.1f} us ({gu / 1e3:7.1f} TFLOP/s)  fused {t_f * 1e3:9.1f} us "
              f"({gf / 1e3:7.1f} TFLOP/s)  speedup {t_u / t_f:5.2f}x  max|diff| {diff:.3e} "
              f"(scale {ref_scale:.3e})")
        rows.append({"kdim": K, "ndim": N, "mdim": M, "dtype": str(dtype).replace("torch.", ""),
                     "baseline_ms": t_u, "fused_ms": t_f, "speedup": t_u / t_f,
                     "fused_gflops": gf, "baseline_gflops": gu, "fused_bandwidth_gbps": bw,
                     "max_error": diff, "max_abs_reference": ref_scale})
        del W, Xt
    if out_prefix:
        with open(out_prefix + ".json", "w") as f:
            json.dump(rows, f, indent=2)
        with open(out_prefix + ".csv", "w", newline="") as f:
            w = csv.DictWriter(f, fieldnames=list(rows[0].keys()) if rows else [])
            w.writeheader()
            w.writerows(rows)
        print(f"Wrote {out_prefix}.json / .csv")
    return rows


# (M, N, B) of fused_ht/fwht_gemv_fusion.cu:643-653
GEMV_CONFIGS = [(256, 256, 512), (512, 512, 1024), (1024, 1024, 2048), (1024, 1024, 256),
                (2048, 2048, 512), (64, 128, 256), (128, 256, 512)]


def gemv_metrics(M: int, N: int, B: int) -> dict[str, float]:
    """The reference's accounting for one fused HT+GEMV shape (fused_ht/fwht_gemv_fusion.cu:576-588):
    N log2 N B butterfly operations plus 2 M N B for the product; the unfused path writes H(X) and
    reads it back, the fused path does not."""
    unfused = 4 * (M * N + 3 * N * B + M * B)
    fused = 4 * (M * N + N * B + M * B)
    return {"flops": N * (N.bit_length() - 1) * B + 2.0 * M * N * B, "bytes_unfused": unfused,
            "bytes_fused": fused, "saved_fraction": (unfused - fused) / unfused}


def run_gemv(configs=None, warmup: int = 10, iters: int = 100, out_prefix: str | None = None):
    """Fused HT+GEMV against the unfused path on the reference's shapes and protocol
    (fused_ht/fwht_gemv_fusion.cu:323-411,521-553: 10 warm-up and 100 timed back-to-back runs, fp32,
    un-normalised transform, uniform [0,1) inputs).  The unfused path is the library's own
    transform down the columns (on an untimed transposed copy of X) followed by the vendor GEMM."""
    rows = []
    g = torch.Generator().manual_seed(42)
    for (M, N, B) in configs or GEMV_CONFIGS:
        W = torch.rand(M, N, generator=g).cuda()
        X = torch.rand(N, B, generator=g).cuda()
        Xcols = X.t().contiguous()
        fused = lambda: fused_ht_gemv(W, X, 1.0)
        unfused = lambda: torch.matmul(W, hadamard_transform(Xcols, 1.0).t())
        # the reference's order (fwht_gemv_fusion.cu:565-568): the unfused path first.  On this chip
        # the order matters: a leg of 100 launches timed right after idle runs at a lower clock than
        # the one behind it (bench.py times both legs past the clock ramp instead)
        t_u, _ = event_window_ms(unfused, iters, warmup)
        t_f, _ = event_window_ms(fused, iters, warmup)
        yu = unfused()
        diff = (fused() - yu).abs().max().item()
        m = gemv_metrics(M, N, B)
        print(f"M={M:5d} N={N:5d} B={B:5d}  unfused {t_u * 1e3:8.1f} us ({m['flops'] / t_u / 1e6:9.1f} GFLOPS)  "
              f"fused {t_f * 1e3:8.1f} us ({m['flops'] / t_f / 1e6:9.1f} GFLOPS)  speedup {t_u / t_f:5.2f}x  "
              f"memory saved {100 * m['saved_fraction']:.1f} %  max|diff| {diff:.3e} (scale {yu.abs().max().item():.3e})")
        rows.append({"M": M, "N": N, "B": B, "unfused_ms": t_u, "fused_ms": t_f, "speedup": t_u / t_f,
                     "fused_gflops": m["flops"] / t_f / 1e6, "unfused_gflops": m["flops"] / t_u / 1e6,
                     "memory_saved_fraction": m["saved_fraction"], "max_error": diff,
                     "max_abs_reference": yu.abs().max().item()})
        del W, X, Xcols
    if out_prefix:
        with open(out_prefix + ".json", "w") as f:
            json.dump(rows, f, indent=2)
        print(f"Wrote {out_prefix}.json")
    return rows


def mfma_probe(shape: int, lds_reads: int, waves_per_simd: int, operands: torch.Tensor,
               steps: int = 4096, repeats: int = 20, warm_ms: float = 30.0) -> dict[str, Any]:
    """One configuration of ``mi_probe_mfma_rate`` (``libmi_probe.so``): nothing but back-to-back bf16 MFMAs on every
    SIMD (plus ``lds_reads`` fragment reads per step), timed past the clock ramp.  ``ghz`` is loop
    cycles (shader clock counter, slowest wavefront) over the event-timed duration of the whole
    launch, so it is a slight underestimate."""
    from . import _lib

    lib = _lib.load_probe()
    stream = torch.cuda.current_stream().cuda_stream
    cycles = torch.zeros(512, dtype=torch.int64, device=operands.device)

    def call():
        _lib.check(lib.mi_probe_mfma_rate(shape, lds_reads, waves_per_simd, steps, operands.data_ptr(),
                                          cycles.data_ptr(), stream), "mfma probe")
    ms, _ = steady_window_ms(call, repeats, warm_ms)
    flops = 256 * 4 * waves_per_simd * steps * 131072
    clk = cycles[:256].double().mean().item()
    return {"mfma": f"{shape}x{shape}x{512 // shape}_bf16", "lds_reads_per_step": lds_reads,
            "waves_per_simd": waves_per_simd, "tflops": flops / ms / 1e9, "ghz": clk / (ms * 1e6),
            "cycles_per_step_per_simd": clk / steps / waves_per_simd, "us_per_launch": ms * 1e3}


def run_mfma_probe(steps: int = 4096, repeats: int = 20) -> list[dict[str, Any]]:
    """Sustained matrix-core rate and shader clock of this chip, with random and with constant
    operands, at 1, 2 and 4 wavefronts per SIMD, with and without LDS fragment reads beside the
    MFMAs.  This is the ceiling the fused GEMM kernels can be read against: the paper peak assumes
    2.4 GHz, the clock under full matrix-core load is lower and depends on the operand data."""
    dev = torch.device("cuda:0")
    patterns = {"random": torch.randn(32768, device=dev).to(torch.bfloat16),
                "constant": torch.full((32768,), 1.0, device=dev, dtype=torch.bfloat16)}
    rows = []
    for pname, ops in patterns.items():
        for shape in (16, 32):
            for reads in (0, 4):
                for wps in (1, 2, 4):
                    row = {"operands": pname, **mfma_probe(shape, reads, wps, ops, steps, repeats)}
                    rows.append(row)
                    print(f"{pname:8s} {row['mfma']:14s} reads/step {reads} waves/SIMD {wps}: "
                          f"{row['tflops']:7.1f} TFLOP/s  {row['ghz']:.2f} GHz  "
                          f"{row['cycles_per_step_per_simd']:.1f} cycles per step per SIMD (128 = issue bound)")
    return rows


ISSUE_KINDS = {"v_add_f32": 0, "v_cvt_pk_bf16_f32": 1, "s_add_u32": 2, "ds_read_b128": 3,
               "v_cvt_pk_fp8_f32": 4, "v_max3_f32": 5, "v_lshlrev_b32": 6}


def run_issue_probe(reps: int = 1000) -> list[dict[str, Any]]:
    """What a SIMD issues per cycle (``mi_probe_issue_rate``): the cost of a group of one MFMA plus n
    other instructions on a lone wavefront (the regime of the register-resident GEMM kernels), and
    the cycles per vector instruction and SIMD at one to four wavefronts per SIMD (the regime of the
    streaming kernels)."""
    from . import _lib

    lib = _lib.load_probe()
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    src = torch.rand(256 * 8, device=dev) + 0.5
    out = torch.zeros(1024, device=dev)
    cycles = torch.zeros(16, dtype=torch.int64, device=dev)
    rows = []

    def run(mode, kind, n, wps):
        for _ in range(2):
            _lib.check(lib.mi_probe_issue_rate(mode, ISSUE_KINDS[kind], n, wps, reps, src.data_ptr(),
                                               out.data_ptr(), cycles.data_ptr(), stream), "issue probe")
        torch.cuda.synchronize()
        return cycles[:4 * wps].max().item()

    for kind in ("v_add_f32", "v_cvt_pk_bf16_f32", "s_add_u32", "ds_read_b128"):
        for n in range(0, 5):
            c = run(0, kind, n, 1) / (8.0 * reps)
            rows.append({"mode": "mfma_plus_n", "kind": kind, "n": n, "cycles_per_group": c})
            print(f"lone wavefront, [1 MFMA 16x16x32 + {n} x {kind}]: {c:6.2f} cycles per group")
    for kind in ("v_add_f32", "v_cvt_pk_bf16_f32", "v_max3_f32", "v_lshlrev_b32", "v_cvt_pk_fp8_f32"):
        for wps in (1, 2, 3, 4):
            c = run(1, kind, 8, wps) / (64.0 * reps * wps)
            rows.append({"mode": "stream", "kind": kind, "waves_per_simd": wps, "cycles_per_instruction_per_simd": c})
            print(f"{wps} wavefront(s) per SIMD, {kind} back to back: {c:5.2f} cycles per instruction per SIMD")
    return rows


def run_stream_probe(bytes_per_wave: int = 256 * 1024, launches: int = 20) -> list[dict[str, Any]]:
    """How fast a compute unit takes data in (``mi_probe_stream_rate``): every compute unit streams
    1 MB (four wavefronts x ``bytes_per_wave``) per launch, through direct global -> LDS transfers or
    ordinary loads, with 4, 8 or 16 KB requested ahead per wavefront, from regions that are read by
    one workgroup (everything comes from beyond the L2), by eight (one reader per XCD: the same) or
    by 32 consecutive ones (four readers per XCD: three of four requests can hit the L2)."""
    from . import _lib

    lib = _lib.load_probe()
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    src = torch.ones(256 * 4 * bytes_per_wave, dtype=torch.uint8, device=dev)
    out = torch.zeros(65536, dtype=torch.int32, device=dev)
    rows = []
    for share in (1, 8, 32):
        for mode, name in ((0, "global_load_lds_dwordx4"), (1, "global_load_dwordx4")):
            for depth in (4, 8, 16):
                def call():
                    _lib.check(lib.mi_probe_stream_rate(mode, depth, share, bytes_per_wave, src.data_ptr(),
                                                        out.data_ptr(), stream), "stream probe")
                for _ in range(3):
                    call()
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                for _ in range(launches):
                    call()
                b.record()
                b.synchronize()
                us = a.elapsed_time(b) * 1e3 / launches
                per_cu = 4 * bytes_per_wave / us * 1e-3
                rows.append({"instruction": name, "kb_ahead_per_wave": depth, "readers_per_region": share,
                             "us_per_launch": us, "gb_per_s_per_cu": per_cu, "tb_per_s_total": per_cu * 256e-3})
                print(f"{name:24s} {depth:2d} KB ahead per wavefront, {share:2d} reader(s) per region: "
                      f"{us:7.2f} us per launch (launch gap included), {per_cu:6.1f} GB/s per compute unit, "
                      f"{per_cu * 256e-3:5.2f} TB/s in all")
    return rows


def _read_power_and_clock() -> dict[str, Any]:
    """Package power (W) and the current shader clock level from the amdgpu sysfs files, which an
    ordinary user may read; empty where the files are absent."""
    import glob

    out: dict[str, Any] = {}
    for path in glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input"):
        try:
            with open(path) as f:
                out["watts"] = int(f.read()) / 1e6
            with open(path.replace("power1_input", "power1_cap")) as f:
                out["cap_watts"] = int(f.read()) / 1e6
        except (OSError, ValueError):
            pass
    for path in glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"):
        try:
            with open(path) as f:
                cur = [line for line in f.read().splitlines() if "*" in line]
            if cur:
                out["sclk_mhz"] = int("".join(ch for ch in cur[0].split(":")[1] if ch.isdigit()))
        except (OSError, ValueError, IndexError):
            pass
    return out


def run_power(seconds: float = 1.5) -> list[dict[str, Any]]:
    """Package power and shader clock while each kernel runs back to back for ``seconds``, next to
    its launch-to-launch time: a matrix-core kernel that sits at the power cap runs at whatever
    clock the cap allows, so its rate is set by the energy a launch needs, not by its cycle count."""
    import threading

    from . import fp8_gemm_rowscale, fused_ht_gemm, rht_quant_fp8

    dev = torch.device("cuda:0")

    def watch(name, fn):
        samples: list[dict[str, Any]] = []
        stop = threading.Event()

        def sampler():
            while not stop.is_set():
                samples.append(_read_power_and_clock())
                time.sleep(0.05)
        th = threading.Thread(target=sampler)
        th.start()
        t0 = time.time()
        while time.time() - t0 < seconds:
            for _ in range(50):
                fn()
            torch.cuda.synchronize()
        stop.set()
        th.join()
        ms, _ = steady_window_ms(fn, 30, 20.0)   # timed after the sampler has stopped
        tail = [x for x in samples[len(samples) // 2:] if "watts" in x]
        row = {"kernel": name, "us_per_launch": ms * 1e3}
        if tail:
            row.update({"watts": sum(x["watts"] for x in tail) / len(tail), "cap_watts": tail[-1].get("cap_watts"),
                        "sclk_mhz": sum(x.get("sclk_mhz", 0) for x in tail) / len(tail)})
        print(f"{name:48s} {row['us_per_launch']:9.2f} us  {row.get('watts', float('nan')):7.0f} W of "
              f"{row.get('cap_watts', float('nan')):.0f}  {row.get('sclk_mhz', float('nan')):6.0f} MHz")
        return row

    rows = [dict(kernel="idle", **_read_power_and_clock())]
    print("idle:", rows[0])
    g = torch.Generator(device=dev).manual_seed(0)
    W = torch.randn(4096, 1024, device=dev, generator=g)
    X = torch.randn(4096, 1024, device=dev, generator=g)
    Wb, Xb = W.to(torch.bfloat16), X.to(torch.bfloat16)
    rows.append(watch("fused HT->GEMM bf16 K=1024 M=N=4096", lambda: fused_ht_gemm(Wb, Xb)))
    rows.append(watch("vendor GEMM bf16 K=1024 M=N=4096 (no transform)", lambda: torch.matmul(Wb, Xb.t())))
    # the same launches on operands that do not toggle the matrix cores' inputs: the instruction
    # stream and the bytes moved are identical, only the energy per MFMA differs
    W1, X1 = torch.ones_like(Wb), torch.ones_like(Xb)
    rows.append(watch("fused HT->GEMM bf16, W constant, X random", lambda: fused_ht_gemm(W1, Xb)))
    rows.append(watch("fused HT->GEMM bf16, W and X constant", lambda: fused_ht_gemm(W1, X1)))
    rows.append(watch("vendor GEMM bf16, W and X constant", lambda: torch.matmul(W1, X1.t())))
    rows.append(watch("fused HT->GEMM fp32 K=1024 M=N=4096", lambda: fused_ht_gemm(W, X)))
    W4 = torch.randn(4096, 4096, device=dev, generator=g).to(torch.bfloat16)
    X4 = torch.randn(4096, 4096, device=dev, generator=g).to(torch.bfloat16)
    rows.append(watch("fused HT->GEMM bf16 K=4096 M=N=4096", lambda: fused_ht_gemm(W4, X4)))
    rows.append(watch("vendor GEMM bf16 K=4096 M=N=4096 (no transform)", lambda: torch.matmul(W4, X4.t())))
    xb = torch.randn(16384, 4096, device=dev, generator=g).to(torch.bfloat16)
    rows.append(watch("FWHT bf16 [16384, 4096] in place", lambda: hadamard_transform(xb, inplace=True)))
    xa = torch.randn(8192, 4096, device=dev, generator=g).to(torch.bfloat16)
    sign = (1 - 2 * torch.randint(0, 2, (4096,))).to(torch.int8).to(dev)
    wq = (torch.randn(14336, 4096, device=dev, generator=g) * 0.02).to(torch.bfloat16)
    qx, sx = rht_quant_fp8(xa, sign)
    qw, sw = rht_quant_fp8(wq, sign)
    rows.append(watch("RHT + FP8 quantize [8192, 4096]", lambda: rht_quant_fp8(xa, sign)))
    rows.append(watch("FP8 GEMM [8192, 4096] x [14336, 4096]^T", lambda: fp8_gemm_rowscale(qx, sx, qw, sw)))
    try:
        rows.append(watch("vendor row-scaled FP8 GEMM, same operands", lambda: torch._scaled_mm(
            qx, qw.t(), scale_a=sx.view(-1, 1), scale_b=sw.view(1, -1), out_dtype=torch.bfloat16)))
    except Exception as ex:  # not every torch build exposes it
        print("vendor row-scaled FP8 GEMM unavailable:", str(ex)[:80])
    return rows


def plot_fused(csv_path: str, out_dir: str = "plots") -> list[str]:
    """Figures and a table from the sweep CSV, the counterpart of the five outputs of
    fused_ht/plot_results.py (speed-up by dimension :23-68, rate / time comparison :72-125, speed-up
    map :129-258, bandwidth :262-304, summary table :308-365): speed-up and TFLOP/s against K for
    every N = M, times of both paths per shape, the speed-up grid over (K, N = M), bandwidth under
    the reference's byte model, and the summary as a Markdown table."""
    import os

    import matplotlib
    matplotlib.use("Agg")
    import matplotlib.pyplot as plt

    with open(csv_path, newline="") as f:
        rows = [{k: (v if k == "dtype" else float(v)) for k, v in r.items()} for r in csv.DictReader(f)]
    os.makedirs(out_dir, exist_ok=True)
    sizes = sorted({int(r["ndim"]) for r in rows})
    kdims = sorted({int(r["kdim"]) for r in rows})
    by_shape = {(int(r["kdim"]), int(r["ndim"])): r for r in rows}
    written = []

    def finish(fig, name):
        path = os.path.join(out_dir, name)
        fig.tight_layout()
        fig.savefig(path, dpi=120)
        plt.close(fig)
        written.append(path)

    # lines against K, one per N = M
    for key, ylabel, name in (("speedup", "fused / unfused speed-up", "speedup_vs_k.png"),
                              ("fused_gflops", "TFLOP/s", "tflops_vs_k.png"),
                              ("fused_bandwidth_gbps", "GB/s of operands and result (fused)",
                               "bandwidth_vs_k.png")):
        fig, ax = plt.subplots(figsize=(7, 4.5))
        for n in sizes:
            sub = sorted((r for r in rows if int(r["ndim"]) == n), key=lambda r: r["kdim"])
            ks = [r["kdim"] for r in sub]
            if key == "fused_gflops":
                ax.plot(ks, [r["fused_gflops"] / 1e3 for r in sub], "o-", label=f"fused N=M={n}")
                ax.plot(ks, [r["baseline_gflops"] / 1e3 for r in sub], "s--", label=f"unfused N=M={n}")
            else:
                ax.plot(ks, [r[key] for r in sub], "o-", label=f"N=M={n}")
        if key == "speedup":
            ax.axhline(1.0, color="gray", linewidth=0.8)
        ax.set_xscale("log", base=2)
        ax.set_xlabel("K")
        ax.set_ylabel(ylabel)
        ax.grid(True, alpha=0.3)
        ax.legend(fontsize=8)
        finish(fig, name)

    # both paths' time per shape, side by side
    fig, ax = plt.subplots(figsize=(max(7, 0.6 * len(rows)), 4.5))
    order = sorted(by_shape)
    pos = range(len(order))
    ax.bar([p - 0.2 for p in pos], [by_shape[s]["baseline_ms"] * 1e3 for s in order], 0.4, label="unfused")
    ax.bar([p + 0.2 for p in pos], [by_shape[s]["fused_ms"] * 1e3 for s in order], 0.4, label="fused")
    ax.set_xticks(list(pos))
    ax.set_xticklabels([f"K={k}\nN=M={n}" for k, n in order], fontsize=7)
    ax.set_ylabel("microseconds per call")
    ax.set_yscale("log")
    ax.legend()
    finish(fig, "time_per_shape.png")

    # speed-up over the (K, N = M) grid
    fig, ax = plt.subplots(figsize=(1.2 * len(kdims) + 2, 0.9 * len(sizes) + 2))
    grid = [[by_shape.get((k, n), {"speedup": float("nan")})["speedup"] for k in kdims] for n in sizes]
    im = ax.imshow(grid, cmap="RdYlGn", vmin=0.25, vmax=2.0, aspect="auto")
    ax.set_xticks(range(len(kdims)))
    ax.set_xticklabels(kdims)
    ax.set_yticks(range(len(sizes)))
    ax.set_yticklabels(sizes)
    ax.set_xlabel("K")
    ax.set_ylabel("N = M")
    for i in range(len(sizes)):
        for j in range(len(kdims)):
            ax.text(j, i, f"{grid[i][j]:.2f}", ha="center", va="center", fontsize=9)
    fig.colorbar(im, ax=ax, label="fused / unfused speed-up")
    finish(fig, "speedup_grid.png")

    # the summary as text
    path = os.path.join(out_dir, "summary.md")
    with open(path, "w") as f:
        f.write("| K | N = M | dtype | unfused us | fused us | speed-up | fused TFLOP/s | max abs diff |\n")
        f.write("|---|---|---|---|---|---|---|---|\n")
        for (k, n) in order:
            r = by_shape[(k, n)]
            f.write(f"| {k} | {n} | {r['dtype']} | {r['baseline_ms'] * 1e3:.1f} | {r['fused_ms'] * 1e3:.1f} | "
                    f"{r['speedup']:.2f} | {r['fused_gflops'] / 1e3:.1f} | {r['max_error']:.3g} |\n")
        wins = [r["speedup"] for r in rows if r["speedup"] >= 1.0]
        f.write(f"\nfused faster on {len(wins)} of {len(rows)} shapes; best {max(r['speedup'] for r in rows):.2f}x, "
                f"worst {min(r['speedup'] for r in rows):.2f}x\n")
    written.append(path)
    return written


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="harness")
    sub = ap.add_subparsers(dest="cmd", required=True)
    p1 = sub.add_parser("fwht")
    p1.add_argument("--check", action="store_true")
    p1.add_argument("--runs-per-size", type=int, default=400)
    p1.add_argument("--json-output-file", default=f"benchmark_{datetime.now():%Y-%m-%d_%H-%M-%S}.json")
    p1.add_argument("--cases", nargs="*", default=list(CASES))
    p1.add_argument("--sizes", nargs="*", type=int, default=[1 << x for x in range(8, 16)])
    p1.add_argument("--elem-counts", nargs="*", type=int, default=[1 << 30])
    p1.add_argument("--dtypes", nargs="*", default=["f16", "bf16"])
    p2 = sub.add_parser("fused")
    p2.add_argument("--dtype", default="bf16", choices=list(DTYPES))
    p2.add_argument("--runs", type=int, default=8)
    p2.add_argument("--out-prefix", default=None)
    p5 = sub.add_parser("gemv")
    p5.add_argument("--iters", type=int, default=100)
    p5.add_argument("--out-prefix", default=None)
    p4 = sub.add_parser("mfma")
    p4.add_argument("--steps", type=int, default=4096)
    sub.add_parser("issue")
    sub.add_parser("stream")
    p6 = sub.add_parser("power")
    p6.add_argument("--seconds", type=float, default=1.5)
    p3 = sub.add_parser("plot")
    p3.add_argument("csv")
    p3.add_argument("--out-dir", default="plots")
    args = ap.parse_args(argv)
    if args.cmd == "plot":
        for path in plot_fused(args.csv, args.out_dir):
            print("wrote", path)
        return 0
    if not torch.cuda.is_available():
        sys.stderr.write("harness: no GPU visible\n")
        return 2
    if args.cmd == "mfma":
        run_mfma_probe(args.steps)
        return 0
    if args.cmd == "issue":
        run_issue_probe()
        return 0
    if args.cmd == "stream":
        run_stream_probe()
        return 0
    if args.cmd == "power":
        run_power(args.seconds)
        return 0
    if args.cmd == "gemv":
        run_gemv(iters=args.iters, out_prefix=args.out_prefix)
        return 0
    if args.cmd == "fwht":
        run_fwht(TestConfig(check=args.check, runs_per_size=args.runs_per_size,
                            json_output_file=args.json_output_file, benchmark_cases=args.cases,
                            test_sizes=args.sizes, elem_counts=args.elem_counts,
                            dtypes=tuple(DTYPES[d] for d in args.dtypes)))
    else:
        run_fused(DTYPES[args.dtype], args.runs, out_prefix=args.out_prefix)
    return 0


if __name__ == "__main__":
    sys.exit(main())
