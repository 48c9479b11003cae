"""The harness end to end on the GPU at small sizes: --check passes for every case and dtype, the
timed run writes the reference's JSON fields (bench/bench.py:226-237,291-300), and the fused sweep
reports fused vs. unfused within the 16-bit tolerance."""
import importlib
import json

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def harness(pkg):
    return importlib.import_module(pkg.__name__ + ".harness")


def test_check_mode_all_cases(harness):
    cfg = harness.TestConfig(check=True, test_sizes=[256, 2048, 32768], elem_counts=[1 << 20])
    assert harness.run_fwht(cfg) == []


def test_check_mode_detects_a_wrong_case(harness):
    harness.CASES["Wrong"] = harness.Case(run=lambda t: t.add_(1), truth=lambda t: t + 2)
    try:
        with pytest.raises(SystemExit):
            harness.run_fwht(harness.TestConfig(check=True, benchmark_cases=["Wrong"],
                                                test_sizes=[256], elem_counts=[1 << 16]))
    finally:
        del harness.CASES["Wrong"]


def test_check_mode_runs_the_full_size_buffer(harness, pkg, monkeypatch):
    # the transform must be called on the whole buffer (the launch path that is timed is chosen by
    # tensor size), not on a cloned slice
    seen = []
    real = harness.hadamard_transform

    def spy(t, *a, **k):
        seen.append(tuple(t.shape))
        return real(t, *a, **k)

    monkeypatch.setattr(harness, "hadamard_transform", spy)
    monkeypatch.setitem(harness.CASES, "Ours",
                        harness.Case(run=lambda t: spy(t, inplace=True), truth=harness.CASES["Ours"].truth))
    cfg = harness.TestConfig(check=True, benchmark_cases=["Ours"], test_sizes=[8192],
                             elem_counts=[1 << 24], dtypes=(torch.bfloat16,))
    assert harness.run_fwht(cfg) == []
    assert seen == [(2048, 8192)]


def test_timed_run_json(harness, tmp_path):
    out = tmp_path / "b.json"
    cfg = harness.TestConfig(runs_per_size=5, json_output_file=str(out), test_sizes=[1024],
                             elem_counts=[1 << 20])
    res = harness.run_fwht(cfg)
    assert len(res) == 4 * 2
    payload = json.loads(out.read_text())
    assert set(payload) == {"device", "cases", "pytorch", "results"}
    for r in payload["results"]:
        assert {"device", "case", "m", "n", "dtype", "runs", "per_iter_ms", "total_ms"} <= set(r)
        assert r["m"] == 1024 and r["n"] == 1024 and r["runs"] == 5 and r["per_iter_ms"] > 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fused_sweep_small(harness, dtype, tmp_path):
    rows = harness.run_fused(dtype, runs=2, configs=[(256, 128, 192), (1024, 256, 256)],
                             out_prefix=str(tmp_path / "s"))
    assert len(rows) == 2
    for r in rows:
        tol = 2e-2 if dtype == torch.bfloat16 else 1e-4
        assert r["max_error"] <= tol * r["max_abs_reference"]
        assert r["fused_ms"] > 0 and r["baseline_ms"] > 0
    assert json.loads((tmp_path / "s.json").read_text())[0]["kdim"] == 256
    assert (tmp_path / "s.csv").read_text().startswith("kdim,ndim,mdim")


def test_gemv_table_small(harness, tmp_path):
    rows = harness.run_gemv(configs=[(64, 128, 256), (256, 256, 512)], warmup=2, iters=5,
                            out_prefix=str(tmp_path / "gemv"))
    assert len(rows) == 2 and (tmp_path / "gemv.json").exists()
    for r in rows:
        # the reference's own bar between its fused and unfused results (fwht_gemv_fusion.cu:293)
        assert r["max_error"] <= 1e-3 * max(1.0, r["max_abs_reference"])
        assert r["fused_ms"] > 0 and r["unfused_ms"] > 0


def test_mfma_probe_structure(harness):
    # structural properties only (rates and clocks depend on the box's power state and belong in the
    # benchmark output): every configuration reports, values are finite and positive, and a step
    # never takes fewer cycles than the 128 its eight MFMAs occupy the matrix-core pipeline
    import math
    rows = harness.run_mfma_probe(steps=1024, repeats=5)
    assert len(rows) == 2 * 2 * 2 * 3
    for r in rows:
        for key in ("tflops", "ghz", "cycles_per_step_per_simd", "us_per_launch"):
            assert math.isfinite(r[key]) and r[key] > 0.0, r
        assert r["cycles_per_step_per_simd"] > 125.0, r


def test_stream_probe_structure(harness):
    # structural properties only: every configuration reports a positive finite rate, and readers
    # that share a region inside an XCD are not slower than readers that share nothing
    import math
    rows = harness.run_stream_probe(bytes_per_wave=64 * 1024, launches=5)
    assert len(rows) == 3 * 2 * 3
    for r in rows:
        assert math.isfinite(r["gb_per_s_per_cu"]) and r["gb_per_s_per_cu"] > 0.0, r
    best = lambda share: max(r["gb_per_s_per_cu"] for r in rows if r["readers_per_region"] == share)
    assert best(32) >= 0.9 * best(1)
