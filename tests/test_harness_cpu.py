"""Host logic of the benchmark harness (no GPU): the shape list and the FLOP/byte model match the
reference's sweep (fused_ht/benchmark_sweep.py:20-45,123-140), and the case registry and
tolerances match its benchmark (bench/bench.py:96-103,177)."""
import importlib

import pytest
import torch


@pytest.fixture(scope="module")
def harness(pkg):
    return importlib.import_module(pkg.__name__ + ".harness")


def test_fused_shape_list(harness):
    cfgs = harness.FUSED_CONFIGS
    assert len(cfgs) == 15 and len(set(cfgs)) == 15
    assert cfgs[0] == (256, 1024, 1024) and cfgs[8] == (1024, 4096, 4096) and cfgs[-1] == (4096, 4096, 4096)
    assert all(n == m for _, n, m in cfgs)
    assert [k for k, _, _ in cfgs] == sorted(k for k, _, _ in cfgs)


def test_sweep_metrics_known_values(harness):
    # K=1024, N=M=4096, 1 ms: transform 1024*10*4096*2 flops + GEMM 2*4096*4096*1024 flops;
    # bytes (K*N + M*K + M*N) * 4.  Numbers written out by hand, not recomputed from the formula.
    gflops, gbps = harness.sweep_metrics(1024, 4096, 4096, 1.0)
    assert gflops == pytest.approx((83_886_080 + 34_359_738_368) / 1e9 / 1e-3)
    assert gbps == pytest.approx(100_663_296 / 1e9 / 1e-3)
    # halving the time doubles both; 2-byte elements halve the bytes only
    g2, b2 = harness.sweep_metrics(1024, 4096, 4096, 0.5, esize=2)
    assert g2 == pytest.approx(2 * gflops) and b2 == pytest.approx(gbps)


def test_gemv_shapes_and_metrics(harness):
    # the seven shapes of fused_ht/fwht_gemv_fusion.cu:643-653 and its accounting (:576-588)
    assert harness.GEMV_CONFIGS == [(256, 256, 512), (512, 512, 1024), (1024, 1024, 2048),
                                    (1024, 1024, 256), (2048, 2048, 512), (64, 128, 256), (128, 256, 512)]
    m = harness.gemv_metrics(256, 256, 512)
    assert m["flops"] == 256 * 8 * 512 + 2 * 256 * 256 * 512
    assert m["bytes_fused"] == 4 * (256 * 256 + 256 * 512 + 256 * 512)
    assert m["bytes_unfused"] - m["bytes_fused"] == 4 * 2 * 256 * 512   # H(X) written and read back
    assert abs(m["saved_fraction"] - 2 * 256 * 512 / (256 * 256 + 3 * 256 * 512 + 256 * 512)) < 1e-12


def test_case_registry_and_tolerances(harness):
    assert list(harness.CASES) == ["AddOne1", "AddOne2", "Ours", "AddOne3"]
    assert harness.ATOL[torch.float16] == 1e-2 and harness.ATOL[torch.bfloat16] == 5e-2
    cfg = harness.TestConfig()
    assert cfg.runs_per_size == 400
    assert cfg.test_sizes == [256, 512, 1024, 2048, 4096, 8192, 16384, 32768]
    assert cfg.elem_counts == [1 << 30]
    t = torch.zeros(4, 8)
    assert torch.equal(harness.CASES["AddOne1"].truth(t), torch.ones(4, 8))
    harness.CASES["AddOne1"].run(t)
    assert torch.equal(t, torch.ones(4, 8))


def test_cli_without_gpu_exits_nonzero(harness):
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    assert harness.main(["fwht", "--check"]) == 2


def test_plot_from_sweep_csv(harness, tmp_path):
    import csv
    rows = []
    for k in (256, 1024, 4096):
        for n in (1024, 4096):
            rows.append({"kdim": k, "ndim": n, "mdim": n, "dtype": "bfloat16", "baseline_ms": 0.05,
                         "fused_ms": 0.04, "speedup": 1.25, "fused_gflops": 5e5, "baseline_gflops": 4e5,
                         "fused_bandwidth_gbps": 100.0, "max_error": 0.1, "max_abs_reference": 30.0})
    path = tmp_path / "s.csv"
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=list(rows[0]))
        w.writeheader()
        w.writerows(rows)
    out = harness.plot_fused(str(path), str(tmp_path / "plots"))
    names = sorted(p.split("/")[-1] for p in out)
    assert names == sorted(["bandwidth_vs_k.png", "speedup_grid.png", "speedup_vs_k.png", "summary.md",
                            "time_per_shape.png", "tflops_vs_k.png"])
    for p in out:
        assert (tmp_path / "plots" / p.split("/")[-1]).stat().st_size > (1000 if p.endswith(".png") else 300)
    text = (tmp_path / "plots" / "summary.md").read_text()
    assert "| 1024 | 4096 | bfloat16 | 50.0 | 40.0 | 1.25 | 500.0 |" in text and "fused faster on 6 of 6 shapes" in text
    assert harness.main(["plot", str(path), "--out-dir", str(tmp_path / "p2")]) == 0
