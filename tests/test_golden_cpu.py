"""The CPU oracle against the committed fixtures (tests/golden/hadamard_fixtures.npz, built by
tests/golden/make_fixtures.py from scipy / numpy / torch-CPU only)."""
import os

import numpy as np
import pytest

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hadamard_fixtures.npz")


@pytest.fixture(scope="module")
def fix():
    return np.load(FIX, allow_pickle=False)


def test_fwht_fixture(oracle, fix):
    for n in (2, 16, 256, 1024):
        y = oracle.fwht_f64(fix[f"fwht_x_{n}"])
        assert np.allclose(y, fix[f"fwht_y_{n}"], rtol=0, atol=1e-12)


def test_fused_fixtures(oracle, fix):
    assert np.allclose(oracle.fused_ht_gemv_f64(fix["gemv_W"], fix["gemv_X"], 1.0), fix["gemv_Y"], atol=1e-11)
    assert np.allclose(oracle.fused_ht_gemm_f64(fix["gemm_W"], fix["gemm_Xt"], 1.0), fix["gemm_C"], atol=1e-10)


def test_fp8_fixtures(oracle, fix):
    assert np.array_equal(oracle.e4m3fn_encode(fix["fp8_values"]), fix["fp8_codes"])
    q, s = oracle.quant_fp8_rows(fix["quant_y"])
    assert np.array_equal(q, fix["quant_codes"])
    assert np.array_equal(s, fix["quant_scale"])
