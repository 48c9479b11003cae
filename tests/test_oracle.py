"""Pins the CPU oracle against things other than its own formulas: scipy's Sylvester matrix,
algebraic invariants, brute force, and torch-CPU conversions.  The reference holds no stored
golden vectors (its checks are computed on the fly, HadaCore/test.py:71-97), so these are the
known answers."""
import math

import numpy as np
import pytest
import scipy.linalg
import torch

SIZES = [1 << p for p in range(0, 16)]


def test_sylvester_equals_scipy(oracle):
    for n in [1, 2, 4, 8, 16, 64, 256, 1024]:
        assert np.array_equal(oracle.sylvester(n), scipy.linalg.hadamard(n).astype(np.int8))


def test_sylvester_kronecker_and_orthogonality(oracle):
    H2 = np.array([[1, 1], [1, -1]], dtype=np.int64)
    for n in [2, 4, 8, 32, 128]:
        H = oracle.sylvester(n).astype(np.int64)
        assert np.array_equal(H @ H, n * np.eye(n, dtype=np.int64))
        assert np.array_equal(oracle.sylvester(2 * n).astype(np.int64), np.kron(H2, H))
        assert np.array_equal(H, H.T)


@pytest.mark.parametrize("n", [1, 2, 4, 16, 64, 256, 1024, 4096])
def test_butterfly_equals_matrix(oracle, n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal((5, n))
    y_bf = oracle.fwht_f64(x)
    y_mat = x @ (scipy.linalg.hadamard(n).astype(np.float64) / math.sqrt(n))
    assert np.max(np.abs(y_bf - y_mat)) < 1e-12 * max(1.0, np.max(np.abs(y_mat)))
    y_c = oracle.fwht_matrix_f64(x)
    assert np.max(np.abs(y_c - y_mat)) < 1e-12 * max(1.0, np.max(np.abs(y_mat)))


@pytest.mark.parametrize("n", [8192, 16384, 32768])
def test_butterfly_large_sizes_bruteforce_rows(oracle, n):
    # two rows by brute force in C (O(n^2) each), all columns
    rng = np.random.default_rng(n)
    x = rng.standard_normal((2, n))
    assert np.allclose(oracle.fwht_f64(x), oracle.fwht_matrix_f64(x), rtol=0, atol=1e-10)


@pytest.mark.parametrize("n", SIZES)
def test_invariants(oracle, n):
    rng = np.random.default_rng(7 + n)
    x = rng.standard_normal((3, n))
    y = oracle.fwht_f64(x)
    # involution and Parseval of the normalised transform
    assert np.allclose(oracle.fwht_f64(y), x, atol=1e-10)
    assert np.allclose(np.linalg.norm(y, axis=1), np.linalg.norm(x, axis=1), rtol=1e-12)
    # unit vector -> row k of H ; constant vector -> n * e_0  (unnormalised)
    k = n // 3
    e = np.zeros((1, n)); e[0, k] = 1.0
    row = oracle.fwht_f64(e, scale=1.0)[0]
    expect = np.array([(-1) ** bin(k & j).count("1") for j in range(n)], dtype=np.float64)
    assert np.array_equal(row, expect)
    ones = oracle.fwht_f64(np.ones((1, n)), scale=1.0)[0]
    assert ones[0] == n and np.all(ones[1:] == 0)
    # linearity
    a, b = x[0:1], x[1:2]
    assert np.allclose(oracle.fwht_f64(2 * a - 3 * b), 2 * oracle.fwht_f64(a) - 3 * oracle.fwht_f64(b),
                       atol=1e-10)


def test_fp32_port_close_to_fp64(oracle):
    x = oracle.inputs_fwht(512, 256, torch.float32).numpy()
    y32 = oracle.fwht_f32(x)
    y64 = oracle.fwht_f64(x)
    assert oracle.rel_err(y32, y64) < 1e-6


def test_matrix_truth_path_config1(oracle):
    # benchmark configuration 1: fp32 [512,256], scale 1/16, x @ H in torch on the CPU
    x = oracle.inputs_fwht(512, 256, torch.float32)
    y = oracle.hadamard_matrix_ref(x).numpy()
    assert oracle.rel_err(y, oracle.fwht_f64(x.numpy())) < 1e-5


def test_fused_gemv_layouts(oracle):
    rng = np.random.default_rng(0)
    for (M, N, B) in [(32, 64, 8), (64, 128, 16), (5, 16, 3)]:
        W = rng.standard_normal((M, N)); X = rng.standard_normal((N, B))
        H = scipy.linalg.hadamard(N).astype(np.float64)
        for s in (1.0, 1 / math.sqrt(N)):
            ref = W @ (s * H @ X)
            assert np.allclose(oracle.fused_ht_gemv_f64(W, X, s), ref, atol=1e-9)
            assert np.allclose(oracle.fused_ht_gemv_f64_blas(W, X, s), ref, atol=1e-9)
    # W = I reduces to the column transform
    N, B = 64, 5
    X = rng.standard_normal((N, B))
    assert np.allclose(oracle.fused_ht_gemv_f64(np.eye(N), X, 1.0), oracle.fwht_f64(X.T, 1.0).T)


def test_fused_gemm_layouts(oracle):
    rng = np.random.default_rng(1)
    for (M, N, K) in [(8, 12, 16), (33, 7, 64), (16, 16, 256)]:
        W = rng.standard_normal((M, K)); Xt = rng.standard_normal((N, K))
        H = scipy.linalg.hadamard(K).astype(np.float64)
        for s in (1.0, 1 / math.sqrt(K)):
            ref = W @ (s * H @ Xt.T)
            assert np.allclose(oracle.fused_ht_gemm_f64(W, Xt, s), ref, atol=1e-9)
            assert np.allclose(oracle.fused_ht_gemm_f64_blas(W, Xt, s), ref, atol=1e-9)
    K, N = 32, 6
    Xt = rng.standard_normal((N, K))
    # W = I: C = H X  ->  C.T = rows of Xt transformed
    assert np.allclose(oracle.fused_ht_gemm_f64(np.eye(K), Xt, 1.0).T, oracle.fwht_f64(Xt, 1.0))
    # scale 1 vs K^-1/2 differ by an exact power of two when K is an even power
    K = 256
    W = rng.standard_normal((4, K)); Xt = rng.standard_normal((3, K))
    assert np.array_equal(oracle.fused_ht_gemm_f64(W, Xt, 1.0) / 16.0,
                          oracle.fused_ht_gemm_f64(W, Xt, 1.0 / 16.0))


def _dense_f32_sweep():
    # every bf16-representable pattern extended with a few low-bit patterns that exercise
    # round-up, round-down and ties
    hi = np.arange(0, 1 << 16, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x1000, 0x2000, 0x3000,
                     0x0FFF, 0x1001, 0xEFFF, 0xF000], dtype=np.uint32)
    bits = (hi[:, None] | lows[None, :]).reshape(-1)
    return bits.view(np.float32)


def test_rne_bf16_matches_torch(oracle):
    x = _dense_f32_sweep()
    got = oracle.f32_to_bf16(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(oracle.bf16_to_f32(got[nan])))


def test_rne_f16_matches_torch(oracle):
    x = _dense_f32_sweep()
    got = oracle.f32_to_f16(x)
    want = torch.from_numpy(x.copy()).to(torch.float16).view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(oracle.f16_to_f32(got[nan])))
    # decode is the exact inverse on all 65536 codes
    codes = np.arange(0, 1 << 16, dtype=np.uint16)
    dec = oracle.f16_to_f32(codes)
    want_dec = torch.from_numpy(codes.view(np.int16).copy()).view(torch.float16).to(torch.float32).numpy()
    ok = ~np.isnan(want_dec)
    assert np.array_equal(dec[ok], want_dec[ok])


def test_rne_converter_reference_points(oracle):
    # the 41 points of test/test_bit.py:18-22, at its tolerance of 0.02
    pts = [0.0] + [2.0 ** (-i / 4) for i in range(-10, 10)] + [-(2.0 ** (-i / 2)) for i in range(-10, 10)]
    x = np.array(pts, dtype=np.float32)
    assert np.all(np.abs(oracle.bf16_to_f32(oracle.f32_to_bf16(x)) - x) <= 0.02 * np.maximum(1, np.abs(x)))
    assert np.all(np.abs(oracle.f16_to_f32(oracle.f32_to_f16(x)) - x) <= 0.02)


def test_e4m3fn_matches_torch_and_format(oracle):
    x = _dense_f32_sweep()
    x = x[np.isfinite(x) & (np.abs(x) <= 448.0)]
    got = oracle.e4m3fn_encode(x)
    want = torch.from_numpy(x.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    # torch keeps the sign of values that round to zero; so does the oracle
    assert np.array_equal(got, want)
    # format definition: all 256 codes decode per OCP E4M3FN and re-encode to themselves
    codes = np.arange(256, dtype=np.uint8)
    dec = oracle.e4m3fn_decode(codes)
    want_dec = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    ok = ~np.isnan(want_dec)
    assert np.array_equal(dec[ok], want_dec[ok])
    assert np.isnan(dec[0x7F]) and np.isnan(dec[0xFF])
    assert dec[0x7E] == 448.0 and dec[0x01] == 2.0 ** -9 and dec[0x08] == 2.0 ** -6
    assert np.array_equal(oracle.e4m3fn_encode(dec[ok]), codes[ok])
    # ties to even between neighbours, saturation above 448
    assert oracle.e4m3fn_encode(np.array([17.0, 19.0, 464.0, 1e9, -1e9], dtype=np.float32)).tolist() == [
        0x58, 0x5A, 0x7E, 0x7E, 0xFE]


def test_quant_rows_against_numpy(oracle):
    rng = np.random.default_rng(3)
    y = rng.standard_normal((7, 64)).astype(np.float32)
    y[2] = 0.0                      # all-zero row
    y[3, 5] = 1000.0                # outlier
    q, s = oracle.quant_fp8_rows(y)
    amax = np.maximum(np.max(np.abs(y), axis=1), np.float32(1e-30)).astype(np.float32)
    assert np.array_equal(s, (amax / np.float32(448.0)).astype(np.float32))
    inv = (np.float32(448.0) / amax).astype(np.float32)
    t = np.clip((y * inv[:, None]).astype(np.float32), -448.0, 448.0)
    want = torch.from_numpy(t).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(q, want)
    assert np.all(q[2] == 0)
    assert q[3, 5] == 0x7E
    # dequantised values are close to y
    deq = oracle.e4m3fn_decode(q) * s[:, None]
    assert np.max(np.abs(deq - y)[[0, 1, 4, 5, 6]]) < 0.07 * np.max(np.abs(y[[0, 1, 4, 5, 6]]))


def test_rht_is_transform_of_signed_input(oracle):
    x, sign = oracle.inputs_rht(16, 256)
    xf = x.to(torch.float32).numpy()
    y = oracle.rht_f64(xf, sign.numpy())
    assert np.allclose(y, oracle.fwht_f64(xf.astype(np.float64) * sign.numpy()[None, :].astype(np.float64)))
    assert set(np.unique(sign.numpy()).tolist()) <= {-1, 1}


def test_seeded_inputs_reproducible(oracle):
    a = oracle.inputs_fwht(4, 16, torch.bfloat16)
    b = oracle.inputs_fwht(4, 16, torch.bfloat16)
    assert torch.equal(a, b)
    W1, X1 = oracle.inputs_gemm(8, 4, 16, torch.float32)
    W2, X2 = oracle.inputs_gemm(8, 4, 16, torch.float32)
    assert torch.equal(W1, W2) and torch.equal(X1, X2)
