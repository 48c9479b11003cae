"""Seeded random shapes (ragged row counts, odd batch sizes, every supported transform length)
for each entry point against the fp64 oracle: the fixed-shape tests pick edge cases by hand, this
file walks the space between them.  Tolerances as everywhere: fp32 <= 1e-5, 16-bit <= 2e-2 on
max|y - y64| / max|y64|; FP8 codes and scales bit-exact given the device's own pre-quant values."""
import math
import random

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _rel(oracle, got, want64):
    return oracle.rel_err(got.cpu().to(torch.float64).numpy(), want64)


def test_fwht_random_shapes(pkg, oracle):
    rnd = random.Random(101)
    for case in range(40):
        p = rnd.randint(0, 15)
        n = 1 << p
        rows = rnd.randint(1, max(1, min(3000, (1 << 21) // n)))
        dt = rnd.choice(DTYPES)
        scale = rnd.choice([None, 1.0, 0.37])
        x = oracle.inputs_fwht(rows, n, dt)
        y = pkg.hadamard_transform(x.cuda(), scale)
        want = oracle.fwht_f64(x.to(torch.float64).numpy(), scale)
        assert _rel(oracle, y, want) <= TOL[dt], (case, rows, n, dt, scale)


def test_gemv_random_shapes(pkg, oracle):
    rnd = random.Random(102)
    for case in range(25):
        N = 1 << rnd.randint(1, 11)
        M = rnd.randint(1, 700)
        B = rnd.randint(1, 300)
        W, X = oracle.inputs_gemv(M, N, B)
        s = rnd.choice([1.0, 1.0 / math.sqrt(N)])
        Y = pkg.fused_ht_gemv(W.cuda(), X.cuda(), s)
        want = oracle.fused_ht_gemv_f64_blas(W.double().numpy(), X.double().numpy(), s)
        assert _rel(oracle, Y, want) <= 1e-5, (case, M, N, B)


def test_gemm_random_shapes(pkg, oracle):
    rnd = random.Random(103)
    for case in range(30):
        dt = rnd.choice(DTYPES)
        K = 1 << rnd.randint(5, 12)
        M = rnd.randint(1, 600)
        N = rnd.randint(1, 400)
        W, Xt = oracle.inputs_gemm(M, N, K, dt)
        s = 1.0 / math.sqrt(K)
        C = pkg.fused_ht_gemm(W.cuda(), Xt.cuda(), s)
        want = oracle.fused_ht_gemm_f64_blas(W.double().numpy(), Xt.double().numpy(), s)
        assert C.shape == (M, N)
        assert _rel(oracle, C, want) <= TOL[dt], (case, M, N, K, dt)


def test_rht_quant_random_shapes(pkg, oracle):
    rnd = random.Random(104)
    for case in range(20):
        n = 1 << rnd.randint(4, 12)
        T = rnd.randint(1, max(1, min(2000, (1 << 20) // n)))
        x, sign = oracle.inputs_rht(T, n)
        q, rs, y = pkg.rht_quant_fp8(x.cuda(), sign, return_prequant=True)
        torch.cuda.synchronize()
        y32 = y.float().cpu().numpy()
        want_q, want_s = oracle.quant_fp8_rows(y32)
        assert np.array_equal(q.view(torch.uint8).cpu().numpy(), want_q), (case, T, n)
        assert np.array_equal(rs.cpu().numpy(), want_s), (case, T, n)
        y64 = oracle.rht_f64(x.to(torch.float32).numpy(), sign.numpy())
        assert oracle.rel_err(y32.astype(np.float64), y64) <= 2e-2, (case, T, n)


def test_fp8_gemm_random_shapes(pkg, oracle):
    rnd = random.Random(105)
    for case in range(12):
        K = 128 * rnd.randint(1, 9)
        T = rnd.randint(1, 700)
        N = rnd.randint(1, 700)
        g = torch.Generator().manual_seed(1000 + case)
        a = torch.randn(T, K, generator=g)
        b = torch.randn(N, K, generator=g) * 0.02
        qa, sa = oracle.quant_fp8_rows(a.numpy())
        qb, sb = oracle.quant_fp8_rows(b.numpy())
        out = pkg.fp8_gemm_rowscale(torch.from_numpy(qa).cuda().view(torch.float8_e4m3fn),
                                    torch.from_numpy(sa).cuda(),
                                    torch.from_numpy(qb).cuda().view(torch.float8_e4m3fn),
                                    torch.from_numpy(sb).cuda())
        da = oracle.e4m3fn_decode(qa).astype(np.float64) * sa[:, None].astype(np.float64)
        db = oracle.e4m3fn_decode(qb).astype(np.float64) * sb[:, None].astype(np.float64)
        assert oracle.rel_err(out.cpu().double().numpy(), da @ db.T) <= 2e-2, (case, T, N, K)
