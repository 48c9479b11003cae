"""Writes tests/golden/hadamard_fixtures.npz: small input/expected-output vectors computed
WITHOUT the oracle (scipy's Sylvester matrix, numpy matmul in fp64, torch's CPU float8 cast), so
that they pin the oracle and the kernels from an independent side.  The reference repository
stores no golden vectors of its own (its checks are computed on the fly, HadaCore/test.py:71-97);
these follow its truth path  x @ (scipy.linalg.hadamard(n) * n**-0.5).

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import math
import os

import numpy as np
import scipy.linalg
import torch

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hadamard_fixtures.npz")


def main():
    rng = np.random.default_rng(20251)
    d = {}
    # transform: x @ H / sqrt(n), fp64, for a few sizes (inputs are bf16-representable so the same
    # vectors serve every dtype)
    for n in (2, 16, 256, 1024):
        x = torch.from_numpy(rng.standard_normal((3, n)).astype(np.float32)).to(torch.bfloat16)
        x = x.to(torch.float64).numpy()
        H = scipy.linalg.hadamard(n).astype(np.float64)
        d[f"fwht_x_{n}"] = x
        d[f"fwht_y_{n}"] = x @ H / math.sqrt(n)
    # fused HT+GEMV at the reference's first correctness shape (M=32, N=64, B=8), unnormalised
    M, N, B = 32, 64, 8
    W = torch.from_numpy(rng.uniform(-1, 1, (M, N)).astype(np.float32)).to(torch.float64).numpy()
    X = torch.from_numpy(rng.uniform(-1, 1, (N, B)).astype(np.float32)).to(torch.float64).numpy()
    d["gemv_W"], d["gemv_X"] = W, X
    d["gemv_Y"] = W @ (scipy.linalg.hadamard(N).astype(np.float64) @ X)
    # fused HT->GEMM, small: C = W @ (H @ Xt.T), unnormalised; bf16-representable inputs
    M, N, K = 24, 20, 64
    W = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.bfloat16).to(torch.float64).numpy()
    Xt = torch.from_numpy(rng.standard_normal((N, K)).astype(np.float32)).to(torch.bfloat16).to(torch.float64).numpy()
    d["gemm_W"], d["gemm_Xt"] = W, Xt
    d["gemm_C"] = W @ (scipy.linalg.hadamard(K).astype(np.float64) @ Xt.T)
    # FP8 E4M3FN codes of a dense value set via torch's CPU cast (RNE), |x| <= 448
    vals = np.concatenate([
        np.linspace(-448, 448, 1793), 2.0 ** np.arange(-12, 9), -(2.0 ** np.arange(-12, 9)),
        np.array([0.0, 17.0, 19.0, 0.0009765625, 0.00146484375, 447.9, 463.9 - 16])]).astype(np.float32)
    d["fp8_values"] = vals
    d["fp8_codes"] = torch.from_numpy(vals).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    # per-row amax quantizer on a small matrix, by numpy + torch cast, under the stated convention
    y = torch.from_numpy(rng.standard_normal((5, 32)).astype(np.float32)).to(torch.bfloat16).to(torch.float32).numpy()
    y[1] = 0
    amax = np.maximum(np.abs(y).max(axis=1), np.float32(1e-30)).astype(np.float32)
    inv = (np.float32(448.0) / amax).astype(np.float32)
    t = np.clip((y * inv[:, None]).astype(np.float32), -448, 448)
    d["quant_y"] = y
    d["quant_scale"] = (amax / np.float32(448.0)).astype(np.float32)
    d["quant_codes"] = torch.from_numpy(t).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    np.savez_compressed(OUT, **d)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
