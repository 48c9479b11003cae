"""ctypes front end of ``liboracle.so`` plus the reference's matrix truth path.

TEST INFRASTRUCTURE ONLY: see the package docstring for who may import this.
"""
from __future__ import annotations

import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

__all__ = [
    "build", "lib", "sylvester", "fwht_f64", "fwht_f32", "fwht_matrix_f64", "hadamard_matrix_ref",
    "fused_ht_gemv_f64", "fused_ht_gemm_f64", "fused_ht_gemv_f64_blas", "fused_ht_gemm_f64_blas",
    "f32_to_bf16", "bf16_to_f32", "f32_to_f16", "f16_to_f32", "e4m3fn_encode", "e4m3fn_decode",
    "quant_fp8_rows", "rht_f64", "rel_err", "default_scale",
    "inputs_fwht", "inputs_gemv", "inputs_gemm", "inputs_rht",
]


def build(force: bool = False) -> str:
    """Compile ``liboracle.so`` with the Makefile beside this file."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "hadamard_oracle.c"))
    ):
        subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, u64, u32, f64, f32 = (ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint32,
                                  ctypes.c_double, ctypes.c_float)
        L.oracle_sylvester.argtypes = [u32, vp]
        L.oracle_fwht_f64.argtypes = [vp, u64, u32, f64]
        L.oracle_fwht_f32.argtypes = [vp, u64, u32, f32]
        L.oracle_fwht_matrix_f64.argtypes = [vp, vp, u64, u32, f64]
        L.oracle_fused_ht_gemv_f64.argtypes = [vp, vp, vp, u32, u32, u32, f64]
        L.oracle_fused_ht_gemm_f64.argtypes = [vp, vp, vp, u32, u32, u32, f64]
        for name in ("oracle_f32_to_bf16_array", "oracle_f32_to_f16_array",
                     "oracle_f16_to_f32_array", "oracle_e4m3fn_encode_array",
                     "oracle_e4m3fn_decode_array"):
            getattr(L, name).argtypes = [vp, vp, u64]
        L.oracle_quant_fp8_rows.argtypes = [vp, vp, vp, u64, u32]
        L.oracle_rht_f64.argtypes = [vp, vp, vp, u64, u32, f64]
        _lib = L
    return _lib


def _p(a: np.ndarray) -> ctypes.c_void_p:
    return ctypes.c_void_p(a.ctypes.data)


def default_scale(n: int) -> float:
    """n**-0.5, the only scale the reference op applies (HadaCore/test.py:24-25)."""
    return 1.0 / math.sqrt(n)


def sylvester(n: int) -> np.ndarray:
    H = np.empty((n, n), dtype=np.int8)
    lib().oracle_sylvester(n, _p(H))
    return H


def fwht_f64(x, scale: float | None = None) -> np.ndarray:
    """Butterfly transform over the last axis in fp64; returns a new array."""
    x = np.array(x, dtype=np.float64, order="C", copy=True)
    n = x.shape[-1]
    rows = x.size // n if n else 0
    s = default_scale(n) if scale is None else scale
    if rows:
        lib().oracle_fwht_f64(_p(x), rows, n, s)
    return x


def fwht_f32(x, scale: float | None = None) -> np.ndarray:
    """Same butterfly in fp32 arithmetic (the scalar CPU port)."""
    x = np.array(x, dtype=np.float32, order="C", copy=True)
    n = x.shape[-1]
    rows = x.size // n if n else 0
    s = default_scale(n) if scale is None else scale
    if rows:
        lib().oracle_fwht_f32(_p(x), rows, n, s)
    return x


def fwht_matrix_f64(x, scale: float | None = None) -> np.ndarray:
    """Brute-force ``x @ (H * scale)`` in C, fp64."""
    x = np.ascontiguousarray(x, dtype=np.float64)
    n = x.shape[-1]
    rows = x.size // n
    y = np.empty_like(x)
    s = default_scale(n) if scale is None else scale
    lib().oracle_fwht_matrix_f64(_p(x), _p(y), rows, n, s)
    return y


def hadamard_matrix_ref(x, scale: float | None = None):
    """The reference's truth path on the CPU with torch: ``x @ (hadamard(n) * scale).to(dtype)``
    (HadaCore/test.py:27-40, bench/bench.py:49-59).  ``x`` is a CPU torch tensor [..., n]."""
    import scipy.linalg
    import torch

    n = x.shape[-1]
    s = default_scale(n) if scale is None else scale
    H = (torch.tensor(scipy.linalg.hadamard(n), dtype=torch.float32) * s).to(x.dtype)
    return x @ H


def fused_ht_gemv_f64(W, X, scale: float = 1.0) -> np.ndarray:
    """Y[M,B] = W[M,N] @ (scale * H_N @ X[N,B]); triple loop in C (small shapes)."""
    W = np.ascontiguousarray(W, dtype=np.float64)
    X = np.ascontiguousarray(X, dtype=np.float64)
    M, N = W.shape
    N2, B = X.shape
    assert N == N2
    Y = np.empty((M, B), dtype=np.float64)
    lib().oracle_fused_ht_gemv_f64(_p(W), _p(X), _p(Y), M, N, B, scale)
    return Y


def fused_ht_gemm_f64(W, Xt, scale: float = 1.0) -> np.ndarray:
    """C[M,N] = W[M,K] @ (scale * H_K @ X[K,N]), X given as Xt[N,K]; triple loop in C."""
    W = np.ascontiguousarray(W, dtype=np.float64)
    Xt = np.ascontiguousarray(Xt, dtype=np.float64)
    M, K = W.shape
    N, K2 = Xt.shape
    assert K == K2
    C = np.empty((M, N), dtype=np.float64)
    lib().oracle_fused_ht_gemm_f64(_p(W), _p(Xt), _p(C), M, N, K, scale)
    return C


def fused_ht_gemv_f64_blas(W, X, scale: float = 1.0) -> np.ndarray:
    """Same result as :func:`fused_ht_gemv_f64` with the contraction done by numpy (large
    shapes): butterfly down dim 0 of X, then ``W @ .``."""
    X = np.asarray(X, dtype=np.float64)
    HX = fwht_f64(X.T, scale).T
    return np.asarray(W, dtype=np.float64) @ HX


def fused_ht_gemm_f64_blas(W, Xt, scale: float = 1.0) -> np.ndarray:
    """Same result as :func:`fused_ht_gemm_f64` with the contraction done by numpy."""
    HXt = fwht_f64(np.asarray(Xt, dtype=np.float64), scale)  # rows of Xt are columns of X
    return np.asarray(W, dtype=np.float64) @ HXt.T


def _conv(name, x, src_dtype, dst_dtype):
    x = np.ascontiguousarray(x, dtype=src_dtype)
    y = np.empty(x.shape, dtype=dst_dtype)
    getattr(lib(), name)(_p(x), _p(y), x.size)
    return y


def f32_to_bf16(x) -> np.ndarray:
    return _conv("oracle_f32_to_bf16_array", x, np.float32, np.uint16)


def bf16_to_f32(bits) -> np.ndarray:
    b = np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16
    return b.view(np.float32)


def f32_to_f16(x) -> np.ndarray:
    return _conv("oracle_f32_to_f16_array", x, np.float32, np.uint16)


def f16_to_f32(bits) -> np.ndarray:
    return _conv("oracle_f16_to_f32_array", bits, np.uint16, np.float32)


def e4m3fn_encode(x) -> np.ndarray:
    return _conv("oracle_e4m3fn_encode_array", x, np.float32, np.uint8)


def e4m3fn_decode(codes) -> np.ndarray:
    return _conv("oracle_e4m3fn_decode_array", codes, np.uint8, np.float32)


def quant_fp8_rows(y):
    """Per-row amax FP8 quantizer on pre-quant values ``y[T,n]`` (fp32).  Returns
    ``(codes uint8 [T,n], row_scale float32 [T])``."""
    y = np.ascontiguousarray(y, dtype=np.float32)
    T, n = y.shape
    q = np.empty((T, n), dtype=np.uint8)
    s = np.empty((T,), dtype=np.float32)
    lib().oracle_quant_fp8_rows(_p(y), _p(q), _p(s), T, n)
    return q, s


def rht_f64(x, sign, scale: float | None = None) -> np.ndarray:
    """y = scale * H_n (sign .* x) per row in fp64."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    sign = np.ascontiguousarray(sign, dtype=np.int8)
    T, n = x.shape
    y = np.empty((T, n), dtype=np.float64)
    s = default_scale(n) if scale is None else scale
    lib().oracle_rht_f64(_p(x), _p(sign), _p(y), T, n, s)
    return y


def rel_err(y, y64) -> float:
    """max|y - y64| / max|y64|: the tolerance metric of the build contract."""
    y = np.asarray(y, dtype=np.float64)
    y64 = np.asarray(y64, dtype=np.float64)
    den = float(np.max(np.abs(y64))) if y64.size else 0.0
    if y64.size == 0:
        return 0.0
    return float(np.max(np.abs(y - y64))) / (den if den > 0 else 1.0)


# ---- seeded inputs: CPU torch generators, seed 0 = X, 1 = W, 2 = sign diagonal, 3 = outliers ----

def _gen(seed):
    import torch
    return torch.Generator().manual_seed(seed)


def inputs_fwht(rows: int, n: int, dtype):
    """X[rows, n] iid N(0,1) from seed 0, cast to ``dtype`` (a torch dtype); CPU tensor."""
    import torch
    return torch.randn(rows, n, generator=_gen(0), dtype=torch.float32).to(dtype)


def inputs_gemv(M: int, N: int, B: int):
    """W[M,N] ~ N(0, 1/N) from seed 1, X[N,B] ~ N(0,1) from seed 0; fp32 CPU tensors."""
    import torch
    W = torch.randn(M, N, generator=_gen(1), dtype=torch.float32) * (1.0 / math.sqrt(N))
    X = torch.randn(N, B, generator=_gen(0), dtype=torch.float32)
    return W, X


def inputs_gemm(M: int, N: int, K: int, dtype):
    """W[M,K] from seed 1 and Xt[N,K] from seed 0, iid N(0,1), cast to ``dtype``."""
    import torch
    W = torch.randn(M, K, generator=_gen(1), dtype=torch.float32).to(dtype)
    Xt = torch.randn(N, K, generator=_gen(0), dtype=torch.float32).to(dtype)
    return W, Xt


def inputs_rht(T: int, n: int, outlier_frac: float = 0.01, outlier_gain: float = 50.0):
    """bf16 activations [T,n] ~ N(0,1) (seed 0) with ``outlier_frac`` of the channels (chosen by
    ``randperm`` from seed 3) multiplied by ``outlier_gain``; sign diagonal in {+1,-1} int8 from
    seed 2.  Returns (x bf16 CPU tensor, sign int8 CPU tensor)."""
    import torch
    x = torch.randn(T, n, generator=_gen(0), dtype=torch.float32)
    k = int(round(n * outlier_frac))
    if k > 0:
        cols = torch.randperm(n, generator=_gen(3))[:k]
        x[:, cols] *= outlier_gain
    sign = (1 - 2 * torch.randint(0, 2, (n,), generator=_gen(2))).to(torch.int8)
    return x.to(torch.bfloat16), sign
