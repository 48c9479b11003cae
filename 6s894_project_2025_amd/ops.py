"""Python-facing ops: thin host code over the C ABI (``include/mi_hadamard.h``).

``hadamard_transform`` keeps the call shape of the reference's pybind op
``hadamard_transform(x, inplace=False)`` (csrc/hadamard_transform.cpp:12-81,
HadaCore/hadamard_transform.cpp:15-59) and adds the ``scale`` argument of the build contract.
torch is used for device memory and streams only; all arithmetic happens in HIP kernels.
"""
from __future__ import annotations

import contextlib
import math

import torch

from . import _lib

_DTYPE_CODE = {torch.float32: _lib.MI_F32, torch.bfloat16: _lib.MI_BF16, torch.float16: _lib.MI_F16}
MAX_LOG_N = 15
# ranges of the C ABI (include/mi_hadamard.h); the wrappers reject the same values it does
GEMV_MAX_N = 2048
GEMM_MIN_K, GEMM_MAX_K = 32, 4096


def _is_pow2(n: int) -> bool:
    return n > 0 and (n & (n - 1)) == 0


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_SAME_DEVICE = contextlib.nullcontext()


def _stream(t: torch.Tensor) -> int:
    """The current stream of ``t``'s device as a raw handle (the direct query when this torch has
    it: a fraction of the cost of building a ``torch.cuda.Stream`` object on every call)."""
    if _RAW_STREAM is not None and t.device.index is not None:
        return _RAW_STREAM(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


def _on_device_of(t: torch.Tensor):
    """Context that makes ``t``'s device current for the launch; nothing to do (and nothing to
    pay) when it already is, the usual case."""
    if t.device.index is None or t.device.index == torch.cuda.current_device():
        return _SAME_DEVICE
    return torch.cuda.device(t.device)


def _require_cuda(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor (got device {t.device})")


def _dense16(t: torch.Tensor) -> torch.Tensor:
    """`t` itself if it is contiguous and 16-byte aligned, else a fresh contiguous copy."""
    if t.is_contiguous():
        return t if t.data_ptr() % 16 == 0 else t.clone()
    return t.contiguous()


def hadamard_transform(x: torch.Tensor, scale: float | None = None, *, inplace: bool = False
                       ) -> torch.Tensor:
    """Walsh-Hadamard transform over the last dimension: ``y = scale * x @ H_n``.

    ``scale=None`` means ``n ** -0.5``, the normalisation the reference always applies.  Any
    leading dimensions are allowed; ``n = x.size(-1)`` must be a power of two up to 2**15;
    dtype fp16, bf16 or fp32.  ``inplace=True`` writes into ``x``'s storage and returns ``x``
    (through a temporary when ``x`` is not dense or not 16-byte aligned, as the reference does,
    csrc/hadamard_transform.cpp:65-68); otherwise a new tensor of the same shape is returned.
    Errors are ``RuntimeError`` like the reference's ``TORCH_CHECK`` failures.
    """
    if x.dtype not in _DTYPE_CODE:
        raise RuntimeError(f"Only fp16, bf16 and fp32 supported currently (got {x.dtype})")
    _require_cuda(x, "x")
    if x.dim() == 0:
        raise RuntimeError("hadamard_transform needs at least one dimension")
    n = x.size(-1)
    if not _is_pow2(n) or n > (1 << MAX_LOG_N):
        raise RuntimeError(
            f"Only power of two Hadamard sizes up to 2^{MAX_LOG_N} are supported, got {n}")
    s = 1.0 / math.sqrt(n) if scale is None else float(scale)
    if x.numel() == 0:
        return x if inplace else torch.empty_like(x)

    src = _dense16(x)
    rows = src.numel() // n
    if inplace:
        dst = src
    else:
        dst = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    lib = _lib.load()
    with _on_device_of(x):
        st = lib.mi_fwht(src.data_ptr(), dst.data_ptr(), rows, n, _DTYPE_CODE[x.dtype], s,
                         _stream(x))
    _lib.check(st, "hadamard_transform")
    if inplace:
        if src is not x:
            x.copy_(src.view(x.shape))
        return x
    return dst


def fused_ht_gemv(W: torch.Tensor, X: torch.Tensor, scale: float | None = None) -> torch.Tensor:
    """``Y[M,B] = W[M,N] @ (scale * H_N @ X[N,B])`` in one kernel, fp32.

    Layouts as the reference indexes them (fused_ht/fwht_gemv_fusion.cu:50-51,146,156): all
    row-major, the transform runs down dim 0 of ``X``.  ``scale=None`` -> ``N ** -0.5``;
    ``scale=1.0`` reproduces the reference kernel (raw +-1 butterfly).
    """
    _require_cuda(W, "W")
    _require_cuda(X, "X")
    if W.dtype != torch.float32 or X.dtype != torch.float32:
        raise RuntimeError("fused_ht_gemv supports fp32 only")
    if W.dim() != 2 or X.dim() != 2 or W.size(1) != X.size(0):
        raise RuntimeError(f"shape mismatch: W {tuple(W.shape)} X {tuple(X.shape)}")
    M, N = W.shape
    B = X.size(1)
    if not _is_pow2(N) or N < 2 or N > GEMV_MAX_N:
        raise RuntimeError(f"N must be a power of two in [2, {GEMV_MAX_N}], got {N}")
    s = 1.0 / math.sqrt(N) if scale is None else float(scale)
    Y = torch.empty((M, B), dtype=torch.float32, device=W.device)
    if M == 0 or B == 0:
        return Y
    Wc, Xc = _dense16(W), _dense16(X)
    lib = _lib.load()
    with _on_device_of(W):
        st = lib.mi_fused_ht_gemv(Wc.data_ptr(), Xc.data_ptr(), Y.data_ptr(), M, N, B,
                                  _lib.MI_F32, s, _stream(W))
    _lib.check(st, "fused_ht_gemv")
    return Y


def fused_ht_gemm(W: torch.Tensor, Xt: torch.Tensor, scale: float | None = None,
                  out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """``C[M,N] = W[M,K] @ (scale * H_K @ X[K,N])`` with ``X`` given as ``Xt[N,K]`` (each column
    of X contiguous), the layout of fused_ht/fusion_pipelined.cu:164,211,220.  The transformed
    operand stays on chip.  fp32 (fp32 MFMA) or bf16/fp16 inputs (fp32 accumulate);
    ``out_dtype`` defaults to the input dtype.  ``scale=None`` -> ``K ** -0.5``; ``scale=1.0``
    reproduces the reference kernel.

    Where fusing pays on this chip: 16-bit inputs with K <= 1024 (the transformed operand of 128
    columns fits a compute unit's registers at K = 1024, of 256 columns at K = 512), and K = 2048
    or 4096 up to about M = N = 2048; fp32 inputs run 1.3 - 3.6 x ahead of the unfused
    route up to about M = N = 1024 and level with it beyond (both at the fp32 matrix-core rate).  For larger problems at K >= 2048,
    ``hadamard_transform(Xt)`` followed by a library GEMM is the faster route (by 10 - 35 %); this
    op still runs those shapes, for callers that cannot afford the intermediate.  K = 4096 is two
    kernels on the current stream, the second adding to what the first stored.
    """
    _require_cuda(W, "W")
    _require_cuda(Xt, "Xt")
    if W.dtype != Xt.dtype or W.dtype not in _DTYPE_CODE:
        raise RuntimeError(f"W and Xt must share a dtype in fp32/bf16/fp16 (got {W.dtype}, {Xt.dtype})")
    if W.dim() != 2 or Xt.dim() != 2 or W.size(1) != Xt.size(1):
        raise RuntimeError(f"shape mismatch: W {tuple(W.shape)} Xt {tuple(Xt.shape)}")
    M, K = W.shape
    N = Xt.size(0)
    if not _is_pow2(K) or K < GEMM_MIN_K or K > GEMM_MAX_K:
        raise RuntimeError(f"K must be a power of two in [{GEMM_MIN_K}, {GEMM_MAX_K}], got {K}")
    od = W.dtype if out_dtype is None else out_dtype
    if od not in (torch.float32, W.dtype):
        raise RuntimeError("out_dtype must be fp32 or the input dtype")
    s = 1.0 / math.sqrt(K) if scale is None else float(scale)
    C = torch.empty((M, N), dtype=od, device=W.device)
    if M == 0 or N == 0:
        return C
    Wc, Xc = _dense16(W), _dense16(Xt)
    lib = _lib.load()
    with _on_device_of(W):
        st = lib.mi_fused_ht_gemm(Wc.data_ptr(), Xc.data_ptr(), C.data_ptr(), M, N, K,
                                  _DTYPE_CODE[W.dtype], _DTYPE_CODE[od], s, _stream(W))
    _lib.check(st, "fused_ht_gemm")
    return C


def rht_quant_fp8(x: torch.Tensor, sign: torch.Tensor, scale: float | None = None,
                  return_prequant: bool = False):
    """Randomized Hadamard + FP8 quantize.  ``y = scale * H_n (sign * x)`` per row, rounded to
    bf16, then per-row amax scaling to OCP E4M3FN.  Returns ``(q, row_scale)`` with ``q`` a
    ``torch.float8_e4m3fn`` tensor and ``row_scale`` fp32 dequantisation factors
    (``y ~ q.float() * row_scale[:, None]``); with ``return_prequant`` also the bf16 ``y``.
    """
    _require_cuda(x, "x")
    if x.dtype != torch.bfloat16:
        raise RuntimeError("rht_quant_fp8 takes bf16 activations")
    if x.dim() != 2:
        raise RuntimeError("x must be [T, n]")
    T, n = x.shape
    if not _is_pow2(n) or n < 16 or n > 4096:
        raise RuntimeError(f"n must be a power of two in [16, 4096], got {n}")
    if sign.numel() != n:
        raise RuntimeError("sign must have n entries")
    s = 1.0 / math.sqrt(n) if scale is None else float(scale)
    sg = sign.to(device=x.device, dtype=torch.int8).contiguous()
    xc = _dense16(x)
    q = torch.empty((T, n), dtype=torch.uint8, device=x.device)
    rs = torch.empty((T,), dtype=torch.float32, device=x.device)
    y = torch.empty((T, n), dtype=torch.bfloat16, device=x.device) if return_prequant else None
    if T:
        lib = _lib.load()
        with _on_device_of(x):
            st = lib.mi_rht_quant_fp8(xc.data_ptr(), sg.data_ptr(), q.data_ptr(), rs.data_ptr(),
                                      y.data_ptr() if y is not None else None, T, n, s, _stream(x))
        _lib.check(st, "rht_quant_fp8")
    q = q.view(torch.float8_e4m3fn)
    return (q, rs, y) if return_prequant else (q, rs)


def fp8_gemm_rowscale(qa: torch.Tensor, sa: torch.Tensor, qb: torch.Tensor, sb: torch.Tensor
                      ) -> torch.Tensor:
    """``out[T,N] = bf16((qa[T,K] @ qb[N,K].T) * sa[:,None] * sb[None,:])`` on the FP8 matrix
    cores, fp32 accumulate.  ``qa``/``qb`` are ``torch.float8_e4m3fn`` (or uint8 codes)."""
    _require_cuda(qa, "qa")
    _require_cuda(qb, "qb")
    if qa.dim() != 2 or qb.dim() != 2 or qa.size(1) != qb.size(1):
        raise RuntimeError("shape mismatch")
    if qa.element_size() != 1 or qb.element_size() != 1:
        raise RuntimeError(f"qa and qb must hold one-byte E4M3FN codes (got {qa.dtype}, {qb.dtype})")
    if qb.device != qa.device:
        raise RuntimeError("qa and qb must be on the same device")
    T, K = qa.shape
    N = qb.size(0)
    if K % 128 != 0:
        raise RuntimeError("K must be a multiple of 128")
    if sa.numel() != T or sb.numel() != N:
        raise RuntimeError(f"scale lengths {sa.numel()}, {sb.numel()} do not match T={T}, N={N}")
    out = torch.empty((T, N), dtype=torch.bfloat16, device=qa.device)
    if T == 0 or N == 0:
        return out
    a = _dense16(qa.view(torch.uint8))
    b = _dense16(qb.view(torch.uint8))
    # the kernel dereferences the scales on the device: bring them there like `sign` above
    sa = sa.to(device=qa.device, dtype=torch.float32).contiguous().view(-1)
    sb = sb.to(device=qa.device, dtype=torch.float32).contiguous().view(-1)
    lib = _lib.load()
    with _on_device_of(qa):
        st = lib.mi_fp8_gemm_rowscale(a.data_ptr(), sa.data_ptr(), b.data_ptr(), sb.data_ptr(),
                                      out.data_ptr(), T, N, K, _stream(qa))
    _lib.check(st, "fp8_gemm_rowscale")
    return out
