"""ctypes binding of ``libmi_hadamard.so`` (declarations: ``include/mi_hadamard.h``) and of the
benchmark harness's ``libmi_probe.so`` (``include/mi_probe.h``)."""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmi_hadamard.so")

MI_F32, MI_BF16, MI_F16 = 0, 1, 2

# name -> (restype, argtypes); mirrors include/mi_hadamard.h one to one
_vp, _u64, _u32, _i, _f = (ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_int,
                           ctypes.c_float)
SIGNATURES = {
    "mi_version": (_i, []),
    "mi_status_string": (ctypes.c_char_p, [_i]),
    "mi_fwht": (_i, [_vp, _vp, _u64, _u32, _i, _f, _vp]),
    "mi_fused_ht_gemv": (_i, [_vp, _vp, _vp, _u32, _u32, _u32, _i, _f, _vp]),
    "mi_fused_ht_gemm": (_i, [_vp, _vp, _vp, _u32, _u32, _u32, _i, _i, _f, _vp]),
    "mi_rht_quant_fp8": (_i, [_vp, _vp, _vp, _vp, _vp, _u64, _u32, _f, _vp]),
    "mi_fp8_gemm_rowscale": (_i, [_vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _vp]),
    "mi_debug_mfma_16x16": (_i, [_i, _vp, _vp, _vp, _vp]),
    "mi_debug_convert": (_i, [_i, _vp, _vp, _u64, _vp]),
    "mi_debug_device_fwht": (_i, [_vp, _vp, _u64, _u32, _i, _f, _vp]),
    "mi_debug_fused_gemm_tiling": (_i, [_u32, _u32, _u32, _vp, _vp, _u32]),
}

PROBE_LIB_PATH = os.path.join(HERE, "libmi_probe.so")
PROBE_SIGNATURES = {
    "mi_probe_mfma_rate": (_i, [_i, _i, _u32, _u32, _vp, _vp, _vp]),
    "mi_probe_issue_rate": (_i, [_i, _i, _i, _u32, _u32, _vp, _vp, _vp, _vp]),
    "mi_probe_stream_rate": (_i, [_i, _u32, _u32, _u64, _vp, _vp, _vp]),
}

_lib = None
_probe = None


def load() -> ctypes.CDLL:
    """Load the library (once).  torch is imported first so that the HIP runtime already in the
    process is the one the library binds to.  There is no fallback: a missing library is an
    error, because every op in this package runs only as a HIP kernel."""
    global _lib
    if _lib is not None:
        return _lib
    import torch  # noqa: F401  (loads libamdhip64 with torch's own copy first)

    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python 6s894_project_2025_amd/build.py` "
            "(there is no CPU or PyTorch fallback for these ops)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def load_probe() -> ctypes.CDLL:
    """Load the matrix-core rate probe (benchmark harness only; no op of the package uses it)."""
    global _probe
    if _probe is not None:
        return _probe
    load()
    if not os.path.exists(PROBE_LIB_PATH):
        raise RuntimeError(f"{PROBE_LIB_PATH} is missing: build it with `python 6s894_project_2025_amd/build.py`")
    lib = ctypes.CDLL(PROBE_LIB_PATH)
    for name, (res, args) in PROBE_SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _probe = lib
    return lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().mi_status_string(status).decode()
        raise RuntimeError(f"{what}: {msg} (status {status})")
