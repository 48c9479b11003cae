"""Builds ``libmi_hadamard.so`` (the C-ABI library) in-tree with hipcc for gfx950.

Run as ``python 6s894_project_2025_amd/build.py`` or through ``__graft_entry__.build()``.
hipcc cross-compiles without a GPU, so this works on a CPU-only machine.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libmi_hadamard.so")

ARCH = "gfx950"
# Packed-fp32 VALU forms are switched off for every device translation unit.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-ffp-contract=off",
    "-Wall", "-Wno-unused-command-line-argument",
    f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}",
]


# Extra flags per translation unit.  The streaming kernels read every MFMA result with VALU code
# straight away, so they keep MFMA destinations in ordinary VGPRs (no accumulator-register copies).
PER_FILE_FLAGS = {
    "fwht.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "rht_fp8.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    # the prologue's MFMA results feed VALU conversions; the main loop's MFMAs are inline assembly
    "fused_gemm_xreg.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "fused_gemm_xreg_f32.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP kernels cannot be built")
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *PER_FILE_FLAGS.get(os.path.basename(src), []), "-c", src, "-o",
           obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True, jobs: int = 4) -> str:
    """Compile every ``csrc/*.hip`` and link the shared library.  Always recompiles."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, srcs))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources")
    return LIB_PATH


if __name__ == "__main__":
    build()
