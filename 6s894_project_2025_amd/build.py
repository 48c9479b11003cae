"""Builds ``libmi_hadamard.so`` (the C-ABI library) in-tree with hipcc for gfx950.

Run as ``python 6s894_project_2025_amd/build.py`` or through ``__graft_entry__.build()``.
hipcc cross-compiles without a GPU, so this works on a CPU-only machine.
"""
from __future__ import annotations

import concurrent.futures
import glob
import os
import re
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
    "fused_gemm_xreg_k2048.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


# The register-resident kernels issue their main-loop MFMAs as inline assembly with the B operand
# named directly in the accumulation-register file.  If register pressure ever makes the compiler
# keep part of that operand elsewhere, it copies the value into one accumulation register right
# before each use - while the previous MFMA may still be reading that register, which silently
# corrupts results.  The build therefore looks at the generated ISA of these files and fails when an
# accumulation register is written anywhere after a kernel's first such MFMA.
ISA_CHECKED = {"fused_gemm_xreg.hip", "fused_gemm_xreg_f32.hip", "fused_gemm_xreg_k2048.hip"}
_MFMA_B_IN_AGPR = re.compile(r"^\s*v_mfma_\S+\s+v\[[0-9:]+\], v\S+, a")
_AGPR_WRITE = re.compile(r"^\s*v_accvgpr_(write|mov)")
_LABEL = re.compile(r"^([A-Za-z_][\w$]*):")


def check_register_resident_isa(asm_text: str, where: str) -> int:
    """Raises if a kernel writes accumulation registers after its first MFMA that reads its B
    operand from them; returns the number of kernels checked."""
    kernels = 0
    name, armed = None, False
    for line in asm_text.splitlines():
        label = _LABEL.match(line)
        if label:  # a function (local labels start with a dot)
            name, armed = label.group(1), False
            continue
        if name is None:
            continue
        if "s_endpgm" in line:
            kernels += armed
            name, armed = None, False
        elif _MFMA_B_IN_AGPR.match(line):
            armed = True
        elif armed and _AGPR_WRITE.match(line):
            raise RuntimeError(f"{where}: {name} writes an accumulation register inside its MFMA loop "
                               f"({line.strip()}): the transformed operand no longer fits the register file")
    return kernels


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP kernels cannot be built")
    return exe


def _compile(src: str) -> str:
    base = os.path.basename(src)
    obj = os.path.join(OBJ_DIR, base[:-4] + ".o")
    checked = base in ISA_CHECKED
    cmd = [_hipcc(), *HIPCC_FLAGS, *PER_FILE_FLAGS.get(base, []), *(["-save-temps=obj"] if checked else []),
           "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    if checked:
        temps = glob.glob(os.path.join(OBJ_DIR, base[:-4] + "-*")) + glob.glob(os.path.join(OBJ_DIR, base + "-*"))
        isa = [t for t in temps if t.endswith(f"{ARCH}.s")]
        if len(isa) != 1:
            raise RuntimeError(f"no device assembly found for {src}")
        with open(isa[0]) as f:
            n = check_register_resident_isa(f.read(), base)
        if n == 0:
            raise RuntimeError(f"{base}: no register-resident MFMA loop found in the device assembly")
        for t in temps:
            os.remove(t)
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
