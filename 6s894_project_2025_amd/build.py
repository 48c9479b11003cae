"""Builds ``libmi_hadamard.so`` (the C-ABI library) and ``libmi_probe.so`` (the benchmark
harness's matrix-core rate probe, kept out of the product library) in-tree with hipcc for gfx950.

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
PROBE_SRC = os.path.join(HERE, "probe")
PROBE_LIB_PATH = os.path.join(HERE, "libmi_probe.so")

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
    "fused_gemv_rows.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


# The register-resident kernels issue their main-loop MFMAs as inline assembly with the B operand
# named directly in the accumulation-register file.  If register pressure ever makes the compiler
# keep part of that operand elsewhere, it copies the value into one accumulation register right
# before each use - while the previous MFMA may still be reading that register, which silently
# corrupts results.  The build therefore looks at the generated ISA of these files and fails when an
# accumulation register is written anywhere after a kernel's first such MFMA.
#
# The compiler does not know either that the result of such an MFMA arrives when the instruction
# retires: an ordinary instruction that touches the destination registers too soon (a register copy
# the allocator puts on a loop edge, say) would see the old value, where for its own MFMAs the
# compiler inserts the wait states.  The build fails when anything but another MFMA reads an
# assembly MFMA's destination within kResultWaitStates issue slots on any path.
ISA_CHECKED = {"fused_gemm_xreg.hip", "fused_gemm_xreg_f32.hip", "fused_gemm_xreg_k2048.hip", "fused_gemv_rows.hip"}
# Files whose MFMAs are the compiler's own but which use the direct global -> LDS transfers (M0 is
# theirs alone) and wait for them by hand before ordinary LDS reads: the M0 and LDS-read checks only.
TRANSFER_CHECKED = {"fused_gemv_stream.hip"}
_MFMA_B_IN_AGPR = re.compile(r"^\s*v_mfma_\S+\s+v\[[0-9:]+\], v\S+, a")
_AGPR_WRITE = re.compile(r"^\s*v_accvgpr_(write|mov)")
_LABEL = re.compile(r"^([A-Za-z_][\w$]*):")
_ANY_LABEL = re.compile(r"^([.A-Za-z_][\w$.]*):")
_VREG_RANGE = re.compile(r"\bv\[(\d+):(\d+)\]")
_VREG = re.compile(r"\bv(\d+)\b")
kResultWaitStates = 11  # an eight-pass MFMA (16x16x32 16-bit, 16x16x4 fp32): passes + 3


def _vregs(text: str) -> set:
    regs = set()
    for m in _VREG_RANGE.finditer(text):
        regs.update(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in _VREG.finditer(text):
        regs.add(int(m.group(1)))
    return regs


_NO_DESTINATION = ("ds_write", "ds_store", "global_store", "global_atomic", "global_load_lds", "scratch_store",
                   "buffer_store", "flat_store")


def _source_operands(text: str) -> str:
    """The operands an instruction reads: all but the first, or all for stores and their like."""
    op, _, rest = text.partition(" ")
    if op.startswith(_NO_DESTINATION):
        return rest
    return rest.partition(",")[2]


def check_mfma_results_not_touched_early(asm_text: str, where: str) -> int:
    """Raises if a non-MFMA instruction reads the destination of an assembly MFMA (one whose B
    operand is an accumulation register) within kResultWaitStates issue slots, on any path the
    branches allow; returns the number of MFMAs checked.  (Writes are left alone: branch conditions
    are not evaluated, and on the impossible path from a block whose result awaits its stores into a
    block variant that has none to do, the allocator rightly reuses those registers.)"""
    checked = 0
    lines = asm_text.splitlines()
    i = 0
    while i < len(lines):
        label = _LABEL.match(lines[i])
        if not label:
            i += 1
            continue
        name = label.group(1)
        # one function: instructions and the positions of its local labels
        ins, labels = [], {}
        i += 1
        while i < len(lines) and not _LABEL.match(lines[i]):
            text = lines[i].split(";")[0].strip()
            local = _ANY_LABEL.match(text)
            if local:
                labels[local.group(1)] = len(ins)
            elif text and not text.startswith("."):
                ins.append(text)
            i += 1
        for at, text in enumerate(ins):
            if not _MFMA_B_IN_AGPR.match(text):
                continue
            checked += 1
            seen = set()
            todo = [(at + 1, kResultWaitStates, frozenset(_vregs(text.split(",")[0])))]
            while todo:
                k, left, pending = todo.pop()
                while left > 0 and pending and k < len(ins) and (k, left, pending) not in seen:
                    seen.add((k, left, pending))
                    t = ins[k]
                    op = t.split()[0]
                    if op == "s_endpgm":
                        break
                    if not op.startswith("v_mfma"):
                        if _vregs(_source_operands(t)) & pending:
                            raise RuntimeError(f"{where}: {name}: `{t}` reads the result of `{text}` "
                                               f"{kResultWaitStates - left} issue slots after it")
                        if not op.startswith(_NO_DESTINATION):  # a register written anew is no longer that result
                            pending = pending - _vregs(t.partition(",")[0])
                    if op == "s_branch":
                        k = labels.get(t.split()[1], len(ins))
                        left -= 1
                        continue
                    if op.startswith("s_cbranch"):
                        todo.append((labels.get(t.split()[1], len(ins)), left - 1, pending))
                    left -= int(t.split()[1], 0) + 1 if op == "s_nop" else 1
                    k += 1
    return checked


kOperandReadSlots = 4  # issue slots during which a 16-pass-or-shorter MFMA may still be reading A


def check_mfma_operands_not_overwritten_early(asm_text: str, where: str) -> int:
    """The matrix core reads the A operand of an MFMA over several cycles after issue, and for an
    inline-assembly MFMA the compiler inserts no wait states for that: a vector instruction that
    writes one of those registers right behind the MFMA corrupts the product (observed with a
    register copy one instruction later).  Raises if, within kOperandReadSlots issue slots of an
    assembly MFMA (one whose B operand is an accumulation register) and on any path the branches
    allow, a vector ALU instruction writes a register of its A operand; returns the number of MFMAs
    checked.  (Loads are left alone: their data arrives far later than that.)"""
    checked = 0
    lines = asm_text.splitlines()
    i = 0
    while i < len(lines):
        label = _LABEL.match(lines[i])
        if not label:
            i += 1
            continue
        name = label.group(1)
        ins, labels = [], {}
        i += 1
        while i < len(lines) and not _LABEL.match(lines[i]):
            text = lines[i].split(";")[0].strip()
            local = _ANY_LABEL.match(text)
            if local:
                labels[local.group(1)] = len(ins)
            elif text and not text.startswith("."):
                ins.append(text)
            i += 1
        for at, text in enumerate(ins):
            if not _MFMA_B_IN_AGPR.match(text):
                continue
            checked += 1
            operand_a = frozenset(_vregs(text.split(",")[1]))
            todo = [(at + 1, kOperandReadSlots)]
            seen = set()
            while todo:
                k, left = todo.pop()
                while left > 0 and k < len(ins) and (k, left) not in seen:
                    seen.add((k, left))
                    t = ins[k]
                    op = t.split()[0]
                    if op == "s_endpgm":
                        break
                    if op.startswith("v_") and not op.startswith("v_mfma") and not op.startswith("v_cmp"):
                        if _vregs(t.partition(" ")[2].split(",")[0]) & operand_a:
                            raise RuntimeError(f"{where}: {name}: `{t}` overwrites the A operand of `{text}` "
                                               f"{kOperandReadSlots - left} issue slots after it")
                    if op == "s_branch":
                        k = labels.get(t.split()[1], len(ins))
                        left -= 1
                        continue
                    if op.startswith("s_cbranch"):
                        todo.append((labels.get(t.split()[1], len(ins)), left - 1))
                    left -= int(t.split()[1], 0) + 1 if op == "s_nop" else 1
                    k += 1
    return checked


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


_M0_USE = re.compile(r"\bm0\b")
_M0_SET_BY_TRANSFER = re.compile(r"^\s*s_add_i32 m0, ")


def check_m0_is_the_transfers_alone(asm_text: str, where: str) -> int:
    """The direct global -> LDS transfers take their LDS base from M0, written by an opaque statement
    one instruction earlier.  Raises if any other instruction of the file names M0 (a compiler use
    between the two would redirect a transfer); returns the number of M0 writes seen."""
    writes = 0
    for line in asm_text.splitlines():
        text = line.split(";")[0]
        if not _M0_USE.search(text) or text.lstrip().startswith("."):
            continue
        if _M0_SET_BY_TRANSFER.match(text):
            writes += 1
        else:
            raise RuntimeError(f"{where}: `{text.strip()}` uses M0, which belongs to the global -> LDS transfers")
    return writes


_LGKM_WAIT = re.compile(r"lgkmcnt\((\d+)\)")
kLdsReadHorizon = 400  # instructions followed per path; a fragment is used within a few K steps


def check_lds_reads_waited_for(asm_text: str, where: str) -> int:
    """An LDS read written as an opaque statement returns a register that holds nothing until a
    hand-placed `s_waitcnt lgkmcnt` has covered it.  Raises if, on any path the branches allow, an
    instruction reads or overwrites the destination of a `ds_read` before a wait that covers it
    (LDS operations complete in order: a wait for at most as many outstanding operations as were
    issued after the read); returns the number of reads checked.  Compiler-generated reads are
    checked alike (the compiler waits before their first use)."""
    checked = 0
    lines = asm_text.splitlines()
    i = 0
    while i < len(lines):
        label = _LABEL.match(lines[i])
        if not label:
            i += 1
            continue
        name = label.group(1)
        ins, labels = [], {}
        i += 1
        while i < len(lines) and not _LABEL.match(lines[i]):
            text = lines[i].split(";")[0].strip()
            local = _ANY_LABEL.match(text)
            if local:
                labels[local.group(1)] = len(ins)
            elif text and not text.startswith("."):
                ins.append(text)
            i += 1
        for at, text in enumerate(ins):
            if not text.startswith("ds_read"):
                continue
            checked += 1
            dest = frozenset(_vregs(text.split(",")[0]))
            seen = set()
            todo = [(at + 1, 0, kLdsReadHorizon)]  # position, LDS operations issued since, steps left
            while todo:
                k, younger, left = todo.pop()
                while left > 0 and k < len(ins) and (k, younger) not in seen:
                    seen.add((k, younger))
                    t = ins[k]
                    op = t.split()[0]
                    if op == "s_endpgm":
                        break
                    if op == "s_waitcnt":
                        m = _LGKM_WAIT.search(t)
                        if m and int(m.group(1)) <= younger:
                            break  # covered on this path
                    elif op == "s_branch":
                        k = labels.get(t.split()[1], len(ins))
                        left -= 1
                        continue
                    else:
                        touched = _vregs(t if op.startswith(_NO_DESTINATION) else t.partition(" ")[2])
                        if touched & dest:
                            raise RuntimeError(f"{where}: {name}: `{t}` touches the destination of `{text}` "
                                               f"before an s_waitcnt lgkmcnt that covers it")
                        if op.startswith("ds_"):
                            younger += 1
                        if op.startswith("s_cbranch"):
                            todo.append((labels.get(t.split()[1], len(ins)), younger, left - 1))
                    left -= 1
                    k += 1
    return checked


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
    transfers = base in TRANSFER_CHECKED
    cmd = [_hipcc(), *HIPCC_FLAGS, *PER_FILE_FLAGS.get(base, []),
           *(["-save-temps=obj"] if checked or transfers else []), "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    if checked or transfers:
        temps = glob.glob(os.path.join(OBJ_DIR, base[:-4] + "-*")) + glob.glob(os.path.join(OBJ_DIR, base + "-*"))
        isa = [t for t in temps if t.endswith(f"{ARCH}.s")]
        if len(isa) != 1:
            raise RuntimeError(f"no device assembly found for {src}")
        with open(isa[0]) as f:
            text = f.read()
        if checked and (check_register_resident_isa(text, base) == 0 or
                        check_mfma_results_not_touched_early(text, base) == 0):
            raise RuntimeError(f"{base}: no register-resident MFMA loop found in the device assembly")
        if check_m0_is_the_transfers_alone(text, base) == 0:
            raise RuntimeError(f"{base}: no global -> LDS transfer found in the device assembly")
        if check_lds_reads_waited_for(text, base) == 0:
            raise RuntimeError(f"{base}: no LDS read found in the device assembly")
        if checked:
            check_mfma_operands_not_overwritten_early(text, base)
        for t in temps:
            os.remove(t)
    return obj


def probe_sources() -> list[str]:
    return sorted(os.path.join(PROBE_SRC, f) for f in os.listdir(PROBE_SRC) if f.endswith(".hip"))


def _link(objs: list[str], lib_path: str) -> None:
    tmp = lib_path + ".tmp"
    cmd = [_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, lib_path)


def build(verbose: bool = True, jobs: int = 4) -> str:
    """Compile every ``csrc/*.hip`` into the product library and every ``probe/*.hip`` into the
    probe library.  Always recompiles."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs, probes = sources(), probe_sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, srcs + probes))
    _link(objs[:len(srcs)], LIB_PATH)
    _link(objs[len(srcs):], PROBE_LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources, {PROBE_LIB_PATH} from {len(probes)}")
    return LIB_PATH


if __name__ == "__main__":
    build()
