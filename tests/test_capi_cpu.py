"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol the header
declares, validates arguments before touching the device, and the Python ops raise the
reference's kind of error (RuntimeError, like TORCH_CHECK) on bad input."""
import importlib
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi_hadamard.h")


PROBE_HEADER = os.path.join(ROOT, "include", "mi_probe.h")


def _declared_symbols(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def libmod(pkg):
    return importlib.import_module(pkg.__name__ + "._lib")


def test_library_exports_every_declared_symbol(libmod):
    lib = libmod.load()
    declared = _declared_symbols()
    assert declared, "header parse found nothing"
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/mi_hadamard.h but not exported"
    assert sorted(libmod.SIGNATURES) == declared


def test_probe_library_is_separate_from_the_product_library(libmod):
    # the matrix-core rate probe is a measurement aid: its own header, its own library, and the
    # product library exports nothing of it
    declared = _declared_symbols(PROBE_HEADER)
    assert declared == sorted(libmod.PROBE_SIGNATURES) == ["mi_probe_issue_rate", "mi_probe_mfma_rate",
                                                           "mi_probe_stream_rate"]
    probe = libmod.load_probe()
    for name in declared:
        assert hasattr(probe, name)
        assert not hasattr(libmod.load(), name)


def test_version_and_status_text(libmod):
    lib = libmod.load()
    assert lib.mi_version() >= 100
    for code in range(0, -8, -1):
        s = lib.mi_status_string(code)
        assert s and b"unknown" not in s
    assert b"unknown" in lib.mi_status_string(-99)


def test_argument_validation_happens_before_any_launch(libmod):
    lib = libmod.load()
    buf = 1 << 20  # fake, 16-byte aligned, never dereferenced: every call below must be rejected
    MI_ERR_DTYPE, MI_ERR_SIZE, MI_ERR_ALIGN, MI_ERR_NULL, MI_ERR_SHAPE, _, MI_ERR_ALIAS = range(-1, -8, -1)
    assert lib.mi_fwht(buf, buf, 4, 24, 1, 1.0, None) == MI_ERR_SIZE          # not a power of two
    assert lib.mi_fwht(buf, buf, 4, 1 << 16, 1, 1.0, None) == MI_ERR_SIZE     # above 2^15
    assert lib.mi_fwht(buf, buf, 0, 64, 1, 1.0, None) == 0                    # nothing to do
    assert lib.mi_fwht(None, buf, 4, 64, 1, 1.0, None) == MI_ERR_NULL
    assert lib.mi_fwht(buf + 2, buf + 2, 4, 64, 1, 1.0, None) == MI_ERR_ALIGN
    assert lib.mi_fwht(buf, buf, 4, 64, 7, 1.0, None) == MI_ERR_DTYPE
    assert lib.mi_fwht(buf, buf + 64, 4, 64, 1, 1.0, None) == MI_ERR_ALIAS    # partial overlap
    assert lib.mi_fused_ht_gemv(buf, buf, buf, 4, 24, 3, 0, 1.0, None) == MI_ERR_SIZE
    assert lib.mi_fused_ht_gemv(buf, buf, buf, 4, 32, 3, 1, 1.0, None) == MI_ERR_DTYPE
    assert lib.mi_fused_ht_gemv(buf, buf, buf, 0, 32, 3, 0, 1.0, None) == 0
    assert lib.mi_fused_ht_gemm(buf, buf, buf, 4, 4, 48, 1, 1, 1.0, None) == MI_ERR_SIZE
    assert lib.mi_fused_ht_gemm(buf, buf, buf, 4, 4, 64, 1, 2, 1.0, None) == MI_ERR_DTYPE
    assert lib.mi_fused_ht_gemm(buf, None, buf, 4, 4, 64, 1, 1, 1.0, None) == MI_ERR_NULL
    # the register-resident kernels address W with 32-bit byte offsets: more than 4 GiB of W is refused
    assert lib.mi_fused_ht_gemm(buf, buf, buf, 1 << 22, 64, 1024, 1, 1, 1.0, None) == MI_ERR_SHAPE
    assert lib.mi_fused_ht_gemm(buf, buf, buf, 1 << 20, 64, 4096, 1, 1, 1.0, None) == MI_ERR_SHAPE
    assert lib.mi_fused_ht_gemm(buf, buf, buf, 1 << 21, 64, 2048, 2, 0, 1.0, None) == MI_ERR_SHAPE
    assert lib.mi_fused_ht_gemm(buf, buf, buf, 1 << 20, 64, 1024, 0, 0, 1.0, None) == MI_ERR_SHAPE
    assert lib.mi_rht_quant_fp8(buf, buf, buf, buf, None, 4, 24, 1.0, None) == MI_ERR_SIZE
    assert lib.mi_rht_quant_fp8(buf, buf, buf, None, None, 4, 64, 1.0, None) == MI_ERR_NULL
    assert lib.mi_fp8_gemm_rowscale(buf, buf, buf, buf, buf, 4, 4, 100, None) == MI_ERR_SHAPE
    assert lib.mi_debug_mfma_16x16(9, buf, buf, buf, None) == MI_ERR_DTYPE
    assert lib.mi_debug_convert(5, buf, buf, 1, None) == MI_ERR_DTYPE


def test_python_ops_raise_runtime_errors_on_cpu_input(pkg):
    with pytest.raises(RuntimeError, match="supported"):
        pkg.hadamard_transform(torch.zeros(2, 8, dtype=torch.float64))
    with pytest.raises(RuntimeError, match="GPU"):
        pkg.hadamard_transform(torch.zeros(2, 8, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError):
        pkg.hadamard_transform(torch.tensor(1.0))
    with pytest.raises(RuntimeError, match="GPU"):
        pkg.fused_ht_gemv(torch.zeros(4, 8), torch.zeros(8, 2))
    with pytest.raises(RuntimeError, match="GPU"):
        pkg.fused_ht_gemm(torch.zeros(4, 32), torch.zeros(2, 32))
    with pytest.raises(RuntimeError, match="GPU"):
        pkg.rht_quant_fp8(torch.zeros(4, 32, dtype=torch.bfloat16), torch.ones(32, dtype=torch.int8))


def test_missing_library_fails_loudly(libmod, monkeypatch):
    monkeypatch.setattr(libmod, "_lib", None)
    monkeypatch.setattr(libmod, "LIB_PATH", os.path.join(ROOT, "does_not_exist.so"))
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        libmod.load()


def test_product_code_never_touches_the_oracle():
    pkgdir = os.path.join(ROOT, "6s894_project_2025_amd")
    for dirpath, _, files in os.walk(pkgdir):
        if os.path.basename(dirpath) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"
    hdr = open(HEADER).read().lower()
    assert "oracle" not in hdr


def _tiling(lib, M, N, K=1024):
    import ctypes

    header = (ctypes.c_uint32 * 8)()
    assert lib.mi_debug_fused_gemm_tiling(M, N, K, header, None, 0) == 0
    ngroups, msplit, m_per_block, mpx, cgx, nrect, grid, _ = list(header)
    tiles = (ctypes.c_uint32 * (2 * grid))()
    assert lib.mi_debug_fused_gemm_tiling(M, N, K, header, tiles, grid) == 0
    return dict(ngroups=ngroups, msplit=msplit, m_per_block=m_per_block, mpx=mpx, cgx=cgx,
                nrect=nrect, grid=grid), [(tiles[2 * i], tiles[2 * i + 1]) for i in range(grid)]


def test_fused_gemm_tiling_covers_every_tile_exactly_once(libmod):
    # host logic of the K = 1024 fused GEMM launch: no GPU call involved
    lib = libmod.load()
    shapes = [(4096, 4096), (1, 1), (64, 128), (65, 129), (577, 1333), (5000, 3000), (12288, 12288),
              (2048, 8192), (8192, 2048), (4096, 16384), (16384, 4096), (700, 4095), (130, 2000),
              (4096, 130), (100000, 128), (64, 100000), (9999, 7777), (8192, 8192), (3968, 31 * 128)]
    for M, N, K in [(m, n, 1024) for m, n in shapes] + [(m, n, 512) for m, n in shapes[:12]] + \
            [(m, n, 2048) for m, n in shapes[:12]] + [(m, n, 4096) for m, n in shapes[:12]]:
        p, tiles = _tiling(lib, M, N, K)
        assert p["ngroups"] == -(-N // max(64, 131072 // K))
        assert p["m_per_block"] % 64 == 0 and p["msplit"] == -(-M // p["m_per_block"])
        assert (p["msplit"] - 1) * p["m_per_block"] < M          # no empty slice
        real = [t for t in tiles if t != (0xFFFFFFFF, 0xFFFFFFFF)]
        want = {(cg, ms) for cg in range(p["ngroups"]) for ms in range(p["msplit"])}
        assert len(real) == len(want) and set(real) == want, (M, N, K, p)
        if True:
            assert p["msplit"] % p["mpx"] == 0 and p["ngroups"] % p["cgx"] == 0
            assert 1 <= p["mpx"] * p["cgx"] <= 32
            # no XCD carries more rounds of 32 workgroups than an even spread would need
            per_xcd = [sum(1 for i, t in enumerate(tiles) if i % 8 == x and t[0] != 0xFFFFFFFF) for x in range(8)]
            assert -(-max(per_xcd) // 32) == -(-(-(-len(real) // 8)) // 32), (M, N, K, p, per_xcd)
            # a rectangle lives on one XCD (workgroup id % 8) and its workgroups are dispatched
            # back to back there
            where = {}
            for i, (cg, ms) in enumerate(tiles):
                if cg != 0xFFFFFFFF:
                    where.setdefault((cg // p["cgx"], ms // p["mpx"]), []).append(i)
            for ids in where.values():
                assert len({i % 8 for i in ids}) == 1
                local = sorted(i // 8 for i in ids)
                assert local == list(range(local[0], local[0] + len(ids)))


def test_fused_gemm_tiling_avoids_a_nearly_empty_last_round(libmod):
    lib = libmod.load()
    # benchmark shape: one workgroup per compute unit, 4 x 8 rectangles, one per XCD
    p, _ = _tiling(lib, 4096, 4096)
    assert (p["ngroups"], p["msplit"], p["m_per_block"], p["mpx"], p["cgx"], p["grid"]) == (32, 8, 512, 4, 8, 256)
    # 96 column groups: three slices would give 288 workgroups = one full round + 32 stragglers
    p, _ = _tiling(lib, 12288, 12288)
    assert (p["ngroups"] * p["msplit"]) % 256 == 0
    # 24 column groups: 11 slices would be 264 workgroups; 10 fit one round
    p, _ = _tiling(lib, 5000, 3000)
    assert p["ngroups"] * p["msplit"] <= 256
    # other K: rejected before anything else
    import ctypes
    assert lib.mi_debug_fused_gemm_tiling(64, 64, 256, (ctypes.c_uint32 * 8)(), None, 0) != 0


def test_build_rejects_accumulation_register_writes_inside_an_mfma_loop():
    """The register-resident kernels name their B operand in the accumulation-register file from
    inline assembly; the build reads the generated ISA and fails if the compiler writes such a
    register after a kernel's first MFMA of that kind (a copy the matrix core may still be reading)."""
    import importlib
    build = importlib.import_module("6s894_project_2025_amd.build")
    good = """
_Zkernel_a: ; @_Zkernel_a
	v_accvgpr_write_b32 a0, v1
	;;#ASMSTART
	v_mfma_f32_16x16x4_f32 v[28:31], v32, a252, 0
	;;#ASMEND
	v_add_u32_e32 v1, v2, v3
	s_endpgm
.Lfunc_end0:
_Zkernel_b: ; @_Zkernel_b
	v_accvgpr_write_b32 a5, v1
	v_mfma_f32_16x16x32_bf16 v[0:3], v[8:11], a[4:7], v[0:3]
	s_endpgm
_Zplain: ; @_Zplain
	v_accvgpr_write_b32 a5, v1
	s_endpgm
"""
    assert build.check_register_resident_isa(good, "good") == 2
    bad = good.replace("v_add_u32_e32 v1, v2, v3", "v_accvgpr_write_b32 a63, v229")
    with pytest.raises(RuntimeError, match="_Zkernel_a writes an accumulation register"):
        build.check_register_resident_isa(bad, "bad")
    assert set(build.ISA_CHECKED) <= {os.path.basename(s) for s in build.sources()}


def test_build_rejects_early_reads_of_an_assembly_mfma_result():
    """The compiler does not know that the result of an inline-assembly MFMA arrives when it retires:
    the build follows every path from such an MFMA for a few issue slots and fails on an ordinary
    instruction that reads its destination there (a copy on a loop edge, say)."""
    import importlib
    build = importlib.import_module("6s894_project_2025_amd.build")
    head = "_Zk: ; @_Zk\n.LBB0_1:\n\tv_mfma_f32_16x16x32_bf16 v[32:35], v[96:99], a[124:127], v[32:35]\n"
    tail = "\ts_endpgm\n"
    filler = "\tv_add_u32_e32 v1, v2, v3\n"

    def check(body):
        return build.check_mfma_results_not_touched_early(head + body + tail, "t")

    # far enough away, behind enough idle cycles, or another MFMA accumulating into it: fine
    assert check(filler * build.kResultWaitStates + "\tv_mov_b32_e32 v100, v33\n") == 1
    assert check("\ts_nop 15\n\tv_mov_b32_e32 v100, v33\n") == 1
    assert check("\tv_mfma_f32_16x16x32_bf16 v[32:35], v[96:99], a[128:131], v[32:35]\n" + filler * 11) == 2
    # a register written anew is no longer the result; stores and LDS writes have no destination
    assert check("\tv_xor_b32 v32, 0x80, v180\n\tds_read_b128 v[64:67], v32 offset:0\n") == 1
    with pytest.raises(RuntimeError, match="reads the result"):
        check(filler * 3 + "\tv_mov_b64_e32 v[114:115], v[34:35]\n")
    with pytest.raises(RuntimeError, match="reads the result"):
        check("\tds_write_b128 v7, v[32:35] offset:1024\n")
    with pytest.raises(RuntimeError, match="reads the result"):
        check("\tglobal_store_dword v5, v33, s[2:3] nt\n")
    # branches are followed both ways
    with pytest.raises(RuntimeError, match="reads the result"):
        check("\ts_cbranch_vccnz .LBB0_9\n" + filler * 20 + ".LBB0_9:\n\tv_cvt_pk_bf16_f32 v9, v32, v33\n")
    with pytest.raises(RuntimeError, match="reads the result"):
        check("\ts_branch .LBB0_9\n" + "\ts_endpgm\n" + ".LBB0_9:\n\tv_cvt_pk_bf16_f32 v9, v32, v33\n")
    assert check("\ts_cbranch_vccnz .LBB0_9\n" + filler * 20 + ".LBB0_9:\n" + filler * 11 + "\tv_mov_b32_e32 v9, v32\n") == 1


def test_build_rejects_other_uses_of_m0():
    """The global -> LDS transfers take their LDS base from M0, set by an opaque statement; the
    build fails if anything else in such a file names M0."""
    import importlib
    build = importlib.import_module("6s894_project_2025_amd.build")
    good = ("_Zk: ; @_Zk\n\ts_add_i32 m0, s5, 0x8000\n\tv_mfma_f32_16x16x32_bf16 v[32:35], v[96:99], a[124:127], v[32:35]\n"
            "\tglobal_load_lds_dwordx4 v7, s[2:3]\n\ts_add_i32 m0, s5, 0x8400 ; comment mentioning m0\n\ts_endpgm\n")
    assert build.check_m0_is_the_transfers_alone(good, "good") == 2
    for other in ("\ts_mov_b32 m0, s9\n", "\ts_mov_b32 s9, m0\n", "\tv_readlane_b32 s4, v3, m0\n"):
        with pytest.raises(RuntimeError, match="uses M0"):
            build.check_m0_is_the_transfers_alone(good.replace("\ts_endpgm\n", other + "\ts_endpgm\n"), "bad")


def test_build_rejects_uses_of_an_lds_read_before_its_wait():
    """An LDS read written as an opaque statement returns a register that holds nothing until a
    hand-placed s_waitcnt lgkmcnt covers it; the build follows every path from each ds_read and fails
    on an instruction that reads or overwrites the destination first (a register copy the allocator
    puts on the edge between two variants of a loop body, say)."""
    import importlib
    build = importlib.import_module("6s894_project_2025_amd.build")
    head = "_Zk: ; @_Zk\n.LBB0_1:\n\tds_read_b128 v[112:115], v128 offset:0\n"
    tail = "\ts_endpgm\n"
    mfma = "\tv_mfma_f32_16x16x32_bf16 v[32:35], v[96:99], a[124:127], v[32:35]\n"
    younger = "\tds_read_b128 v[116:119], v128 offset:0x2000\n"

    def check(body):
        return build.check_lds_reads_waited_for(head + body + tail, "t")

    # waited for, then used; a wait that allows as many outstanding operations as are younger covers it
    assert check(mfma * 4 + "\ts_waitcnt lgkmcnt(0)\n\tv_mov_b64_e32 v[76:77], v[112:113]\n") == 1
    assert check(younger + "\ts_waitcnt lgkmcnt(1)\n\tv_mfma_f32_16x16x32_bf16 v[32:35], v[112:115], a[0:3], v[32:35]\n"
                 "\ts_waitcnt lgkmcnt(0)\n") == 2
    assert check("\ts_waitcnt vmcnt(8) lgkmcnt(0)\n\tv_mov_b32_e32 v1, v112\n") == 1
    # never used on this path: nothing to complain about
    assert check(mfma * 3) == 1
    # used, or overwritten, before any wait, or behind one that does not reach back far enough
    with pytest.raises(RuntimeError, match="touches the destination"):
        check(mfma * 4 + "\tv_mov_b64_e32 v[76:77], v[112:113]\n")
    with pytest.raises(RuntimeError, match="touches the destination"):
        check("\tv_mfma_f32_16x16x32_bf16 v[32:35], v[112:115], a[0:3], v[32:35]\n")
    with pytest.raises(RuntimeError, match="touches the destination"):
        check("\tv_mov_b32_e32 v113, v5\n")
    with pytest.raises(RuntimeError, match="touches the destination"):
        check(younger + "\ts_waitcnt lgkmcnt(2)\n\tv_mov_b32_e32 v1, v112\n")
    with pytest.raises(RuntimeError, match="touches the destination"):
        check("\ts_waitcnt vmcnt(0)\n\tds_write_b128 v7, v[112:115] offset:1024\n")
    # branches are followed both ways: the copy sits on an edge that skips the wait
    with pytest.raises(RuntimeError, match="touches the destination"):
        check("\ts_cbranch_vccnz .LBB0_9\n\ts_waitcnt lgkmcnt(0)\n\ts_endpgm\n.LBB0_9:\n\tv_mov_b64_e32 v[76:77], v[112:113]\n")
    assert check("\ts_waitcnt lgkmcnt(0)\n\ts_cbranch_vccnz .LBB0_9\n\ts_endpgm\n.LBB0_9:\n\tv_mov_b64_e32 v[76:77], v[112:113]\n") == 1


def test_build_rejects_overwriting_an_assembly_mfma_operand_too_soon():
    """The matrix core reads an MFMA's A operand over several cycles after issue; for an inline-assembly
    MFMA the compiler adds no wait states, so the build fails on a vector instruction that writes
    one of those registers within a few issue slots (a register copy right behind the MFMA, say)."""
    import importlib
    build = importlib.import_module("6s894_project_2025_amd.build")
    head = "_Zk: ; @_Zk\n.LBB0_1:\n\tv_mfma_f32_16x16x32_bf16 v[32:35], v[96:99], a[124:127], v[32:35]\n"
    tail = "\ts_endpgm\n"
    filler = "\tv_add_u32_e32 v1, v2, v3\n"

    def check(body):
        return build.check_mfma_operands_not_overwritten_early(head + body + tail, "t")

    # late enough, or not a vector ALU write (a load's data arrives much later; a read is harmless)
    assert check(filler * build.kOperandReadSlots + "\tv_mov_b32_e32 v97, v5\n") == 1
    assert check("\tds_read_b128 v[96:99], v128 offset:0\n") == 1
    assert check("\tv_mov_b32_e32 v5, v97\n") == 1
    assert check("\ts_nop 3\n\tv_mov_b32_e32 v97, v5\n") == 1
    with pytest.raises(RuntimeError, match="overwrites the A operand"):
        check("\tv_mov_b32_e32 v97, v5\n")
    with pytest.raises(RuntimeError, match="overwrites the A operand"):
        check(filler * 2 + "\tv_cvt_pk_bf16_f32 v99, v1, v2\n")
    with pytest.raises(RuntimeError, match="overwrites the A operand"):
        check("\ts_cbranch_vccnz .LBB0_9\n" + filler * 10 + ".LBB0_9:\n\tv_mov_b64_e32 v[98:99], v[4:5]\n")
