"""The compile-time LDS pattern check (csrc/lds_layout.hpp) accepts a swizzled layout and rejects the
same layout without the swizzle: compiled on the host with g++, no GPU.  The kernels apply the check
to their own address functions in static_asserts, so a bad swizzle fails the library build; this
test pins the checker itself (analogue of the reference's static layout checks,
csrc/frag.cuh:94-160)."""

import os
import subprocess
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "6s894_project_2025_amd", "csrc")

SNIPPET = r"""
#include "lds_layout.hpp"
// [64 rows][512 B]; lane (hi, lo) reads row lo, 16-byte chunk hi
constexpr uint32_t swizzled(uint32_t lane) { return (lane & 15u) * 512u + (((lane >> 4) ^ (lane & 15u)) << 4); }
constexpr uint32_t plain(uint32_t lane) { return (lane & 15u) * 512u + ((lane >> 4) << 4); }
constexpr uint32_t contiguous(uint32_t lane) { return 16u * lane; }
constexpr uint32_t misaligned(uint32_t lane) { return 16u * lane + 4u; }
static_assert(mi::lds::conflict_free_b128(swizzled), "swizzled");
static_assert(mi::lds::conflict_free_b128(contiguous), "contiguous");
#ifdef EXPECT_FAIL_PLAIN
static_assert(mi::lds::conflict_free_b128(plain), "plain rows collide");
#endif
#ifdef EXPECT_FAIL_MISALIGNED
static_assert(mi::lds::conflict_free_b128(misaligned), "not one 16-byte access");
#endif
int main() { return 0; }
"""


def _compile(defines):
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "t.cpp")
        with open(src, "w") as f:
            f.write(SNIPPET)
        cmd = ["g++", "-std=c++17", "-fsyntax-only", "-I", CSRC] + [f"-D{x}" for x in defines] + [src]
        return subprocess.run(cmd, capture_output=True, text=True)


def test_checker_accepts_conflict_free_patterns():
    r = _compile([])
    assert r.returncode == 0, r.stderr


def test_checker_rejects_unswizzled_rows_and_misaligned_pieces():
    r = _compile(["EXPECT_FAIL_PLAIN"])
    assert r.returncode != 0 and "plain rows collide" in r.stderr
    r = _compile(["EXPECT_FAIL_MISALIGNED"])
    assert r.returncode != 0 and "not one 16-byte access" in r.stderr


def test_kernels_apply_the_checker_to_their_own_layouts():
    for name in ("xreg_common.hpp", "fused_gemm.hip", "fp8_gemm.hip"):
        text = open(os.path.join(CSRC, name)).read()
        assert "lds::conflict_free_b128" in text and "static_assert" in text, name
