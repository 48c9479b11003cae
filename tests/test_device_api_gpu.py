"""The device-side embedding API (csrc/hadamard_device.hpp), exercised through the minimal kernel
behind mi_debug_device_fwht: every length 1..32768 and element type against the fp64 oracle at the
same tolerances as the stand-alone op, in place and out of place, and bit-identical to mi_fwht
(both are callers of the same device functions).  Counterpart of testing the reference's
hadamard_transform_device through its thin kernel (csrc/main.cu:42-53)."""
from importlib import import_module

import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}
CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


@pytest.fixture(scope="module")
def lib(pkg):
    return import_module(pkg.__name__ + "._lib").load()


def _call(lib, x, out, n, scale):
    rows = x.numel() // n
    st = lib.mi_debug_device_fwht(x.data_ptr(), out.data_ptr(), rows, n, CODE[x.dtype], scale,
                                  torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return st


@pytest.mark.parametrize("dtype", list(TOL))
@pytest.mark.parametrize("p", range(0, 16))
def test_device_api_matches_oracle_and_op(pkg, oracle, lib, p, dtype):
    n = 1 << p
    n_rows = max(1, 512 // n)
    rows = n_rows * (5 if p <= 12 else 3)
    g = torch.Generator().manual_seed(100 + p)
    x_cpu = torch.randn(rows, n, generator=g).to(dtype)
    for scale in (2.0 ** -((p + 1) // 2), 0.37):
        x = x_cpu.cuda()
        out = torch.empty_like(x)
        assert _call(lib, x, out, n, scale) == 0
        y64 = oracle.fwht_f64(x_cpu.to(torch.float64).numpy(), scale)
        err = oracle.rel_err(out.cpu().to(torch.float64).numpy(), y64)
        assert err <= TOL[dtype], f"n={n} {dtype} scale={scale}: {err}"
        if scale != 0.37:
            # power-of-two factors are folded into the matrix-core operands: both callers of the
            # device functions then produce the same bits.  With a residual multiplier the compiler
            # may round fp32 -> 16 bit once (fused multiply-convert) or twice per kernel, so only
            # the tolerance above applies.
            assert torch.equal(out, pkg.hadamard_transform(x, scale))
        # in place
        assert _call(lib, x, x, n, scale) == 0
        assert torch.equal(x, out)


def test_device_api_row_multiple_contract(lib):
    x = torch.zeros(3, 64, dtype=torch.bfloat16, device="cuda")  # N_ROWS = 8 for n = 64
    assert _call(lib, x, x, 64, 1.0) == -5
    x = torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda")
    assert _call(lib, x, x, 64, 1.0) == 0
    assert lib.mi_debug_device_fwht(x.data_ptr(), x.data_ptr(), 8, 48, 1, 1.0, None) == -2
