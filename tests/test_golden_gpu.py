"""The HIP kernels against the committed fixtures, through the C ABI."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hadamard_fixtures.npz")


@pytest.fixture(scope="module")
def fix():
    return np.load(FIX, allow_pickle=False)


@pytest.mark.parametrize("dt,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2), (torch.float16, 2e-2)], ids=str)
def test_fwht_fixture(pkg, oracle, fix, dt, tol):
    for n in (2, 16, 256, 1024):
        x = torch.from_numpy(fix[f"fwht_x_{n}"]).to(dt).cuda()
        y = pkg.hadamard_transform(x)
        assert oracle.rel_err(y.cpu().double().numpy(), fix[f"fwht_y_{n}"]) <= tol


def test_fused_fixtures(pkg, oracle, fix):
    Y = pkg.fused_ht_gemv(torch.from_numpy(fix["gemv_W"]).float().cuda(),
                          torch.from_numpy(fix["gemv_X"]).float().cuda(), 1.0)
    # the reference's own bar for this shape: 1e-3 absolute (fused_ht/fwht_gemv_fusion.cu:293)
    assert np.abs(Y.cpu().double().numpy() - fix["gemv_Y"]).max() < 1e-3
    assert oracle.rel_err(Y.cpu().double().numpy(), fix["gemv_Y"]) <= 1e-5
    for dt, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        C = pkg.fused_ht_gemm(torch.from_numpy(fix["gemm_W"]).to(dt).cuda(),
                              torch.from_numpy(fix["gemm_Xt"]).to(dt).cuda(), 1.0,
                              out_dtype=torch.float32)
        assert oracle.rel_err(C.cpu().double().numpy(), fix["gemm_C"]) <= tol


def test_fp8_fixture_codes(pkg, fix):
    from importlib import import_module
    lib = import_module(pkg.__name__ + "._lib").load()
    v = torch.from_numpy(fix["fp8_values"]).cuda()
    out = torch.empty(v.numel(), dtype=torch.uint8, device="cuda")
    assert lib.mi_debug_convert(2, v.data_ptr(), out.data_ptr(), v.numel(), None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), fix["fp8_codes"])
