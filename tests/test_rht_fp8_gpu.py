"""GPU parity of the randomized-Hadamard FP8 quantize epilogue and the FP8 GEMM.

The reference has no FP8 path, so parity here is against the oracle's stated convention:
codes and scales are bit-exact given identical pre-quant values (the kernel's own bf16 y, which
is itself checked against the fp64 oracle at the bf16 tolerance and against the stand-alone
transform bit for bit)."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _bf16_to_f32_np(t):
    return t.cpu().to(torch.float32).numpy()


@pytest.mark.parametrize("T,n", [(8, 16), (33, 64), (40, 256), (17, 512), (9, 1024), (21, 2048),
                                 (64, 4096), (1, 4096)])
def test_quant_bit_exact_given_prequant(pkg, oracle, T, n):
    x, sign = oracle.inputs_rht(T, n)
    q, rs, y = pkg.rht_quant_fp8(x.cuda(), sign, return_prequant=True)
    torch.cuda.synchronize()
    # pre-quant values: within bf16 tolerance of the fp64 randomized transform
    y64 = oracle.rht_f64(x.to(torch.float32).numpy(), sign.numpy())
    assert oracle.rel_err(_bf16_to_f32_np(y), y64) <= 2e-2
    # and bit-identical to the stand-alone op applied to sign * x
    xs = (x.to(torch.float32) * sign.to(torch.float32)[None, :]).to(torch.bfloat16)
    y_op = pkg.hadamard_transform(xs.cuda())
    assert torch.equal(y_op.view(torch.int16), y.view(torch.int16))
    # codes and scales bit-exact against the oracle on those values
    want_q, want_s = oracle.quant_fp8_rows(_bf16_to_f32_np(y))
    got_q = q.view(torch.uint8).cpu().numpy()
    assert np.array_equal(rs.cpu().numpy().view(np.uint32), want_s.view(np.uint32))
    assert np.array_equal(got_q, want_q), f"{(got_q != want_q).sum()} code mismatches"


def test_quant_zero_row_and_outliers(pkg, oracle):
    x, sign = oracle.inputs_rht(8, 512)
    x[3] = 0
    q, rs, y = pkg.rht_quant_fp8(x.cuda(), sign, return_prequant=True)
    want_q, want_s = oracle.quant_fp8_rows(_bf16_to_f32_np(y))
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), want_q)
    assert np.array_equal(rs.cpu().numpy(), want_s)
    assert (q.view(torch.uint8)[3] == 0).all()
    # the rotation spreads outlier channels: dequantised values track y
    deq = q.float() * rs[:, None]
    assert ((deq - y.float()).abs().max() / y.float().abs().max()).item() < 0.07


def test_quant_full_size_config(pkg, oracle):
    # benchmark configuration 5 activations [8192, 4096]; property checks on the device + sampled rows
    x, sign = oracle.inputs_rht(8192, 4096)
    q, rs, y = pkg.rht_quant_fp8(x.cuda(), sign, return_prequant=True)
    torch.cuda.synchronize()
    idx = [0, 1, 4095, 4096, 8191]
    want_q, want_s = oracle.quant_fp8_rows(_bf16_to_f32_np(y[idx]))
    assert np.array_equal(q.view(torch.uint8)[idx].cpu().numpy(), want_q)
    assert np.array_equal(rs[idx].cpu().numpy(), want_s)
    y64 = oracle.rht_f64(x[idx].to(torch.float32).numpy(), sign.numpy())
    assert oracle.rel_err(_bf16_to_f32_np(y[idx]), y64) <= 2e-2
    # every row uses the top code somewhere (amax maps to +-448) and no NaN code appears
    codes = q.view(torch.uint8)
    assert ((codes & 0x7F) == 0x7E).any(dim=1).all()
    assert not ((codes & 0x7F) == 0x7F).any()


@pytest.mark.parametrize("T,N,K", [(16, 16, 128), (100, 70, 256), (256, 384, 512), (130, 129, 1024),
                                   (16, 16, 384), (600, 520, 640)])
def test_fp8_gemm_against_dequantised_product(pkg, oracle, T, N, K):
    g = torch.Generator().manual_seed(5)
    a = torch.randn(T, K, generator=g)
    b = torch.randn(N, K, generator=g) * 0.02
    qa, sa = oracle.quant_fp8_rows(a.numpy())
    qb, sb = oracle.quant_fp8_rows(b.numpy())
    out = pkg.fp8_gemm_rowscale(torch.from_numpy(qa).cuda().view(torch.float8_e4m3fn),
                                torch.from_numpy(sa).cuda(),
                                torch.from_numpy(qb).cuda().view(torch.float8_e4m3fn),
                                torch.from_numpy(sb).cuda())
    torch.cuda.synchronize()
    da = oracle.e4m3fn_decode(qa).astype(np.float64) * sa[:, None].astype(np.float64)
    db = oracle.e4m3fn_decode(qb).astype(np.float64) * sb[:, None].astype(np.float64)
    want = da @ db.T
    assert oracle.rel_err(out.cpu().double().numpy(), want) <= 2e-2


def test_fp8_gemm_full_size_sampled_rows(pkg, oracle):
    # the benchmark shape (T = 8192, N = 14336, K = 4096): 48 sampled rows of the output against
    # the oracle's dequantised fp64 product; every tile row and every column tile is touched
    T, N, K = 8192, 14336, 4096
    g = torch.Generator().manual_seed(9)
    qa = torch.randint(0, 0x7E, (T, K), generator=g, dtype=torch.uint8)
    qa |= (torch.randint(0, 2, (T, K), generator=g, dtype=torch.uint8) << 7)
    qb = torch.randint(0, 0x7E, (N, K), generator=g, dtype=torch.uint8)
    qb |= (torch.randint(0, 2, (N, K), generator=g, dtype=torch.uint8) << 7)
    sa = torch.rand(T, generator=g) * 1e-2 + 1e-3
    sb = torch.rand(N, generator=g) * 1e-2 + 1e-3
    out = pkg.fp8_gemm_rowscale(qa.cuda().view(torch.float8_e4m3fn), sa.cuda(),
                                qb.cuda().view(torch.float8_e4m3fn), sb.cuda())
    torch.cuda.synchronize()
    rows = torch.cat([torch.arange(0, T, 256) + torch.randint(0, 256, (T // 256,), generator=g),
                      torch.tensor([0, 255, 256, T - 1]), torch.randint(0, T, (12,), generator=g)])
    da = oracle.e4m3fn_decode(qa[rows].numpy()).astype(np.float64) * sa[rows, None].double().numpy()
    db = oracle.e4m3fn_decode(qb.numpy()).astype(np.float64) * sb[:, None].double().numpy()
    want = da @ db.T
    got = out[rows.cuda()].cpu().double().numpy()
    assert oracle.rel_err(got, want) <= 2e-2


def test_rht_fp8_linear_end_to_end(pkg, oracle):
    # config 5 in miniature: y = RHT(x) -> fp8, w rotated the same way -> fp8, product -> bf16;
    # compared with the unquantised x @ w.T (the rotation is orthogonal, so it cancels)
    T, n, N = 256, 1024, 192
    x, sign = oracle.inputs_rht(T, n)
    g = torch.Generator().manual_seed(1)
    w = (torch.randn(N, n, generator=g) * 0.02).to(torch.bfloat16)
    qx, sx = pkg.rht_quant_fp8(x.cuda(), sign)
    qw, sw = pkg.rht_quant_fp8(w.cuda(), sign)
    out = pkg.fp8_gemm_rowscale(qx, sx, qw, sw)
    want = x.double() @ w.double().t()
    err = (out.cpu().double() - want).abs().max().item() / want.abs().max().item()
    assert err < 0.1


def test_fp8_gemm_wrapper_validates_operands(pkg):
    qa = torch.zeros(16, 128, dtype=torch.uint8, device="cuda")
    qb = torch.zeros(24, 128, dtype=torch.uint8, device="cuda")
    sa = torch.ones(16, device="cuda")
    sb = torch.ones(24, device="cuda")
    with pytest.raises(RuntimeError, match="scale lengths"):
        pkg.fp8_gemm_rowscale(qa, sa[:15], qb, sb)
    with pytest.raises(RuntimeError, match="scale lengths"):
        pkg.fp8_gemm_rowscale(qa, sa, qb, sb[:1])
    with pytest.raises(RuntimeError, match="one-byte"):
        pkg.fp8_gemm_rowscale(qa.to(torch.int16), sa, qb, sb)
    # scales handed over on the host are moved to the device, not dereferenced there
    out = pkg.fp8_gemm_rowscale(qa, sa.cpu(), qb, sb.cpu().view(1, -1))
    torch.cuda.synchronize()
    assert out.shape == (16, 24) and out.abs().max().item() == 0.0
