"""GPU parity of the fused products against the fp64 oracle, through the C ABI.

Bars: fp32 <= 1e-5, bf16/fp16 <= 2e-2 on max|c - c64| / max|c64| (build contract), plus the
reference's own self-check, fused == unfused within 1e-3 absolute at its three GEMV shapes
(fused_ht/fwht_gemv_fusion.cu:293,632-634) and at the pipelined shape (fusion_pipelined.cu:694-700).
"""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _rel(oracle, got, want64):
    return oracle.rel_err(got.cpu().to(torch.float64).numpy(), want64)


@pytest.mark.parametrize("M,N,B", [(32, 64, 8), (64, 128, 16), (128, 256, 32), (256, 256, 512),
                                   (5, 16, 3), (100, 32, 17), (33, 2, 5), (7, 4, 40), (19, 8, 16),
                                   (130, 2048, 24), (1024, 1024, 8), (1024, 1024, 64)])
def test_gemv_against_oracle(pkg, oracle, M, N, B):
    W, X = oracle.inputs_gemv(M, N, B)
    for scale in (None, 1.0):
        s = 1.0 / math.sqrt(N) if scale is None else scale
        Y = pkg.fused_ht_gemv(W.cuda(), X.cuda(), scale)
        torch.cuda.synchronize()
        want = oracle.fused_ht_gemv_f64_blas(W.double().numpy(), X.double().numpy(), s)
        assert Y.shape == (M, B)
        assert _rel(oracle, Y, want) <= 1e-5, (M, N, B, scale)


@pytest.mark.parametrize("M,N,B", [(32, 64, 8), (64, 128, 16), (128, 256, 32)])
def test_gemv_reference_self_check(pkg, oracle, M, N, B):
    # reference harness: uniform [-1,1] inputs, unnormalised, fused vs (transform, then GEMM)
    g = torch.Generator().manual_seed(42)
    W = (torch.rand(M, N, generator=g) * 2 - 1).cuda()
    X = (torch.rand(N, B, generator=g) * 2 - 1).cuda()
    fused = pkg.fused_ht_gemv(W, X, 1.0)
    RX = pkg.hadamard_transform(X.t().contiguous(), 1.0).t().contiguous()  # transform down dim 0
    unfused = W.double() @ RX.double()
    assert (fused.double() - unfused).abs().max().item() < 1e-3
    want = oracle.fused_ht_gemv_f64(W.cpu().double().numpy(), X.cpu().double().numpy(), 1.0)
    assert np.abs(fused.cpu().double().numpy() - want).max() < 1e-3


# Launch paths that only larger problems reach: the 64-row workgroup variant (column groups x
# 64-row blocks >= 256; the benchmark's M=N=1024 with B=256 and B=512, the shapes of
# fused_ht/fwht_gemv_fusion.cu:643-653) and a workgroup that walks several row blocks with one
# transformed tile (more row blocks than workgroup rows in the grid).  (The 32-row variant runs
# between 128 and 255 such groups: (1024, 1024, 128) here and (256, 256, 512) above; everything
# smaller runs 16-row workgroups.)
# N >= 512 on shapes with a 64-row, 16-column workgroup for every compute unit run the kernels that
# keep the transformed columns in registers and stream W through LDS.  N = 512 and 1024 (every
# wavefront all of K, 16 rows of a block each): (1024, 1024, 256) and (64, 1024, 4096) with one row
# block per workgroup (the stream ends with its first block), (1024, 1024, 512), (1024, 1024, 2048)
# and (512, 512, 1024) with two to eight (each block requests the first stages of the next),
# (1000, 512, 700) with a ragged last row block and a last column group of 12, (1100, 1024, 531) with
# a row length that rules out 16-byte loads of X, (4100, 1024, 130) with a last column group of two
# and a last block of four rows, (8192, 512, 40) with a long walk over row blocks.  N = 2048 (the
# wavefronts split K, sums meet in LDS): (2048, 2048, 512), (1100, 2048, 531), (4100, 2048, 130),
# (300, 2048, 1024) with a second row block that is the last and ragged, (20000, 2048, 24) with three
# blocks per workgroup, (16384, 2048, 16) with one column group.  N = 256 from 128 pairs of 64 columns
# x 64 rows on runs the row-split kernel with 64 columns per workgroup (two columns per 512-element
# tile of the transform): (4096, 256, 4096), (1000, 256, 1100) ragged both ways, (130, 256, 9000) with
# more column groups than row blocks, (8192, 256, 100) with two column groups, the second of 36
# columns, (512, 256, 1024) right at the threshold.
@pytest.mark.parametrize("M,N,B", [(1024, 1024, 256), (1024, 1024, 512), (1024, 1024, 128),
                                   (4096, 256, 4096), (2000, 64, 1000), (4100, 2048, 130),
                                   (1024, 1024, 2048), (1000, 512, 700), (1100, 1024, 531),
                                   (2048, 2048, 512), (1100, 2048, 531), (300, 2048, 1024),
                                   (20000, 2048, 24), (8192, 512, 40), (16384, 2048, 16),
                                   (512, 512, 1024), (64, 1024, 4096), (4100, 1024, 130),
                                   (1000, 256, 1100), (130, 256, 9000), (8192, 256, 100), (512, 256, 1024)])
def test_gemv_large_launch_paths(pkg, oracle, M, N, B):
    W, X = oracle.inputs_gemv(M, N, B)
    Y = pkg.fused_ht_gemv(W.cuda(), X.cuda())
    torch.cuda.synchronize()
    assert Y.shape == (M, B)
    # every row block boundary of the 64-row variant, first/last rows, and a random sample
    g = torch.Generator().manual_seed(7)
    rows = torch.unique(torch.cat([torch.tensor([0, 1, 63, 64, 65, 127, 128, M // 2, M - 65, M - 64,
                                                 M - 2, M - 1]).clamp(0, M - 1),
                                   torch.randint(0, M, (52,), generator=g)]))
    want = oracle.fused_ht_gemv_f64_blas(W[rows].double().numpy(), X.double().numpy(),
                                         1.0 / math.sqrt(N))
    assert _rel(oracle, Y[rows.cuda()], want) <= 1e-5, (M, N, B)
    # size-independent: column sums of Y equal (column sums of W) . H(X)
    colsum = oracle.fused_ht_gemv_f64_blas(W.double().sum(0, keepdim=True).numpy(),
                                           X.double().numpy(), 1.0 / math.sqrt(N))
    got = Y.double().sum(0, keepdim=True).cpu().numpy()
    assert np.abs(got - colsum).max() / np.abs(colsum).max() <= 1e-5


def test_gemv_random_shapes(pkg, oracle):
    # seeded sweep over the launch logic: every power of two N, row counts around the 16/32/64-row
    # block sizes, batches around the 16- and 32-column tiles (whole, ragged, not a multiple of four)
    rng = np.random.default_rng(20251125)
    for _ in range(48):
        N = 1 << int(rng.integers(1, 12))
        M = int(rng.choice([1, 15, 16, 17, 31, 33, 63, 64, 65, 100, 129, 300, 777, 1024, 1500]))
        B = int(rng.choice([1, 3, 4, 7, 16, 17, 20, 31, 32, 33, 48, 61, 64, 100, 255, 260, 600]))
        if N >= 1024 and M * B > 400000:
            M = 129
        W, X = oracle.inputs_gemv(M, N, B)
        Y = pkg.fused_ht_gemv(W.cuda(), X.cuda())
        torch.cuda.synchronize()
        want = oracle.fused_ht_gemv_f64_blas(W.double().numpy(), X.double().numpy(), 1.0 / math.sqrt(N))
        assert Y.shape == (M, B)
        assert _rel(oracle, Y, want) <= 1e-5, (M, N, B)


def test_gemv_random_large_shapes(pkg, oracle):
    # seeded sweep over the kernels that serve N >= 512 once column groups x 64-row blocks reach 256
    # (rows split over the wavefronts for N = 512 and 1024, K split for N = 2048) and over the launch
    # plan around that threshold: ragged row and column counts, one to many row blocks per workgroup,
    # more column groups than one round of workgroups.  Checked on sampled rows and by column sums.
    rng = np.random.default_rng(20251126)
    g = torch.Generator().manual_seed(11)
    for _ in range(32):
        N = int(rng.choice([256, 512, 1024, 2048]))
        M = int(rng.choice([64, 65, 127, 200, 256, 300, 513, 1000, 1024, 1500, 2048, 3000, 5000]))
        B = int(rng.choice([16, 17, 33, 64, 100, 255, 256, 260, 511, 528, 1000, 1024, 2049, 4100]))
        if M * B > 6_000_000:
            B = 528
        W, X = oracle.inputs_gemv(M, N, B)
        Y = pkg.fused_ht_gemv(W.cuda(), X.cuda())
        torch.cuda.synchronize()
        assert Y.shape == (M, B)
        rows = torch.unique(torch.cat([torch.tensor([0, M // 2, M - 1]), torch.randint(0, M, (29,), generator=g)]))
        want = oracle.fused_ht_gemv_f64_blas(W[rows].double().numpy(), X.double().numpy(), 1.0 / math.sqrt(N))
        assert _rel(oracle, Y[rows.cuda()], want) <= 1e-5, (M, N, B)
        colsum = oracle.fused_ht_gemv_f64_blas(W.double().sum(0, keepdim=True).numpy(), X.double().numpy(),
                                               1.0 / math.sqrt(N))
        got = Y.double().sum(0, keepdim=True).cpu().numpy()
        assert np.abs(got - colsum).max() / np.abs(colsum).max() <= 1e-5, (M, N, B)


@pytest.mark.parametrize("M,N", [(1_100_000, 1024), (550_000, 2048)])
def test_gemv_w_beyond_4_gib(pkg, oracle, M, N):
    # W of 4.5 GB: byte offsets into W pass 2^32 (the streaming kernels address a row block with a
    # 64-bit base and 32-bit offsets inside it); rows on both sides of the 4 GiB line and the last ones
    B = 16
    g = torch.Generator(device="cuda").manual_seed(3)
    W = torch.randn(M, N, generator=g, device="cuda")
    X = torch.randn(N, B, generator=g, device="cuda")
    Y = pkg.fused_ht_gemv(W, X)
    torch.cuda.synchronize()
    line = (1 << 32) // (4 * N)                      # the first row that starts at or beyond 4 GiB
    rows = torch.tensor([0, 1, 63, 64, line - 65, line - 1, line, line + 1, line + 64, M - 65, M - 64, M - 1])
    want = oracle.fused_ht_gemv_f64_blas(W[rows.cuda()].cpu().double().numpy(), X.cpu().double().numpy(),
                                         1.0 / math.sqrt(N))
    assert _rel(oracle, Y[rows.cuda()], want) <= 1e-5
    # every row: Y against the product with the library's own transform, in slices
    T = pkg.hadamard_transform(X.t().contiguous()).t().contiguous()
    worst = 0.0
    for r0 in range(0, M, 200_000):
        ref = W[r0:r0 + 200_000] @ T
        worst = max(worst, (Y[r0:r0 + 200_000] - ref).abs().max().item())
    assert worst / math.sqrt(N) <= 1e-4, worst          # (fp32 against fp32: summation orders differ)


@pytest.mark.parametrize("M,N,B", [(1, 1024, 4096), (1, 2048, 4096), (1, 256, 8192), (3, 512, 4100), (17, 2048, 4097)])
def test_gemv_few_rows_many_columns(pkg, oracle, M, N, B):
    # the large-shape kernels with less than one 16-row fragment of W: every wavefront's rows past
    # the end are clamped to the last row for the loads and masked at the store
    W, X = oracle.inputs_gemv(M, N, B)
    Y = pkg.fused_ht_gemv(W.cuda(), X.cuda())
    torch.cuda.synchronize()
    want = oracle.fused_ht_gemv_f64_blas(W.double().numpy(), X.double().numpy(), 1.0 / math.sqrt(N))
    assert Y.shape == (M, B)
    assert _rel(oracle, Y, want) <= 1e-5


def test_gemv_identity_reduces_to_transform(pkg, oracle):
    N, B = 256, 48
    _, X = oracle.inputs_gemv(N, N, B)
    Y = pkg.fused_ht_gemv(torch.eye(N).cuda(), X.cuda())
    want = oracle.fwht_f64(X.double().numpy().T).T
    assert _rel(oracle, Y, want) <= 1e-5


GEMM_SHAPES = [(8, 12, 32), (33, 7, 64), (64, 64, 128), (70, 130, 256), (256, 192, 512),
               (300, 100, 1024), (96, 40, 2048), (80, 24, 4096), (1100, 50, 4096), (1024, 256, 1024)]


@pytest.mark.parametrize("dt,tol", [(torch.bfloat16, 2e-2), (torch.float16, 2e-2), (torch.float32, 1e-5)],
                         ids=["bf16", "f16", "f32"])
@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_against_oracle(pkg, oracle, M, N, K, dt, tol):
    W, Xt = oracle.inputs_gemm(M, N, K, dt)
    for scale in (None, 1.0):
        if dt == torch.float16 and scale == 1.0 and K >= 1024:
            continue  # unnormalised fp16 overflows the storage range by construction
        s = 1.0 / math.sqrt(K) if scale is None else scale
        C = pkg.fused_ht_gemm(W.cuda(), Xt.cuda(), scale, out_dtype=torch.float32)
        torch.cuda.synchronize()
        want = oracle.fused_ht_gemm_f64_blas(W.double().numpy(), Xt.double().numpy(), s)
        assert C.shape == (M, N)
        assert _rel(oracle, C, want) <= tol, (M, N, K, dt, scale)
    if dt != torch.float32:
        C16 = pkg.fused_ht_gemm(W.cuda(), Xt.cuda())
        assert C16.dtype == dt
        want = oracle.fused_ht_gemm_f64_blas(W.double().numpy(), Xt.double().numpy(), 1.0 / math.sqrt(K))
        assert _rel(oracle, C16, want) <= tol


# K = 512 ... 4096 run the register-resident kernels (K = 2048 its own, with K split over wavefront
# pairs; K = 4096 the same kernel in two passes, the second adding to what the first stored): groups
# of 131072 / K columns (64 at K = 4096), 64-row blocks, results stored while the next row block is
# multiplied or (K = 512) right after it.
# Shapes around every tile boundary, a single row block, N not a multiple of the columns a lane
# stores together (no vector stores), a scale that is not a power of two (separate store path),
# both 16-bit types and both output types.
@pytest.mark.parametrize("K", [1024, 512, 2048, 4096])
@pytest.mark.parametrize("M,N", [(1, 1), (63, 127), (64, 128), (65, 129), (128, 256), (129, 257),
                                 (577, 1333), (130, 2000), (4096, 130), (700, 4095), (200, 514)])
def test_gemm_k1024_tile_boundaries(pkg, oracle, M, N, K):
    for dt in (torch.bfloat16, torch.float16):
        W, Xt = oracle.inputs_gemm(M, N, K, dt)
        for scale, od in ((None, torch.float32), (None, dt), (0.37 / 32.0, torch.float32),
                          (1.0, torch.float32), (1.0 / 64.0, dt)):
            if dt == torch.float16 and scale == 1.0:
                continue  # unnormalised fp16 overflows the storage range by construction
            s = 1.0 / math.sqrt(K) if scale is None else scale
            C = pkg.fused_ht_gemm(W.cuda(), Xt.cuda(), scale, out_dtype=od)
            torch.cuda.synchronize()
            want = oracle.fused_ht_gemm_f64_blas(W.double().numpy(), Xt.double().numpy(), s)
            assert C.shape == (M, N) and C.dtype == od
            # error against the larger of max|C| and the typical magnitude of an output (s K for
            # unit-variance inputs): a 1 x 1 result can be small by chance
            err = np.abs(C.cpu().double().numpy() - want).max() / max(np.abs(want).max(), s * K)
            assert err <= 2e-2, (M, N, K, dt, scale, od)


@pytest.mark.parametrize("K", [1024, 512, 2048, 4096])
def test_gemm_k1024_every_output_written_once(pkg, oracle, K):
    # size-independent check on the full benchmark shape, both output types: C against the
    # unfused product computed on the device from the library's own transform, every element
    M = N = 4096
    s2 = {512: 1.0 / 16.0, 1024: 1.0 / 32.0, 2048: 1.0 / 32.0, 4096: 1.0 / 64.0}[K]   # a power of two
    W, Xt = oracle.inputs_gemm(M, N, K, torch.bfloat16)
    Wd, Xd = W.cuda(), Xt.cuda()
    Y = pkg.hadamard_transform(Xd, s2)                  # bf16, same rounding as the fused operand
    ref = Wd.float() @ Y.float().t()
    scale = ref.abs().max().item()
    for od in (torch.bfloat16, torch.float32):
        for _ in range(3):                               # back-to-back launches reuse LDS and registers
            C = pkg.fused_ht_gemm(Wd, Xd, s2, out_dtype=od)
        torch.cuda.synchronize()
        err = (C.float() - ref).abs().max().item() / scale
        # K = 4096 forms x[0:2048] +- x[2048:4096] inside the first matrix-core stage, so its 16-bit
        # operand is rounded at other places than the stand-alone transform's: this comparison
        # (against the library's own transform) is then between two roundings of the same exact
        # operand; the bound that pins K = 4096 is the one against the fp64 oracle below
        tol32 = 4e-3 if K == 4096 else 2e-3
        assert err <= (8e-3 if od == torch.bfloat16 else tol32), (od, err)


@pytest.mark.parametrize("K", [1024, 2048, 4096])
def test_gemm_bf16_full_size_error_against_oracle(pkg, oracle, K):
    # the full 4096 x 4096 shape, bf16 in, fp32 out, against the fp64 oracle on sampled rows (every
    # position inside a 64-row block, first and last blocks of an M slice).  Measured 3.5e-3 at
    # K = 1024 (the rounding of the transformed operand to bf16); the bar is set where a lost
    # rounding step, a mis-scaled pass or a dropped partial sum would show, not at the 2e-2 contract.
    M = N = 4096
    W, Xt = oracle.inputs_gemm(M, N, K, torch.bfloat16)
    C = pkg.fused_ht_gemm(W.cuda(), Xt.cuda(), out_dtype=torch.float32)
    torch.cuda.synchronize()
    g = torch.Generator().manual_seed(K)
    rows = torch.unique(torch.cat([torch.tensor([0, 1, 15, 16, 63, 64, 511, 512, 2047, 2048, 4032, 4095]),
                                   torch.randint(0, M, (20,), generator=g)]))
    want = oracle.fused_ht_gemm_f64_blas(W[rows].double().numpy(), Xt.double().numpy(), K ** -0.5)
    err = oracle.rel_err(C[rows.cuda()].cpu().double().numpy(), want)
    assert err <= 6e-3, (K, err)


# Shapes whose launch plan differs from the benchmark's: rectangles that do not fill all eight XCDs
# evenly (workgroup ids without work), M slices that are not a power of two, more than one round of
# workgroups, a ragged last slice and last column group.  Every element against the unfused
# product computed on the device from the library's own transform.
@pytest.mark.parametrize("K", [1024, 512, 2048, 4096])
@pytest.mark.parametrize("M,N", [(5000, 3000), (6144, 6144), (2048, 8192), (12288, 1536), (1000, 9000)])
def test_gemm_k1024_launch_plans(pkg, oracle, M, N, K):
    g = torch.Generator(device="cuda").manual_seed(M + N)
    s2 = {512: 1.0 / 16.0, 1024: 1.0 / 32.0, 2048: 1.0 / 32.0, 4096: 1.0 / 64.0}[K]   # a power of two
    Wd = torch.randn(M, K, generator=g, device="cuda").to(torch.bfloat16)
    Xd = torch.randn(N, K, generator=g, device="cuda").to(torch.bfloat16)
    Y = pkg.hadamard_transform(Xd, s2)
    ref = Wd.float() @ Y.float().t()
    scale = ref.abs().max().item()
    C = pkg.fused_ht_gemm(Wd, Xd, s2)
    torch.cuda.synchronize()
    assert torch.isfinite(C.float()).all()
    assert (C.float() - ref).abs().max().item() / scale <= 8e-3
    # a few rows against the fp64 oracle as well
    idx = torch.tensor([0, 63, 64, M // 2, M - 1])
    want = oracle.fused_ht_gemm_f64_blas(Wd[idx].cpu().double().numpy(), Xd.cpu().double().numpy(), s2)
    assert _rel(oracle, C[idx], want) <= 2e-2


# fp32 at K = 512 and 1024 runs the register-resident fp32 kernel on these shapes (too few 16-column
# x 64-row pairs for the GEMV route, all but (700, 1023)): groups of 65536 / K columns, 64-row
# blocks, one store of 1024 / K adjacent columns per lane and row; K = 256 runs the GEMV kernels
# (test_gemm_f32_small_k_both_routes has more of those); K = 2048 and 4096 the register-resident
# variant with the K range split over pairs of wavefronts (groups of 32 columns; K = 4096 in two
# phases, the second adding to what the first stored).  Shapes around every tile
# boundary (edge store path, N that rules out vector stores, one row block, odd and even numbers of
# row blocks), several scales, against the fp64 oracle at 1e-5.
@pytest.mark.parametrize("K", [1024, 512, 256, 2048, 4096])
@pytest.mark.parametrize("M,N", [(1, 1), (31, 33), (63, 63), (64, 64), (65, 65), (128, 64), (129, 127), (192, 130),
                                 (128, 256), (320, 258), (577, 333), (130, 1000), (2048, 70), (700, 1023)])
def test_gemm_f32_xreg_tile_boundaries(pkg, oracle, M, N, K):
    W, Xt = oracle.inputs_gemm(M, N, K, torch.float32)
    for scale in (None, 0.37 / 32.0, 1.0):
        s = 1.0 / math.sqrt(K) if scale is None else scale
        for _ in range(2):                                   # back-to-back launches reuse LDS and registers
            C = pkg.fused_ht_gemm(W.cuda(), Xt.cuda(), scale)
        torch.cuda.synchronize()
        want = oracle.fused_ht_gemm_f64_blas(W.double().numpy(), Xt.double().numpy(), s)
        assert C.shape == (M, N) and C.dtype == torch.float32
        err = np.abs(C.cpu().double().numpy() - want).max() / max(np.abs(want).max(), s * K)
        assert err <= 1e-5, (M, N, scale, err)


# fp32, K = 256 ... 4096, launch plans other than the benchmark's (ragged slices, more than one
# round of workgroups, rectangles that leave workgroup ids without work): every element against the
# product of W with the library's own fp32 transform, accumulated in fp64 on the device.
@pytest.mark.parametrize("K", [1024, 512, 256, 2048, 4096])
@pytest.mark.parametrize("M,N", [(4096, 4096), (5000, 3000), (2048, 8192), (12288, 1536), (1000, 9000)])
def test_gemm_f32_xreg_launch_plans(pkg, oracle, M, N, K):
    g = torch.Generator(device="cuda").manual_seed(M + N)
    Wd = torch.randn(M, K, generator=g, device="cuda")
    Xd = torch.randn(N, K, generator=g, device="cuda")
    Y = pkg.hadamard_transform(Xd, 1.0 / 32.0)
    C = pkg.fused_ht_gemm(Wd, Xd, 1.0 / 32.0)
    torch.cuda.synchronize()
    assert torch.isfinite(C).all()
    worst = 0.0
    for r0 in range(0, M, 1024):                             # fp64 product in slices (memory)
        ref = Wd[r0:r0 + 1024].double() @ Y.double().t()
        worst = max(worst, (C[r0:r0 + 1024].double() - ref).abs().max().item())
    assert worst / (K / 32.0) <= 1e-5, worst            # against the typical magnitude of an output
    idx = torch.tensor([0, 63, 64, M // 2, M - 1])
    want = oracle.fused_ht_gemm_f64_blas(Wd[idx].cpu().double().numpy(), Xd.cpu().double().numpy(), 1.0 / 32.0)
    assert _rel(oracle, C[idx], want) <= 1e-5


# fp32, K = 512 ... 2048 on small and medium outputs (at least 256 pairs of 16 columns x 64 rows, N <=
# 4096, up to 3072^2 outputs, below 2048^2 for K = 2048) runs the GEMV kernels on X given column by
# column: ragged rows and columns, one to many row blocks per workgroup, the shapes just inside and
# just outside the route's limits.
@pytest.mark.parametrize("K", [1024, 512, 2048])
@pytest.mark.parametrize("M,N", [(512, 512), (1024, 1024), (700, 1023), (4100, 130), (64, 4096), (2047, 2048),
                                 (3072, 3072), (8192, 1024), (1000, 4100)])
def test_gemm_f32_through_gemv_kernels(pkg, oracle, M, N, K):
    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    Wd = torch.randn(M, K, generator=g, device="cuda")
    Xd = torch.randn(N, K, generator=g, device="cuda")
    Y = pkg.hadamard_transform(Xd, 1.0 / 32.0)
    for _ in range(2):
        C = pkg.fused_ht_gemm(Wd, Xd, 1.0 / 32.0)
    torch.cuda.synchronize()
    assert C.shape == (M, N) and torch.isfinite(C).all()
    worst = 0.0
    for r0 in range(0, M, 1024):                             # fp64 product in slices (memory)
        ref = Wd[r0:r0 + 1024].double() @ Y.double().t()
        worst = max(worst, (C[r0:r0 + 1024].double() - ref).abs().max().item())
    assert worst / (K / 32.0) <= 1e-5, worst
    idx = torch.unique(torch.tensor([0, 63, 64, M // 2, M - 1]).clamp(0, M - 1))   # (M = 64 has no row 64)
    want = oracle.fused_ht_gemm_f64_blas(Wd[idx].cpu().double().numpy(), Xd.cpu().double().numpy(), 1.0 / 32.0)
    assert _rel(oracle, C[idx], want) <= 1e-5


# fp32, K <= 128: outputs up to 1536 x 1024 run the GEMV kernel (register-butterfly prologue reading
# X column by column), larger ones the LDS-tile GEMM kernel; K = 256 runs the GEMV kernels on every
# shape (the row-split one with 64 columns per workgroup from 128 pairs of 64 columns x 64 rows on).
# Shapes on both sides of the limits, ragged in both directions, and the smallest.
@pytest.mark.parametrize("K", [32, 64, 128, 256])
@pytest.mark.parametrize("M,N", [(1, 1), (33, 7), (512, 512), (700, 1023), (1024, 1536), (1025, 1536), (2048, 1024),
                                 (130, 4100)])
def test_gemm_f32_small_k_both_routes(pkg, oracle, M, N, K):
    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    Wd = torch.randn(M, K, generator=g, device="cuda")
    Xd = torch.randn(N, K, generator=g, device="cuda")
    scale = 1.0 / math.sqrt(K)
    Y = pkg.hadamard_transform(Xd, scale)
    for _ in range(2):
        C = pkg.fused_ht_gemm(Wd, Xd, scale)
    torch.cuda.synchronize()
    assert C.shape == (M, N) and torch.isfinite(C).all()
    ref = Wd.double() @ Y.double().t()
    assert (C.double() - ref).abs().max().item() / math.sqrt(K) <= 1e-5
    idx = torch.unique(torch.tensor([0, 63, 64, M // 2, M - 1]).clamp(0, M - 1))
    want = oracle.fused_ht_gemm_f64_blas(Wd[idx].cpu().double().numpy(), Xd.cpu().double().numpy(), scale)
    # against the typical magnitude of an output (sqrt(K) for these inputs), not the largest of a
    # handful that may all be sums that nearly cancel (M = N = 1)
    err = np.abs(C[idx].cpu().double().numpy() - want).max() / max(np.abs(want).max(), math.sqrt(K))
    assert err <= 1e-5, err


def test_gemm_small_bruteforce(pkg, oracle):
    # triple-loop oracle (no BLAS), fp32
    M, N, K = 16, 20, 64
    W, Xt = oracle.inputs_gemm(M, N, K, torch.float32)
    C = pkg.fused_ht_gemm(W.cuda(), Xt.cuda(), 1.0)
    want = oracle.fused_ht_gemm_f64(W.double().numpy(), Xt.double().numpy(), 1.0)
    assert _rel(oracle, C, want) <= 1e-5


def test_gemm_identity_reduces_to_transform(pkg, oracle):
    K, N = 256, 40
    _, Xt = oracle.inputs_gemm(K, N, K, torch.float32)
    C = pkg.fused_ht_gemm(torch.eye(K).cuda(), Xt.cuda())
    want = oracle.fwht_f64(Xt.double().numpy()).T  # C = H X
    assert _rel(oracle, C, want) <= 1e-5


def test_gemm_reference_self_check_shape(pkg, oracle):
    # fusion_pipelined.cu: K=1024, M=N=4096, uniform [0,1) inputs, fused vs unfused < 1e-3 abs
    # (on a 512 x 512 corner to keep the fp64 host product small), unnormalised, fp32
    g = torch.Generator().manual_seed(123)
    W = torch.rand(4096, 1024, generator=g)
    Xt = torch.rand(4096, 1024, generator=g)
    C = pkg.fused_ht_gemm(W.cuda(), Xt.cuda(), 1.0)
    torch.cuda.synchronize()
    Yht = pkg.hadamard_transform(Xt.cuda(), 1.0)  # unfused: transform, then product
    ref = W[:512].double() @ Yht[:512].cpu().double().t()
    got = C[:512, :512].cpu().double()
    # outputs reach ~5e5 in magnitude for all-positive inputs; the reference's 1e-3 absolute bar
    # is applied relative to that scale here
    assert (got - ref).abs().max().item() / ref.abs().max().item() < 1e-5
    want = oracle.fused_ht_gemm_f64_blas(W[:512].double().numpy(), Xt[:512].double().numpy(), 1.0)
    assert oracle.rel_err(got.numpy(), want) <= 1e-5


@pytest.mark.parametrize("dt,tol", [(torch.bfloat16, 2e-2), (torch.float32, 1e-5)], ids=["bf16", "f32"])
def test_gemm_full_size_config(pkg, oracle, dt, tol):
    # benchmark configuration 4: W [4096,1024], Xt [4096,1024], scale 1/32; checked on sampled rows/cols
    W, Xt = oracle.inputs_gemm(4096, 4096, 1024, dt)
    C = pkg.fused_ht_gemm(W.cuda(), Xt.cuda(), out_dtype=torch.float32)
    torch.cuda.synchronize()
    rows = torch.tensor([0, 1, 63, 64, 511, 512, 2047, 2048, 4095])
    want = oracle.fused_ht_gemm_f64_blas(W[rows].double().numpy(), Xt.double().numpy(), 1.0 / 32.0)
    assert oracle.rel_err(C[rows.cuda()].cpu().double().numpy(), want) <= tol


def test_fused_size_limits_match_the_c_abi(pkg, oracle):
    # boundary values of the documented ranges: GEMV N in [2, 2048], GEMM K in [32, 4096]
    for N in (2, 2048):
        W, X = oracle.inputs_gemv(8, N, 5)
        Y = pkg.fused_ht_gemv(W.cuda(), X.cuda())
        want = oracle.fused_ht_gemv_f64_blas(W.double().numpy(), X.double().numpy(), N ** -0.5)
        assert _rel(oracle, Y, want) <= 1e-5
    for N in (1, 4096):
        with pytest.raises(RuntimeError, match="power of two in"):
            pkg.fused_ht_gemv(torch.zeros(8, N, device="cuda"), torch.zeros(N, 5, device="cuda"))
    for K in (32, 4096):
        W, Xt = oracle.inputs_gemm(8, 5, K, torch.bfloat16)
        C = pkg.fused_ht_gemm(W.cuda(), Xt.cuda(), out_dtype=torch.float32)
        want = oracle.fused_ht_gemm_f64_blas(W.double().numpy(), Xt.double().numpy(), K ** -0.5)
        assert _rel(oracle, C, want) <= 2e-2
    for K in (16, 8192):
        with pytest.raises(RuntimeError, match="power of two in"):
            pkg.fused_ht_gemm(torch.zeros(8, K, device="cuda", dtype=torch.bfloat16),
                              torch.zeros(5, K, device="cuda", dtype=torch.bfloat16))


def test_fused_errors(pkg):
    z = torch.zeros(4, 24, device="cuda")
    with pytest.raises(RuntimeError):
        pkg.fused_ht_gemv(z, torch.zeros(24, 3, device="cuda"))
    with pytest.raises(RuntimeError):
        pkg.fused_ht_gemm(z, torch.zeros(5, 24, device="cuda"))
    with pytest.raises(RuntimeError):
        pkg.fused_ht_gemm(torch.zeros(4, 64, device="cuda"), torch.zeros(5, 32, device="cuda"))


def test_gemm_f32_k4096_does_not_depend_on_what_c_held(pkg, oracle):
    # fp32 at K = 4096 is two kernels, the second adding to what the first stored in C: the first
    # must overwrite whatever C held (NaN here), also in the masked edge blocks
    import importlib
    lib = importlib.import_module("6s894_project_2025_amd._lib")
    K = 4096
    for M, N in ((200, 70), (128, 64)):
        W, Xt = oracle.inputs_gemm(M, N, K, torch.float32)
        Wd, Xd = W.cuda(), Xt.cuda()
        C = torch.full((M, N), float("nan"), device="cuda")
        st = lib.load().mi_fused_ht_gemm(Wd.data_ptr(), Xd.data_ptr(), C.data_ptr(), M, N, K, lib.MI_F32,
                                         lib.MI_F32, 1.0 / 64.0, torch.cuda.current_stream().cuda_stream)
        assert st == 0
        torch.cuda.synchronize()
        want = oracle.fused_ht_gemm_f64_blas(W.double().numpy(), Xt.double().numpy(), 1.0 / 64.0)
        assert _rel(oracle, C, want) <= 1e-5


def test_gemm16_k4096_does_not_depend_on_what_c_held(pkg, oracle):
    # the same for 16-bit inputs (two passes of the split-K kernel, the second adding in the L2), all
    # four type combinations, shapes with and without edge blocks, twice in a row into the same C
    import importlib
    lib = importlib.import_module("6s894_project_2025_amd._lib")
    K = 4096
    for dt, code in ((torch.bfloat16, lib.MI_BF16), (torch.float16, lib.MI_F16)):
        for M, N in ((200, 70), (128, 64), (640, 256)):
            W, Xt = oracle.inputs_gemm(M, N, K, dt)
            Wd, Xd = W.cuda(), Xt.cuda()
            want = oracle.fused_ht_gemm_f64_blas(W.double().numpy(), Xt.double().numpy(), 1.0 / 64.0)
            for od, ocode in ((torch.float32, lib.MI_F32), (dt, code)):
                C = torch.full((M, N), float("nan"), device="cuda", dtype=od)
                for _ in range(2):
                    st = lib.load().mi_fused_ht_gemm(Wd.data_ptr(), Xd.data_ptr(), C.data_ptr(), M, N, K, code,
                                                     ocode, 1.0 / 64.0, torch.cuda.current_stream().cuda_stream)
                    assert st == 0
                torch.cuda.synchronize()
                assert _rel(oracle, C, want) <= 2e-2, (dt, od, M, N)


# The register-resident kernels issue their main-loop MFMAs, LDS reads, transfers and stores as
# hand-placed opaque statements whose hazards (result latency, operand reads that last several
# cycles, transfers that must have landed) the compiler does not see.  A timing-dependent slip
# there would corrupt a lane now and then, not every time: 30 back-to-back launches on the same
# inputs must give the same bits, and the first must be right.  Shapes with more workgroups than
# compute units (several rounds, so a workgroup also starts on a compute unit whose registers and LDS
# another one has just left) and ragged edges.
def _bits(t):
    return t.view(torch.int32 if t.element_size() == 4 else torch.int16)


@pytest.mark.parametrize("dt,K", [(torch.bfloat16, 512), (torch.bfloat16, 1024), (torch.bfloat16, 2048),
                                  (torch.bfloat16, 4096), (torch.float16, 512), (torch.float16, 1024),
                                  (torch.float16, 2048), (torch.float16, 4096), (torch.float32, 256),
                                  (torch.float32, 512), (torch.float32, 1024), (torch.float32, 2048),
                                  (torch.float32, 4096)],
                         ids=lambda v: str(v).replace("torch.", ""))
def test_gemm_register_resident_kernels_are_deterministic(pkg, oracle, dt, K):
    import importlib
    lib = importlib.import_module("6s894_project_2025_amd._lib")
    M, N = 2500, 5000
    if dt != torch.float32:
        import ctypes
        header = (ctypes.c_uint32 * 8)()
        for M, N in ((2500, 5000), (5000, 9000), (200, 70000)):   # the first whose plan has several rounds
            assert lib.load().mi_debug_fused_gemm_tiling(M, N, K, header, None, 0) == 0
            if header[6] > 256:
                break
        assert header[6] > 256, "the shape is meant to need more than one round of workgroups"
    W, Xt = oracle.inputs_gemm(M, N, K, dt)
    Wd, Xd = W.cuda(), Xt.cuda()
    for od in ((torch.float32,) if dt == torch.float32 else (torch.float32, dt)):
        first = pkg.fused_ht_gemm(Wd, Xd, out_dtype=od)
        torch.cuda.synchronize()
        rows = torch.tensor([0, 63, 64, M // 3, M // 2 - 1, M // 2, M - 64, M - 1])
        want = oracle.fused_ht_gemm_f64_blas(W[rows].double().numpy(), Xt.double().numpy(), K ** -0.5)
        assert _rel(oracle, first[rows.cuda()], want) <= (1e-5 if dt == torch.float32 else 2e-2), (dt, K, od)
        for i in range(1, 30):
            again = pkg.fused_ht_gemm(Wd, Xd, out_dtype=od)
            same = torch.equal(_bits(again), _bits(first))
            if not same:
                bad = (_bits(again) != _bits(first)).nonzero()
                pytest.fail(f"launch {i} differs from launch 0 in {len(bad)} elements, first at {bad[0].tolist()} "
                            f"({dt}, K={K}, out {od})")


def slack_of(Wd, Y, eps16):
    # The kernel rounds the transformed operand H(x) to 16 bits (relative error eps16 per element,
    # independent between elements): the sum over K of |w y| eps16 would be the worst case, its
    # root-mean-square size is smaller by sqrt(K); six times that is never reached in practice.
    K = Wd.shape[1]
    return 6.0 * eps16 * (Wd.double().abs() @ Y.abs().t()) / K ** 0.5


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_gemm16_k4096_sixteen_bit_output_contract(pkg, oracle, dt):
    # K = 4096 with 16-bit output runs two passes that meet in C in 16-bit arithmetic: the stated bound
    # is ulp16(P0) + ulp16(P1) + ulp16(C) around the exact result, with P0, P1 the half-K sums.  Checked
    # against the fp32-output result (both halves in fp32) on ordinary data and on data whose halves
    # nearly cancel: W[:, 2048:] = -W[:, :2048] + small, and columns of X whose second half is zero, so
    # that H(x)[2048:] = H(x)[:2048] and P1 = -P0 + small.
    K, M, N = 4096, 300, 200                       # edge blocks (fp32 add) and full blocks (16-bit add)
    eps16 = 2.0 ** (-8 if dt == torch.bfloat16 else -11)   # half the relative spacing of the type

    def ulp(v):                                     # spacing of the 16-bit type at |v| (normal range)
        return torch.pow(2.0, torch.floor(torch.log2(v.abs().clamp_min(1e-30)))) * (2.0 * eps16)

    g = torch.Generator().manual_seed(11)
    for case in ("random", "cancelling"):
        W = torch.randn(M, K, generator=g)
        Xt = torch.randn(N, K, generator=g)
        if case == "cancelling":
            W[:, 2048:] = -W[:, :2048] + 0.01 * torch.randn(M, 2048, generator=g)
            Xt[:, 2048:] = 0.0
        Wd, Xd = W.to(dt).cuda(), Xt.to(dt).cuda()
        C32 = pkg.fused_ht_gemm(Wd, Xd, out_dtype=torch.float32)
        C16 = pkg.fused_ht_gemm(Wd, Xd, out_dtype=dt)
        torch.cuda.synchronize()
        assert torch.isfinite(C16.float()).all()
        # the halves, from the library's own transform (fp64 products on the device)
        Y = pkg.hadamard_transform(Xd.float(), 1.0 / 64.0).double()
        P0 = Wd[:, :2048].double() @ Y[:, :2048].t()
        P1 = Wd[:, 2048:].double() @ Y[:, 2048:].t()
        exact = P0 + P1
        # fp32 output: both halves meet in fp32; what is left is the 16-bit rounding of the operand
        assert ((C32.double() - exact).abs() <= slack_of(Wd, Y, eps16) + 1e-5 * exact.abs()).all()
        bound = ulp(P0) + ulp(P1) + ulp(exact)
        # (the operand H(x) itself is rounded to 16 bits inside the kernel: allow for that too, one
        # part in 2^8 or 2^11 of the typical magnitude of a half-K sum's terms)
        slack = slack_of(Wd, Y, eps16)
        worst = ((C16.double() - exact).abs() - bound - slack).max().item()
        assert worst <= 0.0, (case, worst)
        if case == "cancelling":
            # the point of the case: the partial sums dwarf the result
            assert (P0.abs().median() > 20 * exact.abs().median()).item()
