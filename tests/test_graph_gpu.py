"""The entry points neither allocate nor synchronise, so a caller can record them into a HIP graph.
Capture a short pipeline (in-place transform, fused HT->GEMM in bf16 at K = 1024 and, in bf16 and in
fp32, at K = 4096, which is two kernels of which the second adds to the first's result, RHT + FP8
quantize), replay it
several times with new inputs and the program's own eager work between the replays, and compare
every replay with the eager result on the same inputs (bit for bit: same kernels, same data)."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_pipeline_replays_from_a_hip_graph(pkg):
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cuda").manual_seed(11)

    def fresh():
        return (torch.randn(512, 4096, generator=g, device=dev).to(torch.bfloat16),
                torch.randn(300, 1024, generator=g, device=dev).to(torch.bfloat16),
                torch.randn(260, 1024, generator=g, device=dev).to(torch.bfloat16),
                torch.randn(200, 4096, generator=g, device=dev),
                torch.randn(70, 4096, generator=g, device=dev),
                torch.randn(192, 4096, generator=g, device=dev).to(torch.bfloat16),
                torch.randn(130, 4096, generator=g, device=dev).to(torch.bfloat16))

    sign = (1 - 2 * torch.randint(0, 2, (4096,), generator=g, device=dev)).to(torch.int8)

    def pipeline(x, W, Xt, W32, Xt32, Wk, Xtk):
        y = pkg.hadamard_transform(x.clone(), inplace=True)
        C = pkg.fused_ht_gemm(W, Xt)
        C32 = pkg.fused_ht_gemm(W32, Xt32)
        Ck = pkg.fused_ht_gemm(Wk, Xtk)
        q, s = pkg.rht_quant_fp8(x, sign)
        return y, C, C32, Ck, q, s

    bufs = fresh()
    pipeline(*bufs)  # first use outside the capture (library load, kernel attributes)
    torch.cuda.synchronize()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            outs = pipeline(*bufs)
    torch.cuda.current_stream().wait_stream(side)

    for rep in range(4):
        new = fresh()
        for dst, src in zip(bufs, new):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = pipeline(*new)  # eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a.view(torch.uint8) if a.dtype == torch.float8_e4m3fn else a,
                               b.view(torch.uint8) if b.dtype == torch.float8_e4m3fn else b), rep
