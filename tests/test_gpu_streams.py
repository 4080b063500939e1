"""Calls that overlap in time on different streams use different workspaces (one per stream, as the host side hands
them out) and must not disturb each other's cross-workgroup exchanges."""
import pytest
import torch

from hidet_amd.graph.ops import quant
from gpu_util import announce

pytestmark = pytest.mark.gpu


def test_two_streams_overlap():
    announce('two streams, w8a16 gemv + gemm with K split')
    g = torch.Generator(device='cuda').manual_seed(7)
    k, n = 4096, 2048
    w = torch.randint(-127, 128, (k, n), device='cuda', dtype=torch.int8, generator=g)
    s = (torch.rand(n, device='cuda', generator=g) * 0.01).half()
    xs = [torch.randn(m, k, device='cuda', generator=g).half() for m in (1, 40)]
    want = [quant.symmetric_quant_matmul(x, w, s) for x in xs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[], []]
    for rep in range(40):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                outs[i].append(quant.symmetric_quant_matmul(xs[i], w, s))
    torch.cuda.synchronize()
    for i in range(2):
        for rep, o in enumerate(outs[i]):
            assert torch.equal(o, want[i]), (i, rep)
