"""The launches are capturable in a HIP graph: no allocation, no memset, and the cross-workgroup exchanges return their
counters to zero, so a captured launch can be replayed. Each case captures one call whose kernel exchanges partial
results between workgroups, replays it several times with fresh activations and eager work on other streams in
between, and compares every replay bit for bit with an eager call on the same inputs."""
import numpy as np
import pytest
import torch

from hidet_amd.graph.ops import quant
from hidet_amd.graph.ops.matmul import matmul_f8 as F8
from gpu_util import announce

pytestmark = pytest.mark.gpu


def _w8(m, k, n):
    g = torch.Generator(device='cuda').manual_seed(m * 7 + n)
    a = torch.randn(m, k, device='cuda', generator=g).half()
    w = torch.randint(-127, 128, (k, n), device='cuda', dtype=torch.int8, generator=g)
    s = (torch.rand(n, device='cuda', generator=g) * 0.01).half()
    return a, (lambda x: quant.symmetric_quant_matmul(x, w, s))


def _w4(m, k, n):
    g = torch.Generator(device='cuda').manual_seed(m * 11 + n)
    a = torch.randn(m, k, device='cuda', generator=g).bfloat16()
    w = torch.randint(0, 256, (k, n // 2), device='cuda', dtype=torch.uint8, generator=g)
    s = (torch.rand(k // 128, n, device='cuda', generator=g) * 0.01).bfloat16()
    return a, (lambda x: quant.symmetric_quant_matmul_w4a16(x, w, s, 128))


def _w8_nk(m, k, n):
    g = torch.Generator(device='cuda').manual_seed(m * 17 + n)
    a = torch.randn(m, k, device='cuda', generator=g).half()
    w = quant.to_decode_layout(torch.randint(-127, 128, (k, n), device='cuda', dtype=torch.int8, generator=g))
    s = (torch.rand(n, device='cuda', generator=g) * 0.01).half()
    return a, (lambda x: quant.symmetric_quant_matmul(x, w, s))


def _w4_nk(m, k, n):
    g = torch.Generator(device='cuda').manual_seed(m * 19 + n)
    a = torch.randn(m, k, device='cuda', generator=g).bfloat16()
    w = quant.to_decode_layout_int4(torch.randint(0, 256, (k, n // 2), device='cuda', dtype=torch.uint8, generator=g))
    s = (torch.rand(k // 128, n, device='cuda', generator=g) * 0.01).bfloat16()
    return a, (lambda x: quant.symmetric_quant_matmul_w4a16_decode(x, w, s, 128))


def _f8(m, k, n):
    g = torch.Generator(device='cuda').manual_seed(m * 13 + n)
    a = torch.randint(0, 0x7F, (m, k), device='cuda', dtype=torch.uint8, generator=g).view(torch.float8_e4m3fn)
    b = torch.randint(0, 0x7F, (n, k), device='cuda', dtype=torch.uint8, generator=g).view(torch.float8_e4m3fn)
    return a, (lambda x: F8.matmul_f8(x, b, output_dtype='float32'))


CASES = [('w8a16 gemv, K slices', _w8, 1, 4096, 1024), ('w8a16 gemm, K ranges of short tiles', _w8, 48, 4096, 1024),
         ('w8a16 16 rows', _w8, 16, 4096, 512), ('w4a16 gemv', _w4, 1, 4096, 1024), ('w4a16 gemm, K ranges', _w4, 129, 4096, 512),
         ('fp8 gemm, K ranges', _f8, 100, 8192, 1024), ('fp8 16 rows', _f8, 16, 4096, 1024),
         ('w8a16 decode layout', _w8_nk, 8, 4096, 1024), ('w4a16 decode layout', _w4_nk, 8, 4096, 1024)]


@pytest.mark.parametrize('name,make,m,k,n', CASES, ids=[c[0] for c in CASES])
def test_replays_match_eager(name, make, m, k, n):
    announce('graph capture', name, m, k, n)
    a, op = make(m, k, n)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        op(a)  # eager warm-up on the capture stream: its workspace exists before the capture begins
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out = op(a)
    for rep in range(4):
        if a.dtype == torch.float8_e4m3fn:
            fresh = torch.randint(0, 0x7F, a.shape, device='cuda', dtype=torch.uint8).view(torch.float8_e4m3fn)
            a.view(torch.uint8).copy_(fresh.view(torch.uint8))
        else:
            a.copy_(torch.randn(a.shape, device='cuda').to(a.dtype))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = op(a)  # eager, default stream, its own workspace
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.uint8) if got.dtype == torch.float8_e4m3fn else got,
                           want.view(torch.uint8) if want.dtype == torch.float8_e4m3fn else want), (name, rep)
