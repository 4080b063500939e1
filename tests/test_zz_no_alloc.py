"""GPU test of hidet_symmetric_quant_matmul_f16_i8_static, the entry point that allocates nothing and keeps its
split-K scratch in a static device array: its output must equal, bit for bit, what
hidet_symmetric_quant_matmul_f16_i8 writes for the same operands with a workspace of the same size, on
consecutive calls that share the array (the second smaller than the first), and both must agree with the oracle."""
import numpy as np
import pytest
import torch

from hidet_amd import ffi
from oracle import clib
from oracle import oracle as O
from gpu_util import announce, dev, host

pytestmark = pytest.mark.gpu


def _case(seed, m, k, n):
    a32, w32 = O.make_inputs(seed, m, k, n)
    q, s32 = O.symmetric_quantize(w32, 'int8', dims=0)
    return a32.astype(np.float16), q, s32.astype(np.float16)


def _static(a, q, s, parts=0):
    m, k = a.shape
    n = q.shape[1]
    c = torch.full((m, n), float('nan'), dtype=torch.float16, device=a.device)
    ffi.call('hidet_symmetric_quant_matmul_f16_i8_static', a, q, s, c, m, k, n, a.stride(0), parts,
             ffi.current_stream(a.device))
    return c


def _with_workspace(a, q, s, ws, parts=0):
    m, k = a.shape
    n = q.shape[1]
    c = torch.full((m, n), float('nan'), dtype=torch.float16, device=a.device)
    ffi.call('hidet_symmetric_quant_matmul_f16_i8', a, q, s, c, m, k, n, a.stride(0), parts, ws, ws.numel(),
             ffi.current_stream(a.device))
    return c


def test_static_scratch_matches_workspace_entry_point():
    nbytes = ffi.load_library().hidet_qmm_static_scratch_bytes()
    assert nbytes == (16 << 20) + (64 << 10)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device='cuda')
    # consecutive calls on one stream share the static array; each is smaller than, or as large as, the one before:
    # a decode GEMV with 8 K slices, a 16-row pass, a GEMV on a narrower matrix, a GEMM computed in K ranges, a tiny one
    shapes = [(1, 4096, 11008), (16, 4096, 4096), (1, 2048, 1024), (40, 4096, 4096), (3, 256, 512), (1, 4096, 11008)]
    for seed, (m, k, n) in enumerate(shapes):
        announce('static scratch', m, k, n)
        a, q, s = _case(seed, m, k, n)
        da, dq, ds = dev(a), dev(q), dev(s)
        got = host(_static(da, dq, ds))
        want = host(_with_workspace(da, dq, ds, ws))
        assert not np.isnan(got).any()
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), (m, k, n)
        if m * k * n <= 16 * 4096 * 4096:
            ref = clib.quant_matmul_f32acc(a, q, s)
            assert O.max_rel_err(got, ref) <= 1e-2
    # back to back without a host synchronisation in between, results read at the end
    a1, q1, s1 = _case(10, 4, 4096, 8192)
    a2, q2, s2 = _case(11, 2, 1024, 768)
    d1 = [dev(x) for x in (a1, q1, s1)]
    d2 = [dev(x) for x in (a2, q2, s2)]
    announce('static scratch back to back')
    c1 = _static(*d1)
    c2 = _static(*d2)
    c1b = _static(*d1)
    torch.cuda.synchronize()
    assert np.array_equal(host(c1).view(np.uint16), host(_with_workspace(*d1, ws)).view(np.uint16))
    assert np.array_equal(host(c2).view(np.uint16), host(_with_workspace(*d2, ws)).view(np.uint16))
    assert np.array_equal(host(c1).view(np.uint16), host(c1b).view(np.uint16))


def test_static_scratch_allocates_nothing_and_replays_from_a_graph():
    # device memory in use is the same before and after the calls (the library's side; the output tensors are made first)
    a, q, s = _case(31, 1, 4096, 11008)
    a2, q2, s2 = _case(32, 8, 2048, 1024)
    d1 = [dev(x) for x in (a, q, s)]
    d2 = [dev(x) for x in (a2, q2, s2)]
    announce('static scratch: memory in use')
    stream = ffi.current_stream(d1[0].device)
    outs = [torch.empty((x[0].shape[0], x[1].shape[1]), dtype=torch.float16, device='cuda') for x in (d1, d2)]

    def call(d, c):
        ffi.call('hidet_symmetric_quant_matmul_f16_i8_static', d[0], d[1], d[2], c, d[0].shape[0], d[0].shape[1], d[1].shape[1],
                 d[0].stride(0), 0, ffi.current_stream(d[0].device))

    call(d1, outs[0])  # the first call on a device looks up the array's address: outside the measurement and any capture
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        call(d1, outs[0])
        call(d2, outs[1])
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    eager = [host(o).copy() for o in outs]
    assert ffi.call('hidet_qmm_exchange_status', None, 0, stream) == 0

    # captured into a graph (the launches only: no allocation, no memset node), replayed with eager work in between
    announce('static scratch: graph replays')
    graph = torch.cuda.CUDAGraph()
    g_outs = [torch.zeros_like(o) for o in outs]
    with torch.cuda.graph(graph):
        call(d1, g_outs[0])
        call(d2, g_outs[1])
    for rep in range(4):
        for o in g_outs:
            o.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for o, e in zip(g_outs, eager):
            assert np.array_equal(host(o).view(np.uint16), e.view(np.uint16)), rep
        call(d2, outs[1])  # the program's own eager work between the replays, on the same array
        torch.cuda.synchronize()
        assert np.array_equal(host(outs[1]).view(np.uint16), eager[1].view(np.uint16))


def test_static_scratch_exact_on_small_integers():
    rng = np.random.default_rng(5)
    for m, k, n, parts in [(5, 2048, 4096, 0), (2, 512, 256, 3), (16, 1024, 11008, 0)]:
        announce('static scratch exact', m, k, n, parts)
        a = rng.integers(-2, 3, (m, k)).astype(np.float16)
        q = rng.integers(-127, 128, (k, n)).astype(np.int8)
        s = (2.0 ** rng.integers(-12, -9, n)).astype(np.float16)
        want = (a.astype(np.int64) @ q.astype(np.int64)).astype(np.float64) * s.astype(np.float64)[None, :]
        got = host(_static(dev(a), dev(q), dev(s), parts))
        assert np.array_equal(got, want.astype(np.float32).astype(np.float16))


def test_static_scratch_rejects_oversized_split():
    # 16 rows, K = 16384, N = 32768, 16 K slices asked for: 128 column tiles x 16 slices x 16 KiB of partial tiles = 32 MiB,
    # more than the mailbox share (4 MiB) of the static array
    m, k, n = 16, 16384, 32768
    announce('static scratch reject', m, k, n)
    a = torch.zeros((m, k), dtype=torch.float16, device='cuda')
    q = torch.zeros((k, n), dtype=torch.int8, device='cuda')
    s = torch.ones(n, dtype=torch.float16, device='cuda')
    with pytest.raises(ffi.BackendException, match='scratch too small'):
        _static(a, q, s, 21)
    # the error left the array usable
    a2, q2, s2 = _case(3, 1, 1024, 512)
    got = host(_static(dev(a2), dev(q2), dev(s2)))
    assert O.max_rel_err(got, clib.quant_matmul_f32acc(a2, q2, s2)) <= 1e-2


def test_task_library_launch_matches_the_operator(tmp_path):
    # hidet_launch_0(a, weight, scale, c) of a generated task library (pointers only, shapes fixed at build time) runs the
    # entry point that needs no workspace; same result as the operator, on the stream set for the task
    import ctypes
    from hidet_amd.drivers import build_task_library
    from hidet_amd.graph.ops import quant
    m, k, n = 2, 2048, 1024
    announce('task library', m, k, n)
    a, q, s = _case(21, m, k, n)
    da, dq, ds = dev(a), dev(q), dev(s)
    lib = ctypes.CDLL(build_task_library(str(tmp_path), m, k, n))
    lib.hidet_launch_0.argtypes = [ctypes.c_void_p] * 4
    lib.hidet_qmm_task_set_stream.argtypes = [ctypes.c_void_p]
    c = torch.full((m, n), float('nan'), dtype=torch.float16, device='cuda')
    lib.hidet_qmm_task_set_stream(ffi.current_stream(da.device))
    lib.hidet_launch_0(da.data_ptr(), dq.data_ptr(), ds.data_ptr(), c.data_ptr())
    assert ffi.get_last_error() is None
    want = quant.symmetric_quant_matmul(da, dq, ds)
    assert torch.equal(c, want)
    assert O.max_rel_err(host(c), clib.quant_matmul_f32acc(a, q, s)) <= 1e-2
