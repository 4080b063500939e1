"""GPU parity of the W8A16 matmul entry points against the oracle (dequantize, then matmul with fp32
accumulation): max |out - ref| / max |ref| <= 1e-2, and exact equality on small-integer inputs."""
import numpy as np
import pytest
import torch

import hidet_amd
from oracle import clib
from oracle import oracle as O
from hidet_amd.graph.ops import quant
from gpu_util import announce, dev, host

pytestmark = pytest.mark.gpu
TOL = 1e-2  # max relative error (normalised by max |ref|) for float16 outputs


def _case(seed, m, k, n):
    a32, w32 = O.make_inputs(seed, m, k, n)
    a = a32.astype(np.float16)
    q, s32 = O.symmetric_quantize(w32, 'int8', dims=0)
    return a, q, s32.astype(np.float16)


def _int_case(seed, m, k, n):
    rng = np.random.default_rng(seed)
    a = rng.integers(-2, 3, (m, k)).astype(np.float16)
    q = rng.integers(-127, 128, (k, n)).astype(np.int8)
    s = (2.0 ** rng.integers(-12, -9, n)).astype(np.float16)
    return a, q, s


@pytest.mark.parametrize('m,k,n', [(1, 256, 256), (1, 4096, 512), (3, 1024, 768), (16, 512, 256), (7, 96, 48),
                                   (1, 40, 16), (2, 8, 16), (1, 4096, 272), (16, 4096, 4096),
                                   (9, 4096, 8192), (16, 1024, 11008), (12, 512, 8200),  # 9 to 16 rows on wide outputs
                                   # one and two rows on at least 32 column tiles: runs of (tile, step) units across the tiles -
                                   # the headline shape, K not a multiple of 32, a last tile of 16 columns, fewer runs than CUs,
                                   # a long K on few tiles, two contributors per tile, as many tiles as runs (nothing exchanged)
                                   (1, 4096, 11008), (2, 4096, 11008), (1, 1000, 8208), (2, 544, 12288), (1, 96, 16400),
                                   (1, 11008, 8192), (2, 2080, 32768), (2, 2080, 65536), (3, 4096, 11008)])
def test_exact_on_small_integers(m, k, n):
    # integer activations and codes with power-of-two scales: every product and partial sum is exact in
    # fp32, so any dropped row, wrong byte or lost K slice shows as a whole-number difference
    announce('w8a16 exact', m, k, n)
    a, q, s = _int_case(m * 1000 + n, m, k, n)
    want = ((a.astype(np.int64) @ q.astype(np.int64)).astype(np.float64) * s.astype(np.float64)[None, :])
    got = host(quant.symmetric_quant_matmul(dev(a), dev(q), dev(s)))
    assert np.array_equal(got, want.astype(np.float32).astype(np.float16))


@pytest.mark.parametrize('x_shape,w_shape', [[[2, 32, 32], [32, 32]], [[1, 64, 64], [64, 128]]])
def test_reference_recipe(x_shape, w_shape):
    # tests/operators_core/test_quantization.py:39-47: quantized result vs the UNquantized matmul at 2e-1
    announce('w8a16 reference recipe', x_shape, w_shape)
    rng = np.random.default_rng(12)
    x = rng.standard_normal(x_shape).astype(np.float16)
    w = rng.standard_normal(w_shape).astype(np.float16)
    wq, scale = quant.symmetric_quantize(dev(w), dims=0, quant_type='int8')
    yq = quant.symmetric_quant_matmul_f16_i8(dev(x), wq, scale)
    assert tuple(yq.shape) == (1,) + tuple(x_shape[:-1]) + (w_shape[1],)
    y = np.matmul(x.astype(np.float32), w.astype(np.float32))
    assert np.allclose(y, host(yq.sum(0)).astype(np.float32), atol=2e-1, rtol=2e-1)
    y2 = quant.symmetric_quant_matmul(dev(x), wq, scale)
    assert np.allclose(y, host(y2).astype(np.float32), atol=2e-1, rtol=2e-1)


@pytest.mark.parametrize('m,k,n,seed', [(16, 4096, 4096, 0), (1, 4096, 11008, 0), (1, 4096, 11008, 1),
                                        (1, 4096, 11008, 2), (1, 4096, 11008, 3), (1, 11008, 4096, 0),
                                        (1, 11008, 4096, 1), (1, 11008, 4096, 2), (1, 11008, 4096, 3), (5, 1000, 528, 0), (33, 512, 256, 0), (13, 4096, 11008, 0)])
def test_parity_with_oracle(m, k, n, seed):
    announce('w8a16 parity', m, k, n, seed)
    a, q, s = _case(seed, m, k, n)
    ref = clib.quant_matmul_f32acc(a, q, s)
    got = host(quant.symmetric_quant_matmul(dev(a), dev(q), dev(s)))
    err = O.max_rel_err(got, ref)
    print('max_rel_err', err)
    assert err <= TOL
    assert err <= 2e-3  # in practice only float16 rounding of the output separates the two


def test_split_k_parts_api_and_hints():
    announce('w8a16 split-k api')
    a, q, s = _int_case(5, 3, 100, 32)
    a[:] = np.clip(a, -2, 2)
    q[:] = np.clip(q, -7, 7)
    ta, tq, ts = dev(a), dev(q), dev(s)
    full = host(quant.symmetric_quant_matmul(ta, tq, ts)).astype(np.float64)
    for parts in (1, 2, 3, 7, 128):
        c = quant.symmetric_quant_matmul_f16_i8(ta, tq, ts, parallel_k_parts=parts)
        assert tuple(c.shape) == (parts, 3, 32)
        ref = O.quant_matmul_split_k(a, q, s, parts)
        assert np.array_equal(host(c), ref), parts
        assert np.array_equal(host(c).astype(np.float64).sum(0), full)
    for parts in (1, 4, 32):
        c = quant.symmetric_quant_matmul_atomic_f16_i8(ta, tq, ts, parallel_k_parts=parts)
        assert np.array_equal(host(c).astype(np.float64), full)
    a, q, s = _case(0, 2, 2048, 512)
    base = quant.symmetric_quant_matmul(dev(a), dev(q), dev(s))
    for hint in (1, 2, 5, 16):
        hidet_amd.option.parallel_k(hint)
        try:
            c = quant.symmetric_quant_matmul(dev(a), dev(q), dev(s))
        finally:
            hidet_amd.option.parallel_k('disabled')
        assert O.max_rel_err(host(c), host(base)) < 1e-3


@pytest.mark.parametrize('m,k,n,layout', [(1, 4096, 11008, 'kn'), (3, 1024, 768, 'kn'), (8, 2048, 4096, 'kn'), (16, 512, 256, 'kn'),
                                          (12, 512, 8200, 'kn'), (40, 2048, 520, 'kn'), (300, 512, 1100, 'kn'), (2, 100, 40, 'kn'),
                                          (1, 4096, 1024, 'nk'), (16, 1024, 512, 'nk'), (40, 2048, 520, 'nk'), (12, 8192, 8192, 'nk')])
def test_bias_in_the_epilogue_exact(m, k, n, layout):
    # c = f16(f16(acc * scale) + bias): integer operands, power-of-two scales and a bias of small multiples of
    # 2^-10 make every step exact; every kernel family that has the epilogue (both tail layouts of the
    # bandwidth-bound kernel, the MFMA GEMM, the element-wise fallback, the kernels for K-contiguous weights)
    announce('w8a16 bias', m, k, n, layout)
    a, q, s = _int_case(m * 7 + n, m, k, n)
    rng = np.random.default_rng(n)
    b = (rng.integers(-64, 65, n) / 1024.0).astype(np.float16)
    product = ((a.astype(np.int64) @ q.astype(np.int64)).astype(np.float64) * s.astype(np.float64)[None, :]).astype(np.float32).astype(np.float16)
    want = (product.astype(np.float32) + b.astype(np.float32)[None, :]).astype(np.float16)
    tq = dev(q)
    if layout == 'nk':
        tq = quant.to_decode_layout(tq)
    got = host(quant.symmetric_quant_matmul(dev(a), tq, dev(s), dev(b)))
    assert np.array_equal(got, want)
    plain = host(quant.symmetric_quant_matmul(dev(a), tq, dev(s)))  # the same call without bias is unchanged
    assert np.array_equal(plain, product)
    with pytest.raises(ValueError, match='bias must be'):
        quant.symmetric_quant_matmul(dev(a), tq, dev(s), dev(b[:-1]))


@pytest.mark.parametrize('m,k,n,layout', [(1, 4096, 11008, 'kn'), (8, 2048, 4096, 'kn'), (16, 1024, 768, 'kn'), (40, 2048, 520, 'kn'),
                                          (300, 512, 1100, 'kn'), (2, 100, 40, 'kn'), (1, 4096, 1024, 'nk'), (16, 1024, 512, 'nk'),
                                          (40, 2048, 520, 'nk')])
def test_fused_bias_gives_the_bits_of_matmul_then_add(m, k, n, layout):
    # random operands, where one rounding and two differ in the last bit of some outputs: the fused epilogue rounds the
    # scaled sum to float16 and adds the bias to that (python/hidet/graph/ops/quant/matmul_f16_i8.py:95-99: the reference's
    # epilogue fusion applies the add to the value the template stores), so it equals the unfused pair bit for bit
    announce('w8a16 fused bias == matmul + add', m, k, n, layout)
    a32, w32 = O.make_inputs(m * 11 + n, m, k, n)
    q, s32 = O.symmetric_quantize(w32, 'int8', dims=0)
    a, s = a32.astype(np.float16), s32.astype(np.float16)
    b = (np.random.default_rng(n).standard_normal(n) * 0.5).astype(np.float16)
    tq = dev(q)
    if layout == 'nk':
        tq = quant.to_decode_layout(tq)
    fused = host(quant.symmetric_quant_matmul(dev(a), tq, dev(s), dev(b)))
    plain = host(quant.symmetric_quant_matmul(dev(a), tq, dev(s)))
    want = (plain.astype(np.float32) + b.astype(np.float32)[None, :]).astype(np.float16)  # a float16 add, rounded once
    assert np.array_equal(fused.view(np.uint16), want.view(np.uint16))
    single = (clib.quant_matmul_f32acc(a, q, s).astype(np.float64))  # sanity: the bias really changed something
    assert not np.array_equal(fused, plain) and single.shape == fused.shape


@pytest.mark.parametrize('m,k,n,parts', [(2, 8192, 16384, 32), (16, 4096, 8192, 16), (1, 16384, 4096, 64)])
def test_more_workgroups_than_the_chip_holds(m, k, n, parts):
    # a forced K split far beyond one round (2048 / 512 / 1024 workgroups of 8 waves on 256 CUs): the workgroup that
    # collects a column tile's partial sums is the last of that tile in launch order, so everything it waits for was
    # started before it; the result is exact, twice in a row (the mailbox is clean again after the first call)
    announce('w8a16 oversubscribed', m, k, n, parts)
    a, q, s = _int_case(m + k, m, k, n)
    want = ((a.astype(np.int64) @ q.astype(np.int64)).astype(np.float64) * s.astype(np.float64)[None, :])
    ta, tq, ts = dev(a), dev(q), dev(s)
    for _ in range(2):
        c = torch.full((m, n), float('nan'), dtype=torch.float16, device='cuda')
        ws = hidet_amd.ffi.workspace(ta.device)
        hidet_amd.ffi.call('hidet_symmetric_quant_matmul_f16_i8', ta, tq, ts, c, m, k, n, k, parts, ws, ws.numel(),
                           hidet_amd.ffi.current_stream(ta.device))
        assert np.array_equal(host(c), want.astype(np.float32).astype(np.float16))


def test_parallel_k_search():
    # hidet.option.parallel_k('search') (reference resolve.py:53-92): the candidates are timed on the GPU, the winner is
    # one of them (or 0, the library's own plan), is remembered per shape, and the result equals the unsplit one
    from hidet_amd.graph.ops.quant import resolve
    announce('w8a16 parallel_k search')
    a, q, s = _int_case(11, 2, 1024, 512)
    ta, tq, ts = dev(a), dev(q), dev(s)
    want = host(quant.symmetric_quant_matmul(ta, tq, ts))
    resolve._SEARCH_CACHE.clear()
    hidet_amd.option.parallel_k('search')
    try:
        got = host(quant.symmetric_quant_matmul(ta, tq, ts))
        hint = resolve.resolve_parallel_k_parts('search', ta, tq)
    finally:
        hidet_amd.option.parallel_k('disabled')
    assert hint in [0] + resolve.SEARCH_CANDIDATES
    assert resolve._SEARCH_CACHE == {((2, 1024), (1024, 512)): hint}
    assert np.array_equal(got, want)  # small integers: exact whatever the split


def test_deterministic_and_counters_reset():
    announce('w8a16 determinism')
    a, q, s = _case(1, 4, 4096, 1024)
    ta, tq, ts = dev(a), dev(q), dev(s)
    first = quant.symmetric_quant_matmul(ta, tq, ts)
    for _ in range(5):
        assert torch.equal(quant.symmetric_quant_matmul(ta, tq, ts), first)
    ws = hidet_amd.ffi.workspace(ta.device)
    torch.cuda.synchronize()
    assert int(ws[: (16 << 20) + (64 << 10)].view(torch.int32).abs().sum()) == 0  # counters and the split-K mailbox are back at zero


def test_strided_rows_and_unaligned_shapes():
    announce('w8a16 strided / unaligned')
    a, q, s = _case(2, 4, 512, 256)
    big = torch.zeros(4, 1024, dtype=torch.float16, device='cuda')
    big[:, 256:768] = dev(a)
    got = host(quant.symmetric_quant_matmul(big[:, 256:768], dev(q), dev(s)))
    assert O.max_rel_err(got, clib.quant_matmul_f32acc(a, q, s)) <= 2e-3
    # K not a multiple of 8 (activation rows cannot be loaded 16 bytes at a time), N not a multiple of 16
    for (m, k, n) in ((2, 100, 64), (3, 64, 40), (1, 34, 6)):
        a, q, s = _case(3, m, k, n)
        got = host(quant.symmetric_quant_matmul(dev(a), dev(q), dev(s)))
        assert O.max_rel_err(got, clib.quant_matmul_f32acc(a, q, s)) <= 2e-3, (m, k, n)


@pytest.mark.parametrize('ws_bytes', [0, 1024, (64 << 10) + (2 << 20)])
def test_small_workspace_means_fewer_k_slices(ws_bytes):
    # the plan for 8 x 4096 x 4096 wants 8 K slices = 1 MiB of partial tiles in the mailbox (a quarter of what follows
    # the 64 KiB of counters); with less the launcher takes the K split that fits (none without a workspace) and the
    # result stays exact
    announce('w8a16 small workspace', ws_bytes)
    m, k, n = 8, 4096, 4096
    a, q, s = _int_case(77, m, k, n)
    want = ((a.astype(np.int64) @ q.astype(np.int64)).astype(np.float64) * s.astype(np.float64)[None, :])
    ta, tq, ts = dev(a), dev(q), dev(s)
    c = torch.full((m, n), float('nan'), dtype=torch.float16, device='cuda')
    ws = torch.zeros(max(ws_bytes, 16), dtype=torch.uint8, device='cuda')
    hidet_amd.ffi.call('hidet_symmetric_quant_matmul_f16_i8', ta, tq, ts, c, m, k, n, k, 0, ws if ws_bytes else None,
                       ws_bytes, hidet_amd.ffi.current_stream(ta.device))
    assert np.array_equal(host(c), want.astype(np.float32).astype(np.float16))


# ---- prefill GEMM (M > 16 goes to the MFMA kernel) ------------------------------------------------------------

@pytest.mark.parametrize('m,k,n', [(128, 64, 256), (256, 512, 512), (65, 128, 64), (200, 200, 260), (130, 72, 12),
                                   (512, 1024, 1100), (256, 2048, 520), (384, 4096, 1100), (1100, 1536, 2100),
                                   (17, 128, 64), (40, 2048, 520), (64, 64, 256),
                                   (40, 100, 64), (33, 72, 48)])  # the last two: K not a multiple of 64, 16-row passes
def test_gemm_exact_on_small_integers(m, k, n):
    announce('w8a16 gemm exact', m, k, n)
    a, q, s = _int_case(m + n, m, k, n)
    want = ((a.astype(np.int64) @ q.astype(np.int64)).astype(np.float64) * s.astype(np.float64)[None, :])
    got = host(quant.symmetric_quant_matmul(dev(a), dev(q), dev(s)))
    assert np.array_equal(got, want.astype(np.float32).astype(np.float16))


@pytest.mark.parametrize('m,k,n', [(128, 4096, 512), (300, 1000, 528), (1024, 512, 768)])
def test_gemm_parity_with_oracle(m, k, n):
    announce('w8a16 gemm parity', m, k, n)
    a, q, s = _case(0, m, k, n)
    ref = clib.quant_matmul_f32acc(a, q, s)
    got = host(quant.symmetric_quant_matmul(dev(a), dev(q), dev(s)))
    err = O.max_rel_err(got, ref)
    print('max_rel_err', err)
    assert err <= TOL and err <= 2e-3


@pytest.mark.parametrize('n', [11008, 12288])
def test_gemm_full_size_prefill_rows_sample(n):
    # M = 2048, K = 4096 at the benchmark's two weight shapes: the oracle is evaluated on a sample of rows
    # that touches the first, last and interior row tiles; the skinny kernel (already checked against the
    # oracle) must agree with the GEMM kernel on the same rows, and batching must not change a row.
    m, k = 2048, 4096
    announce('w8a16 gemm full size', m, k, n)
    a, q, s = _case(0, m, k, n)
    ta, tq, ts = dev(a), dev(q), dev(s)
    got = quant.symmetric_quant_matmul(ta, tq, ts)
    rows = np.array([0, 1, 15, 16, 127, 128, 129, 1000, 1023, 1024, 1500, 2046, 2047])
    ref = clib.quant_matmul_f32acc(a[rows], q, s)
    err = O.max_rel_err(host(got)[rows], ref)
    print('max_rel_err', err)
    assert err <= TOL and err <= 2e-3
    skinny = quant.symmetric_quant_matmul(ta[torch.from_numpy(rows).cuda()], tq, ts)
    assert O.max_rel_err(host(skinny), host(got)[rows]) <= 1e-3
    # batch axes are folded into M: [4, 512, K] gives the same numbers as [2048, K]
    got3 = quant.symmetric_quant_matmul(ta.reshape(4, 512, k), tq, ts)
    assert tuple(got3.shape) == (4, 512, n) and torch.equal(got3.reshape(m, n), got)


def test_gemm_k_split_matches_unsplit_and_is_deterministic():
    # With a workspace and fewer tiles than CUs, every tile is computed in K ranges by several workgroups and summed in
    # a fixed order; without a workspace every tile is computed whole. Both must agree to fp32 rounding, the split
    # result must not change from run to run, and the arrival counters must be back at zero.
    m, k, n = 128, 4096, 11008
    announce('w8a16 gemm k split', m, k, n)
    a, q, s = _case(1, m, k, n)
    ta, tq, ts = dev(a), dev(q), dev(s)
    stream = hidet_amd.ffi.current_stream(ta.device)
    whole = torch.empty(m, n, dtype=torch.float16, device='cuda')
    hidet_amd.ffi.call('hidet_symmetric_quant_matmul_f16_i8', ta, tq, ts, whole, m, k, n, k, 0, None, 0, stream)
    assert O.max_rel_err(host(whole), clib.quant_matmul_f32acc(a, q, s)) <= 2e-3
    first = quant.symmetric_quant_matmul(ta, tq, ts)
    assert O.max_rel_err(host(first), host(whole)) <= 1e-3
    for _ in range(3):
        assert torch.equal(quant.symmetric_quant_matmul(ta, tq, ts), first)
    ws = hidet_amd.ffi.workspace(ta.device)
    torch.cuda.synchronize()
    assert int(ws[: 64 << 10].view(torch.int32).abs().sum()) == 0


@pytest.mark.parametrize('m,k,n', [(1, 4096, 11008), (1, 11008, 4096), (16, 4096, 4096), (3, 512, 48), (7, 144, 20), (1, 16, 2),
                                   (20, 1024, 264), (32, 4096, 512), (2, 384, 32), (5, 1152, 8200), (4, 2176, 8192),
                                   (9, 1040, 40), (9, 1152, 8200), (16, 4096, 11008), (5, 1024, 8192), (21, 1280, 8256), (12, 8192, 8200), (3, 2048, 64),
                                   (16, 1024, 8192), (2, 16384, 48), (3, 32768, 16),
                                   # more than 16 rows: the MFMA GEMM on the same layout (row blocks left out, K ranges, ragged edges)
                                   (17, 4096, 11008), (100, 512, 264), (129, 4096, 512), (300, 256, 1056), (520, 2048, 264),
                                   (33, 4096, 520), (700, 1024, 2048), (64, 192, 8), (40, 1040, 64)])
def test_k_contiguous_weights_exact(m, k, n):
    # the [K, N] weight held with strides (1, K): same operator, same results, the kernel that reduces along the
    # contiguous axis; small integers make every product and partial sum exact.  K a multiple of 128 or not, 4 and 8
    # waves per workgroup, waves with an empty K range, a second 16-row pass, activations fetched directly (1-2 rows)
    # and through LDS, 16 and 32 columns per workgroup.
    announce('w8a16 k-contiguous', m, k, n)
    a, q, s = _int_case(m * 31 + n, m, k, n)
    want = ((a.astype(np.int64) @ q.astype(np.int64)).astype(np.float64) * s.astype(np.float64)[None, :])
    want = want.astype(np.float32).astype(np.float16)
    w_nk = quant.to_decode_layout(dev(q))
    assert tuple(w_nk.shape) == (k, n) and w_nk.stride() == (1, k)
    ta, ts = dev(a), dev(s)
    # the operator: picks this kernel for a few rows and copies the weight to the row-major layout otherwise
    assert np.array_equal(host(quant.symmetric_quant_matmul(ta, w_nk, ts)), want)
    # the entry point itself, whatever the row count
    c = torch.full((m, n), float('nan'), dtype=torch.float16, device='cuda')
    ws = hidet_amd.ffi.workspace(c.device)
    hidet_amd.ffi.call('hidet_symmetric_quant_matmul_f16_i8_nk', ta, w_nk, ts, c, m, k, n, k, k, ws, ws.numel(),
                       hidet_amd.ffi.current_stream(c.device))
    assert np.array_equal(host(c), want)


def test_k_contiguous_weights_padded_rows():
    # rows of the stored [N, K] matrix further apart than K (a slice of a wider matrix), activations with a row stride
    announce('w8a16 k-contiguous padded')
    m, k, n, ldw, lda = 3, 640, 72, 1024, 768
    a, q, s = _int_case(77, m, k, n)
    want = ((a.astype(np.int64) @ q.astype(np.int64)).astype(np.float64) * s.astype(np.float64)[None, :])
    wide = torch.full((n, ldw), 99, dtype=torch.int8, device='cuda')
    wide[:, :k] = dev(q).t()
    abuf = torch.full((m, lda), 7.0, dtype=torch.float16, device='cuda')
    abuf[:, :k] = dev(a)
    got = host(quant.symmetric_quant_matmul(abuf[:, :k], wide[:, :k].t(), dev(s)))
    assert np.array_equal(got, want.astype(np.float32).astype(np.float16))


def test_k_contiguous_weights_parity_and_fallback():
    announce('w8a16 k-contiguous parity')
    a, q, s = _case(0, 1, 4096, 11008)
    ref = clib.quant_matmul_f32acc(a, q, s)
    w_nk = quant.to_decode_layout(dev(q))
    got = host(quant.symmetric_quant_matmul(dev(a), w_nk, dev(s)))
    assert O.max_rel_err(got, ref) <= 2e-3
    # many rows, or a K that is not a multiple of 16: the weight is copied to the row-major layout and the result is the same
    a2, q2, s2 = _int_case(5, 100, 72, 64)
    want = ((a2.astype(np.int64) @ q2.astype(np.int64)).astype(np.float64) * s2.astype(np.float64)[None, :])
    got2 = host(quant.symmetric_quant_matmul(dev(a2), quant.to_decode_layout(dev(q2)), dev(s2)))
    assert np.array_equal(got2, want.astype(np.float32).astype(np.float16))
    # the C entry point refuses what it cannot take
    from hidet_amd import ffi
    bad = torch.zeros(8, 24, device='cuda', dtype=torch.int8)
    with pytest.raises(hidet_amd.BackendException):
        ffi.call('hidet_symmetric_quant_matmul_f16_i8_nk', torch.zeros(1, 24, device='cuda', dtype=torch.float16), bad,
                 torch.zeros(8, device='cuda', dtype=torch.float16), torch.zeros(1, 8, device='cuda', dtype=torch.float16),
                 1, 24, 8, 24, 24, None, 0, ffi.current_stream(bad.device))
