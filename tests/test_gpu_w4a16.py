"""GPU parity of group-wise int4 quantization (bit-exact) and the W4A16 matmul (max relative error <= 1e-2
against the oracle: dequantize to the 16-bit type, then matmul with fp32 accumulation).

The reference has no operator for this configuration: PARITY UNPINNED by reference tests; the oracle is pinned
by closed forms and the reference's packing convention (tests/test_oracle.py)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from hidet_amd.graph.ops import quant
from gpu_util import announce, dev, host

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _bits16(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize('k,n,g,sdt', [(256, 64, 128, 'bfloat16'), (512, 200, 64, 'float16'), (4096, 11008, 128, 'bfloat16'),
                                       (128, 2, 32, 'bfloat16')])
def test_group_quantize_int4_bit_exact(k, n, g, sdt):
    announce('int4 quantize', k, n, g, sdt)
    _, w = O.make_inputs(0, 1, k, n)
    w[0:g, 1] = 0  # an all-zero group: scale 0, codes 0
    packed, scales = quant.symmetric_group_quantize_int4(dev(w), g, sdt)
    p0, s0, q0 = O.group_quantize_int4(w, g, sdt)
    assert np.array_equal(host(packed), p0)
    want = O.bf16_bits(s0) if sdt == 'bfloat16' else s0.view(np.uint16)
    assert np.array_equal(_bits16(scales), want)
    assert np.array_equal(O.unpack_int4(host(packed)), q0)


def _case(seed, m, k, n, g, dtype):
    a32, w = O.make_inputs(seed, m, k, n)
    packed, scales, q = O.group_quantize_int4(w, g, dtype)
    if dtype == 'bfloat16':
        a = O.to_bf16(a32)
        return a, packed, scales, dev(a, torch.bfloat16), dev(packed), dev(scales, torch.bfloat16)
    a = a32.astype(np.float16)
    return a, packed, scales, dev(a), dev(packed), dev(scales)


@pytest.mark.parametrize('m,k,n,g', [(1, 256, 256, 128), (3, 512, 768, 128), (16, 4096, 512, 128), (1, 384, 272, 32),
                                     (7, 128, 48, 64), (2, 96, 6, 32), (1, 4096, 11008, 128), (16, 4096, 11008, 128)])
@pytest.mark.parametrize('dtype', ['bfloat16', 'float16'])
def test_skinny_parity(m, k, n, g, dtype):
    announce('w4a16 skinny', m, k, n, g, dtype)
    a, packed, scales, ta, tp, ts = _case(0, m, k, n, g, dtype)
    ref = O.w4a16_matmul(a, packed, scales, g, dtype)
    got = host(quant.symmetric_quant_matmul_w4a16(ta, tp, ts, g))
    err = O.max_rel_err(got, ref)
    print('max_rel_err', err)
    assert err <= TOL
    assert err <= (8e-3 if dtype == 'bfloat16' else 2e-3)  # bf16 output rounding is 2^-9 relative


@pytest.mark.parametrize('m,k,n,g', [(128, 256, 256, 128), (65, 128, 264, 32), (512, 4096, 1024, 128), (300, 512, 520, 64),
                                     (33, 4096, 512, 128), (40, 512, 264, 64), (24, 512, 256, 128),
                                     # 256-row tiles widened once per workgroup: a short last tile, K split with mostly
                                     # empty tiles, a ragged last column tile, waves without rows
                                     (129, 4096, 512, 128), (500, 512, 544, 64), (1000, 256, 1056, 128),
                                     (40, 4096, 544, 128), (70, 1024, 2080, 64)])
@pytest.mark.parametrize('dtype', ['bfloat16', 'float16'])
def test_gemm_parity(m, k, n, g, dtype):
    announce('w4a16 gemm', m, k, n, g, dtype)
    a, packed, scales, ta, tp, ts = _case(1, m, k, n, g, dtype)
    ref = O.w4a16_matmul(a, packed, scales, g, dtype)
    got = host(quant.symmetric_quant_matmul_w4a16(ta, tp, ts, g))
    err = O.max_rel_err(got, ref)
    print('max_rel_err', err)
    assert err <= TOL
    assert err <= (8e-3 if dtype == 'bfloat16' else 2e-3)


def test_exact_on_small_integers():
    announce('w4a16 exact')
    rng = np.random.default_rng(21)
    for (m, k, n) in ((4, 256, 256), (128, 256, 128), (200, 4096, 256), (48, 4096, 1024)):  # the last two split K
        a = rng.integers(-3, 4, (m, k)).astype(np.float32)
        q = rng.integers(-8, 8, (k, n)).astype(np.int8)  # -8 is representable and must decode correctly
        scales = (2.0 ** rng.integers(-3, 1, (k // 128, n))).astype(np.float32)
        want = np.zeros((m, n))
        for g in range(k // 128):
            want += (a[:, g * 128:(g + 1) * 128].astype(np.int64) @ q[g * 128:(g + 1) * 128].astype(np.int64)) * scales[g]
        got = host(quant.symmetric_quant_matmul_w4a16(dev(a, torch.bfloat16), dev(O.pack_int4(q)), dev(scales, torch.bfloat16), 128))
        assert np.array_equal(got, O.to_bf16(want.astype(np.float32))), (m, k, n)


@pytest.mark.parametrize('m,k,n,g', [(1, 4096, 11008, 128), (16, 4096, 11008, 128), (2, 1024, 4096, 256), (5, 384, 40, 128),
                                     (9, 1152, 72, 128), (3, 128, 16, 128), (21, 2048, 528, 1024), (1, 11008 - 11008 % 128, 4096, 128),
                                     (2, 4096, 4096, 128)])  # the last two: sixteen waves per workgroup
@pytest.mark.parametrize('dtype', ['bfloat16', 'float16'])
def test_decode_layout_parity_and_same_result_as_row_major(m, k, n, g, dtype):
    # the weight repacked K-contiguous for decode: same operator, compared with the oracle and with the row-major kernels
    # (4 and 8 waves, direct and LDS-staged activations, waves with an empty K range, a second 16-row pass, groups of
    # several steps)
    announce('w4a16 decode layout', m, k, n, g, dtype)
    a, packed, scales, ta, tp, ts = _case(m * 13 + n, m, k, n, g, dtype)
    tp_nk = quant.to_decode_layout_int4(tp)
    assert tuple(tp_nk.shape) == (n, k // 2) and tp_nk.is_contiguous()
    got = host(quant.symmetric_quant_matmul_w4a16_decode(ta, tp_nk, ts, g))
    ref = O.w4a16_matmul(a, packed, scales, g, dtype)
    err = O.max_rel_err(got, ref)
    assert err <= TOL, err
    other = host(quant.symmetric_quant_matmul_w4a16(ta, tp, ts, g))
    assert O.max_rel_err(got, other) <= 1e-2


def test_decode_layout_exact_and_errors():
    announce('w4a16 decode layout exact')
    rng = np.random.default_rng(11)
    for m, k, n, g in ((1, 256, 32, 128), (4, 1280, 8200, 256), (16, 4096, 64, 128)):
        a = rng.integers(-4, 5, (m, k)).astype(np.float32)
        q = rng.integers(-7, 8, (k, n)).astype(np.int8)
        s = np.exp2(rng.integers(-3, 2, (k // g, n))).astype(np.float32)
        packed = O.pack_int4(q)
        want = np.zeros((m, n), np.float64)
        for gi in range(k // g):
            want += (a[:, gi * g:(gi + 1) * g].astype(np.float64) @ q[gi * g:(gi + 1) * g].astype(np.float64)) * s[gi][None, :]
        tp_nk = quant.to_decode_layout_int4(dev(packed))
        got = quant.symmetric_quant_matmul_w4a16_decode(dev(a, torch.bfloat16), tp_nk, dev(s, torch.bfloat16), g)
        assert np.array_equal(host(got), O.to_bf16(want.astype(np.float32))), (m, k, n)
    import hidet_amd
    with pytest.raises(hidet_amd.BackendException, match='multiple of 128'):
        quant.symmetric_quant_matmul_w4a16_decode(torch.zeros(1, 64, device='cuda', dtype=torch.bfloat16),
                                                  torch.zeros(16, 32, device='cuda', dtype=torch.uint8),
                                                  torch.zeros(1, 16, device='cuda', dtype=torch.bfloat16), 64)
    with pytest.raises(ValueError, match='scales must be'):
        quant.symmetric_quant_matmul_w4a16_decode(torch.zeros(1, 128, device='cuda', dtype=torch.bfloat16),
                                                  torch.zeros(16, 64, device='cuda', dtype=torch.uint8),
                                                  torch.zeros(2, 16, device='cuda', dtype=torch.bfloat16), 128)


@pytest.mark.parametrize('m,k,n,g', [(1, 4096, 11008, 128), (16, 4096, 11008, 128), (3, 512, 272, 64), (20, 1024, 528, 128),
                                     (1, 256, 40, 128),                     # N not a multiple of 16: the one-thread-per-element kernel
                                     (48, 4096, 1024, 128), (300, 512, 544, 64), (512, 4096, 1024, 128), (768, 2048, 11008, 128)])
@pytest.mark.parametrize('dtype', ['bfloat16', 'float16'])
def test_bias_exact_and_the_bits_of_matmul_then_add(m, k, n, g, dtype):
    """bias[n] of the output's type, added to the rounded result (two roundings). Small integers, power-of-two scales and
    biases that are multiples of 1/8: integer arithmetic says what both roundings must give; and on random operands the
    fused call returns the bits of the plain call followed by torch's add in the same type. Up to 32 rows the add rides
    in the kernel's epilogue, above it follows the GEMM as a pass of its own."""
    announce('w4a16 bias', m, k, n, g, dtype)
    tdt = torch.bfloat16 if dtype == 'bfloat16' else torch.float16
    rng = np.random.default_rng(m + n)
    a = rng.integers(-3, 4, (m, k)).astype(np.float32)
    q = rng.integers(-8, 8, (k, n)).astype(np.int8)
    scales = (2.0 ** rng.integers(-3, 1, (k // g, n))).astype(np.float32)
    bias = (rng.integers(-40, 41, n) / 8.0).astype(np.float32)
    want = np.zeros((m, n))
    for gi in range(k // g):
        want += (a[:, gi * g:(gi + 1) * g].astype(np.float64) @ q[gi * g:(gi + 1) * g].astype(np.float64)) * scales[gi]
    if dtype == 'bfloat16':
        want = O.to_bf16(O.to_bf16(want.astype(np.float32)) + bias)
    else:
        with np.errstate(over='ignore'):
            want = (want.astype(np.float32).astype(np.float16).astype(np.float32) + bias).astype(np.float16).astype(np.float32)
    tp, ts, tb = dev(O.pack_int4(q)), dev(scales, tdt), dev(bias, tdt)
    got = quant.symmetric_quant_matmul_w4a16(dev(a, tdt), tp, ts, g, bias=tb)
    assert np.array_equal(got.float().cpu().numpy(), want)
    # random operands: fused == plain + add, bit for bit
    _, _, _, ta, tp, ts = _case(7, m, k, n, g, dtype)
    tb = dev(np.random.default_rng(3).normal(0, 1, n).astype(np.float32), tdt)
    fused = quant.symmetric_quant_matmul_w4a16(ta, tp, ts, g, bias=tb)
    plain = quant.symmetric_quant_matmul_w4a16(ta, tp, ts, g)
    assert torch.equal(fused, plain + tb)


def test_bias_argument_errors():
    a = torch.zeros(2, 128, device='cuda', dtype=torch.bfloat16)
    packed = torch.zeros(128, 8, device='cuda', dtype=torch.uint8)
    scales = torch.zeros(1, 16, device='cuda', dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        quant.symmetric_quant_matmul_w4a16(a, packed, scales, 128, bias=torch.zeros(16, device='cuda', dtype=torch.float16))
    with pytest.raises(ValueError):
        quant.symmetric_quant_matmul_w4a16(a, packed, scales, 128, bias=torch.zeros(8, device='cuda', dtype=torch.bfloat16))


def test_k_split_is_deterministic():
    m, k, n, g = 129, 4096, 512, 128
    announce('w4a16 k split twice', m, k, n)
    _, _, _, ta, tp, ts = _case(3, m, k, n, g, 'bfloat16')
    first = host(quant.symmetric_quant_matmul_w4a16(ta, tp, ts, g))
    for _ in range(3):
        assert np.array_equal(host(quant.symmetric_quant_matmul_w4a16(ta, tp, ts, g)), first)


@pytest.mark.parametrize('m,k,n', [(768, 2048, 11008), (1536, 1024, 11008), (700, 4096, 11008)])
def test_runs_across_the_tiles(m, k, n):
    """33 (65) tiles of 256 x 128 on the busiest XCD, one (one) more than whole rounds of 32 workgroups: the launcher deals
    every XCD's (tile, stage) units to 32 workgroups in equal runs, and tiles computed in pieces are summed by the last
    workgroup to arrive. Small integers and power-of-two scales: every sum is exact whatever the pieces, so the
    result must equal integer arithmetic bit for bit; and twice the same."""
    announce('w4a16 runs across tiles', m, k, n)
    rng = np.random.default_rng(m + k)
    a = rng.integers(-3, 4, (m, k)).astype(np.float32)
    q = rng.integers(-8, 8, (k, n)).astype(np.int8)
    scales = (2.0 ** rng.integers(-3, 1, (k // 128, n))).astype(np.float32)
    ta, tp, ts = dev(a, torch.bfloat16), dev(O.pack_int4(q)), dev(scales, torch.bfloat16)
    got = host(quant.symmetric_quant_matmul_w4a16(ta, tp, ts, 128))
    rows = np.unique(np.concatenate([np.arange(0, m, 37), [255, 256, 511, 512, m - 1]]))
    want = np.zeros((len(rows), n))
    for g in range(k // 128):
        want += (a[rows, g * 128:(g + 1) * 128].astype(np.int64) @ q[g * 128:(g + 1) * 128].astype(np.int64)) * scales[g]
    assert np.array_equal(got[rows], O.to_bf16(want.astype(np.float32)))
    assert np.array_equal(host(quant.symmetric_quant_matmul_w4a16(ta, tp, ts, 128)), got)
    # against the rows computed one 16-row batch at a time by the bandwidth-bound kernel (no tiles, no pieces)
    idx = torch.from_numpy(rows[:16]).cuda()
    assert np.array_equal(host(quant.symmetric_quant_matmul_w4a16(ta[idx].contiguous(), tp, ts, 128)), got[rows[:16]])


def test_runs_across_the_tiles_random_operands():
    m, k, n, g = 768, 2048, 11008, 128
    announce('w4a16 runs across tiles, random', m, k, n)
    a, packed, scales, ta, tp, ts = _case(5, m, k, n, g, 'bfloat16')
    got = host(quant.symmetric_quant_matmul_w4a16(ta, tp, ts, g))
    rows = np.array([0, 100, 255, 256, 300, 511, 512, 640, 767])
    ref = O.w4a16_matmul(a[rows], packed, scales, g, 'bfloat16')
    err = O.max_rel_err(got[rows], ref)
    print('max_rel_err', err)
    assert err <= 8e-3


def test_full_size_prefill_rows_sample():
    m, k, n, g = 512, 4096, 11008, 128
    announce('w4a16 full size', m, k, n)
    a, packed, scales, ta, tp, ts = _case(0, m, k, n, g, 'bfloat16')
    got = quant.symmetric_quant_matmul_w4a16(ta, tp, ts, g)
    rows = np.array([0, 15, 16, 63, 64, 200, 255, 256, 511])
    ref = O.w4a16_matmul(a[rows], packed, scales, g, 'bfloat16')
    err = O.max_rel_err(host(got)[rows], ref)
    print('max_rel_err', err)
    assert err <= 8e-3
    skinny = quant.symmetric_quant_matmul_w4a16(ta[torch.from_numpy(rows).cuda()], tp, ts, g)
    assert O.max_rel_err(host(skinny), host(got)[rows]) <= 8e-3
