"""GPU parity of the FP8 e4m3 path: per-tensor quantization bit-exact against the oracle, matmul_f8 /
matmul_f8_scaled exact on the reference's integer-valued test recipes
(tests/operators_core/test_matmul.py:250-373), and max relative error <= 3e-2 on N(0,1) data."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from hidet_amd.graph.ops.matmul import matmul_f8 as F8
from gpu_util import announce, dev, host

pytestmark = pytest.mark.gpu
TOL = 3e-2  # max relative error (normalised by max |ref|) for fp8 matmuls


def codes_of(t: torch.Tensor) -> np.ndarray:
    return t.view(torch.uint8).cpu().numpy()


def f8(codes: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(codes)).cuda().view(torch.float8_e4m3fn)


def test_quantize_per_tensor_bit_exact():
    announce('fp8 quantize')
    rng = np.random.default_rng(3)
    tab = O.e4m3_decode(np.arange(0, 0x7F, dtype=np.uint8)).astype(np.float64)
    mids = ((tab[:-1] + tab[1:]) / 2).astype(np.float32)
    # amax = 448 makes the scale exactly 1, so the codes are e4m3(x): every tie and neighbour of a tie
    x = np.concatenate([np.array([448.0, -448.0], dtype=np.float32), tab.astype(np.float32), mids, -mids,
                        np.nextafter(mids, np.float32(1e9)), np.nextafter(mids, np.float32(-1e9)),
                        rng.uniform(-448, 448, 20000).astype(np.float32),
                        (rng.standard_normal(20000) * 10.0 ** rng.uniform(-6, 1, 20000)).astype(np.float32)])
    x = x[np.abs(x) <= 448]
    codes, scale = F8.fp8_quantize_per_tensor(dev(x))
    c0, s0 = O.fp8_quantize_per_tensor(x)
    assert float(scale.item()) == 1.0 == float(s0)
    assert np.array_equal(codes_of(codes), c0)
    for shape, dt in (((300, 70), torch.float32), ((64, 64), torch.bfloat16), ((1, 5), torch.float16), ((0,), torch.float32),
                      # more than 65536 elements: the two-pass kernels; 16-bit inputs with and without whole 16-byte groups
                      ((400, 200), torch.float32), ((513, 136), torch.float16), ((513, 136), torch.bfloat16),
                      ((257, 260), torch.bfloat16), ((2100, 1024), torch.bfloat16)):
        y = (rng.standard_normal(shape) * 3).astype(np.float32)
        ty = dev(y).to(dt)
        y = ty.float().cpu().numpy()
        codes, scale = F8.fp8_quantize_per_tensor(ty)
        c0, s0 = O.fp8_quantize_per_tensor(y)
        assert np.float32(scale.item()) == s0 and np.array_equal(codes_of(codes), c0), (shape, dt)
    z, zs = F8.fp8_quantize_per_tensor(torch.zeros(8, 8, device='cuda'))
    assert zs.item() == 0 and not codes_of(z).any()


def test_quantize_per_tensor_every_rounding_boundary():
    # amax = 448 makes the scale exactly 1, so the codes are e4m3(x): every midpoint between two neighbouring e4m3 values
    # and its two float32 neighbours, both signs, plus the values themselves. The fast kernel converts in hardware, the
    # oracle in integer arithmetic; ties must go to even in both.
    announce('fp8 quantize rounding boundaries')
    vals = O.e4m3_decode(np.arange(0, 0x7F, dtype=np.uint8)).astype(np.float32)      # 0 .. 448, ascending
    mids = ((vals[:-1].astype(np.float64) + vals[1:].astype(np.float64)) / 2).astype(np.float32)
    pts = np.concatenate([vals, mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9)),
                          np.array([2.0 ** -10, 2.0 ** -10 * 0.99, 2.0 ** -11, 1e-12, 447.99, 440.0], dtype=np.float32)])
    pts = np.concatenate([pts, -pts]).astype(np.float32)
    pts = np.concatenate([pts, np.zeros((-pts.size) % 4, dtype=np.float32)])          # multiple of 4: the vector kernel
    big = np.tile(pts, 70000 // pts.size + 1)   # more than 65536 elements: the two-pass kernels instead of the one-launch one
    assert big.size > 65536 and big.size % 4 == 0
    for x in (pts, pts[:-1], big, big[:-1]):                                          # ... and the scalar ones
        codes, scale = F8.fp8_quantize_per_tensor(dev(x))
        assert scale.item() == 1.0
        assert np.array_equal(codes_of(codes), O.e4m3_encode(x))
    for dt in (torch.float16, torch.bfloat16):                                        # narrow inputs through both paths
        for x in (pts, big):
            t = dev(x).to(dt)
            codes, scale = F8.fp8_quantize_per_tensor(t)
            assert scale.item() == 1.0
            assert np.array_equal(codes_of(codes), O.e4m3_encode(t.float().cpu().numpy()))


@pytest.mark.parametrize('a_shape, b_shape', [[[256, 128], [256, 128]], [[4096, 4096], [4096, 4096]], [[512, 256], [128, 256]],
                                              [[1, 256], [48, 256]], [[16, 1024], [200, 1024]], [[100, 48], [36, 48]],
                                              [[300, 272], [260, 272]],
                                              # 512 tiles of 256 x 256 (two rounds of workgroups), 2 and 1 k-steps each; ragged edges
                                              [[4096, 256], [8192, 256]], [[4096, 128], [8192, 128]], [[4000, 384], [8100, 384]],
                                              # few tiles, long K: tiles computed in K ranges; short matrices in tall tiles
                                              [[17, 4096], [2048, 4096]], [[64, 8192], [1024, 8192]], [[100, 2048], [520, 2048]],
                                              [[200, 4096], [1152, 4096]], [[300, 2048], [1024, 2048]]])
def test_matmul_f8_reference_recipe(a_shape, b_shape):
    # tests/operators_core/test_matmul.py:250-288: randint(-3, 3) inputs; the exact integer result is the answer
    announce('matmul_f8', a_shape, b_shape)
    rng = np.random.default_rng(41)
    ai = rng.integers(-3, 3, a_shape)
    bi = rng.integers(-3, 3, b_shape)
    ta, tb = f8(O.e4m3_encode(ai.astype(np.float32))), f8(O.e4m3_encode(bi.astype(np.float32)))
    exact = (ai.astype(np.float64) @ bi.astype(np.float64).T).astype(np.int64)  # float64 BLAS: exact on these integers
    got32 = F8.matmul_f8(ta, tb, output_dtype='float32')
    assert np.array_equal(host(got32).astype(np.int64), exact)
    got8 = F8.matmul_f8(ta, tb)  # default output dtype: the fp8 input type, as in the reference
    assert got8.dtype == torch.float8_e4m3fn
    assert np.array_equal(codes_of(got8), O.e4m3_encode(exact.astype(np.float32)))
    gotb = F8.matmul_f8(ta, tb, output_dtype='bfloat16')
    assert np.array_equal(host(gotb), O.to_bf16(exact.astype(np.float32)))
    goth = F8.matmul_f8(ta, tb, output_dtype='f16')
    with np.errstate(over='ignore'):
        assert np.array_equal(host(goth), exact.astype(np.float32).astype(np.float16))


@pytest.mark.parametrize('a_shape, b_shape', [[[4096, 4096], [4096, 4096]], [[2048, 256], [4096, 256]], [[100, 384], [256, 384]],
                                              [[16384, 7168], [1536, 7168]],
                                              [[40, 4096], [1024, 4096]], [[130, 2048], [512, 2048]], [[500, 7168], [1536, 7168]],  # K ranges
                                              # up to 16 rows: the bandwidth-bound kernel, 8 and 4 waves per workgroup
                                              [[1, 7168], [1536, 7168]], [[16, 4096], [4096, 4096]], [[5, 384], [256, 384]],
                                              [[9, 2048], [8192, 2048]], [[3, 128], [128, 128]]])
def test_matmul_f8_scaled_reference_recipe(a_shape, b_shape):
    # tests/operators_core/test_matmul.py:291-373: integers in [-5, 4], integer scales 1..4, bf16 output; the
    # expected value is built by pre-multiplying the scales into the operands (exact in int64)
    announce('matmul_f8_scaled', a_shape, b_shape)
    rng = np.random.default_rng(42)
    (m, k), n = a_shape, b_shape[0]
    ai = rng.integers(-5, 5, a_shape)
    bi = rng.integers(-5, 5, b_shape)
    sa = rng.integers(1, 5, (k // 128, m)).astype(np.float32)
    sb = rng.integers(1, 5, (n // 128, k // 128)).astype(np.float32)
    got = F8.matmul_f8_scaled(f8(O.e4m3_encode(ai.astype(np.float32))), f8(O.e4m3_encode(bi.astype(np.float32))),
                              scale_a=dev(sa), scale_b=dev(sb), output_dtype='float32')
    a2 = ai.astype(np.int64) * np.repeat(sa.T.astype(np.int64), 128, axis=1)
    b2 = bi.astype(np.int64) * np.repeat(np.repeat(sb.astype(np.int64), 128, axis=0), 128, axis=1)
    exact = (a2.astype(np.float64) @ b2.astype(np.float64).T).astype(np.int64)  # float64 BLAS: exact on these integers
    assert np.array_equal(host(got).astype(np.int64), exact)
    gotb = F8.matmul_f8_scaled(f8(O.e4m3_encode(ai.astype(np.float32))), f8(O.e4m3_encode(bi.astype(np.float32))),
                               scale_a=dev(sa), scale_b=dev(sb), output_dtype='bfloat16')
    assert np.array_equal(host(gotb), O.to_bf16(exact.astype(np.float32)))
    if m <= 128:
        ref = O.matmul_f8_scaled(O.e4m3_encode(ai.astype(np.float32)), O.e4m3_encode(bi.astype(np.float32)), sa, sb, 'float32')
        assert np.array_equal(host(got), ref)


@pytest.mark.parametrize('m,k,n', [(1, 4096, 4096), (7, 7168, 1536), (16, 2048, 8192), (40, 1024, 512)])
def test_matmul_f8_scaled_parity_real_scales(m, k, n):
    # random e4m3 codes and real-valued block scales against the oracle, tolerance 3e-2 (fp32 sums in another order)
    announce('matmul_f8_scaled real scales', m, k, n)
    rng = np.random.default_rng(m + k)
    ac = O.e4m3_encode(rng.standard_normal((m, k)).astype(np.float32))
    bc = O.e4m3_encode((rng.standard_normal((n, k)) * 0.5).astype(np.float32))
    sa = rng.uniform(0.5, 2.0, (k // 128, m)).astype(np.float32)
    sb = rng.uniform(0.01, 0.05, (n // 128, k // 128)).astype(np.float32)
    got = F8.matmul_f8_scaled(f8(ac), f8(bc), scale_a=dev(sa), scale_b=dev(sb), output_dtype='float32')
    ref = O.matmul_f8_scaled(ac, bc, sa, sb, 'float32')
    err = O.max_rel_err(host(got), ref)
    assert err <= 3e-2, err
    assert err <= 1e-4, err  # fp32 accumulation on both sides: only the order of the sums differs


@pytest.mark.parametrize('a_shape, b_shape', [[[2048, 256], [4096, 256]], [[100, 384], [256, 384]], [[40, 4096], [1024, 4096]],
                                              [[500, 7168], [1536, 7168]], [[1, 7168], [1536, 7168]], [[16, 4096], [4096, 4096]],
                                              [[5, 384], [256, 384]], [[3, 128], [128, 128]]])
def test_matmul_f8_scaled_e5m2_reference_recipe(a_shape, b_shape):
    # the scaled task takes both operands float8_e5m2 as well (matmul_f8.py:386-389, 709-712): the recipe of
    # tests/operators_core/test_matmul.py:291-373 on e5m2 codes - integers in [-4, 4] and integer scales are exact in e5m2 -
    # through every kernel of the scaled path (8-wave tiles with and without K ranges, the bandwidth-bound kernel)
    announce('matmul_f8_scaled e5m2', a_shape, b_shape)
    rng = np.random.default_rng(43)
    (m, k), n = a_shape, b_shape[0]
    ai = rng.integers(-4, 5, a_shape)
    bi = rng.integers(-4, 5, b_shape)
    sa = rng.integers(1, 5, (k // 128, m)).astype(np.float32)
    sb = rng.integers(1, 5, (n // 128, k // 128)).astype(np.float32)
    ac, bc = O.e5m2_encode(ai.astype(np.float32)), O.e5m2_encode(bi.astype(np.float32))
    assert np.array_equal(O.e5m2_decode(ac), ai) and np.array_equal(O.e5m2_decode(bc), bi)
    ta, tb = dev(ac).view(torch.float8_e5m2), dev(bc).view(torch.float8_e5m2)
    got = F8.matmul_f8_scaled(ta, tb, scale_a=dev(sa), scale_b=dev(sb), output_dtype='float32')
    a2 = ai.astype(np.int64) * np.repeat(sa.T.astype(np.int64), 128, axis=1)
    b2 = bi.astype(np.int64) * np.repeat(np.repeat(sb.astype(np.int64), 128, axis=0), 128, axis=1)
    exact = (a2.astype(np.float64) @ b2.astype(np.float64).T).astype(np.int64)
    assert np.array_equal(host(got).astype(np.int64), exact)
    gotb = F8.matmul_f8_scaled(ta, tb, scale_a=dev(sa), scale_b=dev(sb), output_dtype='bfloat16')
    assert np.array_equal(host(gotb), O.to_bf16(exact.astype(np.float32)))
    got8 = F8.matmul_f8_scaled(ta, tb, scale_a=dev(sa), scale_b=dev(sb))  # default: the operands' own type
    assert got8.dtype == torch.float8_e5m2
    assert np.array_equal(got8.view(torch.uint8).cpu().numpy(), O.e5m2_encode(exact.astype(np.float32)))
    with pytest.raises(ValueError, match='unsupported output dtype'):
        F8.matmul_f8_scaled(ta, tb, scale_a=dev(sa), scale_b=dev(sb), output_dtype=torch.float8_e4m3fn)
    if m <= 128:
        ref = O.matmul_f8_scaled(ac, bc, sa, sb, 'float32', in_dtype='float8_e5m2')
        assert np.array_equal(host(got), ref)


@pytest.mark.parametrize('m,k,n', [(1, 4096, 4096), (16, 2048, 8192), (40, 1024, 512), (300, 512, 768)])
def test_matmul_f8_scaled_e5m2_parity_real_scales(m, k, n):
    # random e5m2 codes (subnormals and large magnitudes included) and real-valued block scales against the oracle
    announce('matmul_f8_scaled e5m2 real scales', m, k, n)
    rng = np.random.default_rng(m + k + 1)
    ac = O.e5m2_encode((rng.standard_normal((m, k)) * np.exp2(rng.integers(-16, 3, (m, k)))).astype(np.float32))
    bc = O.e5m2_encode((rng.standard_normal((n, k)) * 0.5).astype(np.float32))
    sa = rng.uniform(0.5, 2.0, (k // 128, m)).astype(np.float32)
    sb = rng.uniform(0.01, 0.05, (n // 128, k // 128)).astype(np.float32)
    got = F8.matmul_f8_scaled(dev(ac).view(torch.float8_e5m2), dev(bc).view(torch.float8_e5m2), scale_a=dev(sa), scale_b=dev(sb),
                              output_dtype='float32')
    ref = O.matmul_f8_scaled(ac, bc, sa, sb, 'float32', in_dtype='float8_e5m2')
    err = O.max_rel_err(host(got), ref)
    assert err <= 1e-4, err  # fp32 accumulation on both sides: only the order of the sums differs


@pytest.mark.parametrize('m,k,n', [(1, 8192, 8192), (16, 1024, 512), (256, 512, 768), (4096, 8192, 8192), (33, 400, 260)])
def test_per_tensor_parity(m, k, n):
    announce('fp8 per-tensor', m, k, n)
    a32, b32 = O.make_inputs(0, m, k, n)
    b32 = np.ascontiguousarray(b32.T)  # [N, K]
    ta, sa = F8.fp8_quantize_per_tensor(dev(a32))
    tb, sb = F8.fp8_quantize_per_tensor(dev(b32))
    ac, sa0 = O.fp8_quantize_per_tensor(a32)
    bc, sb0 = O.fp8_quantize_per_tensor(b32)
    assert np.array_equal(codes_of(ta), ac) and np.array_equal(codes_of(tb), bc)
    assert np.float32(sa.item()) == sa0 and np.float32(sb.item()) == sb0
    got = F8.matmul_f8_per_tensor(ta, tb, sa, sb, 'bfloat16')
    rows = np.arange(m) if m <= 256 else np.array([0, 15, 16, 255, 256, 1000, 2047, 2048, 4095])
    ref = O.fp8_matmul_per_tensor(ac[rows], bc, sa0, sb0, 'bfloat16')
    err = O.max_rel_err(host(got)[rows], ref)
    print('max_rel_err vs oracle', err)
    assert err <= TOL and err <= 8e-3  # same codes on both sides: only bf16 output rounding and sum order differ
    # against the unquantized product the fp8 quantization error itself stays inside the gate
    want = a32[rows].astype(np.float64) @ b32.astype(np.float64).T
    print('max_rel_err vs unquantized', O.max_rel_err(host(got)[rows], want))


def test_k_split_is_deterministic_and_optional():
    announce('fp8 k split twice / without workspace')
    from hidet_amd import ffi
    rng = np.random.default_rng(5)
    m, k, n = 100, 8192, 1024
    ta = f8(rng.integers(0, 0x7F, (m, k)).astype(np.uint8))
    tb = f8(rng.integers(0, 0x7F, (n, k)).astype(np.uint8))
    first = host(F8.matmul_f8(ta, tb, output_dtype='float32'))
    for _ in range(3):
        assert np.array_equal(host(F8.matmul_f8(ta, tb, output_dtype='float32')), first)
    # no workspace: every tile by one workgroup; same sums in a different order
    c = torch.empty(m, n, device='cuda', dtype=torch.float32)
    ffi.call('hidet_matmul_f8', ta, tb, c, m, n, k, k, k, ffi.DTYPE_CODE[torch.float32], None, None, None, 0,
             ffi.current_stream(c.device))
    ref = host(c)
    assert O.max_rel_err(first, ref) <= 1e-5


@pytest.mark.parametrize('m,k,n', [(1, 128, 16), (3, 384, 40), (7, 1152, 72), (16, 8192, 8192), (2, 4096, 4096), (16, 2048, 8200),
                                   (5, 1040, 48), (9, 11008, 520), (13, 1024, 24)])
def test_skinny_exact_on_small_integers(m, k, n):
    # 1..16 rows: integer operands make every product and partial sum exact, so the result must be the integer
    # product whichever kernel runs (K a multiple of 128 or not, 4 or 8 waves, waves with an empty K range,
    # columns that do not fill the last workgroup), also for a row stride larger than K
    announce('fp8 skinny exact', m, k, n)
    rng = np.random.default_rng(m * 1000 + n)
    ai, bi = rng.integers(-4, 5, (m, k)), rng.integers(-4, 5, (n, k))
    want = ai.astype(np.int64) @ bi.astype(np.int64).T
    ta, tb = f8(O.e4m3_encode(ai.astype(np.float32))), f8(O.e4m3_encode(bi.astype(np.float32)))
    assert np.array_equal(host(F8.matmul_f8(ta, tb, output_dtype='float32')).astype(np.int64), want)
    wide = torch.full((m, k + 256), 0x38, dtype=torch.uint8, device='cuda')  # 1.0 outside the operand
    wide[:, 128:128 + k] = ta.view(torch.uint8)
    got = F8.matmul_f8(wide[:, 128:128 + k].view(torch.float8_e4m3fn), tb, output_dtype='float32')
    assert np.array_equal(host(got).astype(np.int64), want)


def test_batched_and_strided_operands():
    announce('fp8 batched')
    rng = np.random.default_rng(5)
    ai = rng.integers(-3, 3, (3, 20, 64))
    bi = rng.integers(-3, 3, (40, 64))
    ta, tb = f8(O.e4m3_encode(ai.astype(np.float32))), f8(O.e4m3_encode(bi.astype(np.float32)))
    got = F8.matmul_f8(ta, tb, output_dtype='float32')
    assert tuple(got.shape) == (3, 20, 40)
    assert np.array_equal(host(got).astype(np.int64), ai.astype(np.int64) @ bi.astype(np.int64).T)
    b3 = rng.integers(-3, 3, (3, 40, 64))
    got = F8.matmul_f8(ta, f8(O.e4m3_encode(b3.astype(np.float32))), output_dtype='float32')
    assert np.array_equal(host(got).astype(np.int64), np.einsum('bmk,bnk->bmn', ai.astype(np.int64), b3.astype(np.int64)))
    wide = torch.zeros(20, 256, dtype=torch.uint8, device='cuda')
    wide[:, 64:128] = ta[0].view(torch.uint8)
    got = F8.matmul_f8(wide[:, 64:128].view(torch.float8_e4m3fn), tb, output_dtype='float32')  # row stride 256
    assert np.array_equal(host(got).astype(np.int64), ai[0].astype(np.int64) @ bi.astype(np.int64).T)


@pytest.mark.parametrize('m,k,n', [(6, 128, 16), (1, 1024, 512), (40, 512, 384), (300, 256, 520)])
def test_per_tensor_exact_case(m, k, n):
    # integer-valued codes and power-of-two scales: products, sums and the rescaling are exact in fp32
    announce('fp8 per-tensor exact', m, k, n)
    rng = np.random.default_rng(m + n)
    ai, bi = rng.integers(-8, 9, (m, k)), rng.integers(-8, 9, (n, k))
    ta, tb = f8(O.e4m3_encode(ai.astype(np.float32))), f8(O.e4m3_encode(bi.astype(np.float32)))
    for sa, sb in ((0.5, 4.0), (2.0 ** -6, 2.0 ** 3)):
        want = (ai.astype(np.int64) @ bi.astype(np.int64).T).astype(np.float64) * sa * sb
        dsa, dsb = dev(np.array([sa], dtype=np.float32)), dev(np.array([sb], dtype=np.float32))
        got = F8.matmul_f8_per_tensor(ta, tb, dsa, dsb, 'float32')
        assert np.array_equal(host(got).astype(np.float64), want)
        gotb = F8.matmul_f8_per_tensor(ta, tb, dsa, dsb, 'bfloat16')
        assert np.array_equal(host(gotb), O.to_bf16(want.astype(np.float32)))
        assert np.array_equal(host(got), O.fp8_matmul_per_tensor(host(ta.view(torch.uint8)), host(tb.view(torch.uint8)),
                                                                 np.float32(sa), np.float32(sb), 'float32'))


@pytest.mark.parametrize('a_shape, b_shape', [[[256, 128], [256, 128]], [[512, 256], [128, 256]], [[1, 256], [48, 256]],
                                              [[16, 1024], [200, 1024]], [[100, 48], [36, 48]], [[300, 272], [260, 272]],
                                              [[7, 100], [33, 100]], [[1000, 512], [520, 512]]])
def test_matmul_f8_e5m2_reference_recipe(a_shape, b_shape):
    # the reference accepts both operands float8_e5m2 as well (matmul_f8.py:709-712); same integer recipe
    # (tests/operators_core/test_matmul.py:250-288). Up to 16 rows: the bandwidth-bound kernel; aligned shapes: the tile
    # kernel on the MFMA's bf8 format; the rest: the element-wise kernel.
    announce('matmul_f8 e5m2', a_shape, b_shape)
    rng = np.random.default_rng(44)
    ai, bi = rng.integers(-3, 3, a_shape), rng.integers(-3, 3, b_shape)
    ta = dev(O.e5m2_encode(ai.astype(np.float32))).view(torch.float8_e5m2)
    tb = dev(O.e5m2_encode(bi.astype(np.float32))).view(torch.float8_e5m2)
    exact = (ai.astype(np.float64) @ bi.astype(np.float64).T).astype(np.int64)
    got32 = F8.matmul_f8(ta, tb, output_dtype='float32')
    assert np.array_equal(host(got32).astype(np.int64), exact)
    got8 = F8.matmul_f8(ta, tb)
    assert got8.dtype == torch.float8_e5m2
    assert np.array_equal(got8.view(torch.uint8).cpu().numpy(), O.e5m2_encode(exact.astype(np.float32)))
    gotb = F8.matmul_f8(ta, tb, output_dtype='bfloat16')
    assert np.array_equal(host(gotb), O.to_bf16(exact.astype(np.float32)))
    assert np.array_equal(host(got32), O.matmul_f8(host(ta.view(torch.uint8)), host(tb.view(torch.uint8)), 'float32',
                                                   in_dtype='float8_e5m2'))


def test_e5m2_output_conversion_every_boundary():
    # float32 -> e5m2 in the epilogue: a 1 x 1 x K product that lands on every midpoint between neighbouring codes
    # and just beside it, plus saturation; a = [x, 0, ...] in e5m2 cannot carry these values, so the values are built
    # as sums of two exactly representable operands: x = hi + lo with b = [1, 1, 0, ...]
    announce('e5m2 output rounding')
    tab = O.e5m2_decode(np.arange(0x7C, dtype=np.uint8)).astype(np.float64)
    cases = []
    for i in range(0x10, 0x7B):  # normal range: midpoint = tab[i] + half a step, half a step is itself a code value
        half = (tab[i + 1] - tab[i]) / 2
        if O.e5m2_decode(O.e5m2_encode(np.array([half], dtype=np.float32)))[0] == half:
            cases.append((tab[i], half))
    hi = np.array([c[0] for c in cases], dtype=np.float32)
    lo = np.array([c[1] for c in cases], dtype=np.float32)
    a = np.zeros((len(cases), 16), dtype=np.float32)
    a[:, 0], a[:, 1] = hi, lo
    b = np.zeros((4, 16), dtype=np.float32)
    b[0, :2] = 1.0
    b[1, 0] = 1.0
    ta = dev(O.e5m2_encode(a)).view(torch.float8_e5m2)
    tb = dev(O.e5m2_encode(b)).view(torch.float8_e5m2)
    got = F8.matmul_f8(ta, tb).view(torch.uint8).cpu().numpy()
    want = O.e5m2_encode((hi.astype(np.float64) + lo.astype(np.float64)).astype(np.float32))
    assert np.array_equal(got[:, 0], want) and np.array_equal(got[:, 1], O.e5m2_encode(hi))
    big = dev(O.e5m2_encode(np.full((2, 16), 57344.0, dtype=np.float32))).view(torch.float8_e5m2)
    ones = dev(O.e5m2_encode(np.ones((4, 16), dtype=np.float32))).view(torch.float8_e5m2)
    assert set(F8.matmul_f8(big, ones).view(torch.uint8).cpu().numpy().ravel().tolist()) == {0x7B}  # saturates, no infinity


def test_expanded_and_transposed_operands():
    # operands whose rows cannot be addressed with a stride >= K (one row expanded to M rows, a transposed view) are
    # copied by the operator before they reach the kernel
    announce('fp8 expanded operands')
    rng = np.random.default_rng(8)
    row = rng.integers(-3, 3, (1, 256))
    bi = rng.integers(-3, 3, (48, 256))
    ta, tb = f8(O.e4m3_encode(row.astype(np.float32))), f8(O.e4m3_encode(bi.astype(np.float32)))
    got = F8.matmul_f8(ta.expand(20, 256), tb, output_dtype='float32')
    want = np.repeat(row.astype(np.int64), 20, axis=0) @ bi.astype(np.int64).T
    assert np.array_equal(host(got).astype(np.int64), want)
    at = rng.integers(-3, 3, (256, 24))
    tt = f8(O.e4m3_encode(at.astype(np.float32)))
    got = F8.matmul_f8(tt.t(), tb, output_dtype='float32')
    assert np.array_equal(host(got).astype(np.int64), at.T.astype(np.int64) @ bi.astype(np.int64).T)
    got = F8.matmul_f8(ta, tb.view(torch.uint8)[:1].expand(48, 256).view(torch.float8_e4m3fn), output_dtype='float32')
    assert np.array_equal(host(got).astype(np.int64), row.astype(np.int64) @ np.repeat(bi[:1].astype(np.int64), 48, axis=0).T)


def test_scaled_batched_activations_against_2d_weight():
    # the task accepts mutually broadcastable heads (reference matmul_f8.py:372-376): [B, M, K] x [N, K]
    announce('fp8 scaled batched')
    rng = np.random.default_rng(9)
    B, m, k, n = 3, 5, 256, 128
    ai = rng.integers(-5, 5, (B, m, k))
    bi = rng.integers(-5, 5, (n, k))
    sa = rng.integers(1, 5, (B, k // 128, m)).astype(np.float32)
    sb = rng.integers(1, 5, (n // 128, k // 128)).astype(np.float32)
    got = F8.matmul_f8_scaled(f8(O.e4m3_encode(ai.astype(np.float32))), f8(O.e4m3_encode(bi.astype(np.float32))),
                              scale_a=dev(sa), scale_b=dev(sb), output_dtype='float32')
    assert tuple(got.shape) == (B, m, n)
    b2 = bi.astype(np.int64) * np.repeat(np.repeat(sb.astype(np.int64), 128, axis=0), 128, axis=1)
    for i in range(B):
        a2 = ai[i].astype(np.int64) * np.repeat(sa[i].T.astype(np.int64), 128, axis=1)
        assert np.array_equal(host(got[i]).astype(np.int64), a2 @ b2.T)


def test_argument_errors():
    announce('fp8 errors')
    a = torch.zeros(4, 64, device='cuda').to(torch.float8_e4m3fn)
    with pytest.raises(ValueError, match='only supports both operands'):
        F8.matmul_f8(a, torch.zeros(4, 64, device='cuda'))
    with pytest.raises(ValueError, match='at least 2 dimensions'):
        F8.matmul_f8(a[0], a)
    with pytest.raises(ValueError, match=r'\[\.\.\.,M,K\] and \[\.\.\.,N,K\]'):
        F8.matmul_f8(a, torch.zeros(4, 32, device='cuda').to(torch.float8_e4m3fn))
    with pytest.raises(ValueError, match='only supports both operands'):  # mixed formats, scaled form
        F8.matmul_f8_scaled(a, a.to(torch.float8_e5m2), torch.ones(1, 4, device='cuda'), torch.ones(1, 1, device='cuda'))
    with pytest.raises(ValueError, match='unsupported output dtype'):
        F8.matmul_f8(a, a, output_dtype='float8_e5m2')
    with pytest.raises(ValueError, match='bias is not supported'):
        F8.matmul_f8_scaled(a, a, torch.ones(1, 4, device='cuda'), torch.ones(1, 1, device='cuda'), bias=torch.ones(4, device='cuda'))
