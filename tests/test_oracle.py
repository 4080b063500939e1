"""Pins the CPU oracle: against the reference's own half type (oracle/_ref, where built), against
the literal known answers and test recipes the reference's tests hold, and against what the
mathematics fixes (closed forms, invariants, brute force, exact small-integer cases).

Reference tests reproduced here: tests/operators_core/test_symmetric_quant.py:19-26,
tests/operators_core/test_quantization.py:21-47, tests/operators_core/test_matmul.py:250-373,
tests/ir/dtypes/test_fp8e4m3.py:13-35.
"""
import numpy as np
import pytest
import torch

from oracle import clib
from oracle import oracle as O


# ----------------------------------------------------------------------------- rounding / fp16

def test_round_half_away_ties_and_c_roundf():
    ties = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5, 0.49999997, -0.49999997, 0.0, -0.0, 127.0],
                    dtype=np.float32)
    want = np.array([1, 2, 3, -1, -2, -3, 127, -127, 0, 0, 0, 0, 127], dtype=np.float32)
    assert np.array_equal(O.round_half_away(ties), want)
    # numpy's own round is ties-to-even and must disagree on 0.5 and 2.5: the explicit form matters
    assert np.round(np.float32(2.5)) == 2.0
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.uniform(-130, 130, 20000).astype(np.float32),
                        (rng.integers(-127, 127, 2000) + 0.5).astype(np.float32)])
    L = clib.lib()
    c = np.array([L.oracle_roundf(float(v)) for v in x], dtype=np.float32)
    assert np.array_equal(O.round_half_away(x), c)


def test_half_conversions_exhaustive():
    L = clib.lib()
    R = clib.ref_lib()
    codes = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    as_f32 = codes.view(np.float16).astype(np.float32)
    mine = np.array([L.oracle_f16_to_f32(int(c)) for c in codes], dtype=np.float32)
    assert np.array_equal(mine.view(np.uint32)[~np.isnan(as_f32)], as_f32.view(np.uint32)[~np.isnan(as_f32)])
    back = np.array([L.oracle_f32_to_f16(float(v)) for v in as_f32], dtype=np.uint16)
    ok = ~np.isnan(as_f32)
    assert np.array_equal(back[ok], codes[ok])
    if R is not None:
        theirs = np.array([R.ref_f16_to_f32(int(c)) for c in codes], dtype=np.float32)
        assert np.array_equal(theirs.view(np.uint32)[ok], mine.view(np.uint32)[ok])


def test_f32_to_half_rounding_matches_numpy_and_reference_type():
    L = clib.lib()
    R = clib.ref_lib()
    rng = np.random.default_rng(2)
    # random values over the whole half range, every halfway point between adjacent halves, and the edges
    h = np.arange(0, 0x7C00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    mid = ((lo[:-1] + lo[1:]) / 2).astype(np.float32)  # exactly representable in f32
    x = np.concatenate([
        (rng.standard_normal(20000) * 10.0 ** rng.uniform(-9, 5, 20000)).astype(np.float32), mid, -mid,
        np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
        np.array([65504, 65519.996, 65520, 70000, 2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1)),
                  2.0 ** -24, 0.0, -0.0, np.inf, -np.inf], dtype=np.float32)])
    with np.errstate(over='ignore'):
        want = x.astype(np.float16).view(np.uint16)
    mine = np.array([L.oracle_f32_to_f16(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(mine, want)
    if R is not None:
        theirs = np.array([R.ref_f32_to_f16(float(v)) for v in x], dtype=np.uint16)
        assert np.array_equal(theirs, want)


@pytest.mark.skipif(clib.ref_lib() is None, reason='oracle/_ref not built (reference checkout absent)')
def test_half_operators_of_reference_type_are_f32_op_then_rne():
    R = clib.ref_lib()
    rng = np.random.default_rng(3)
    a = rng.integers(0, 0x7C00, 4000).astype(np.uint16) | (rng.integers(0, 2, 4000).astype(np.uint16) << 15)
    b = rng.integers(1, 0x7C00, 4000).astype(np.uint16) | (rng.integers(0, 2, 4000).astype(np.uint16) << 15)
    fa, fb = a.view(np.float16).astype(np.float32), b.view(np.float16).astype(np.float32)
    with np.errstate(over='ignore', divide='ignore', invalid='ignore'):
        for name, op in (('ref_half_mul', fa * fb), ('ref_half_add', fa + fb), ('ref_half_div', fa / fb)):
            got = np.array([getattr(R, name)(int(x), int(y)) for x, y in zip(a, b)], dtype=np.uint16)
            assert np.array_equal(got, op.astype(np.float32).astype(np.float16).view(np.uint16)), name
    # round(half) is std::round: ties away from zero (100.5 -> 101, 2.5 -> 3, -2.5 -> -3)
    for v, w in ((100.5, 101.0), (2.5, 3.0), (-2.5, -3.0), (0.5, 1.0), (1.4990234375, 1.0)):
        bits = int(np.float16(v).view(np.uint16))
        assert np.uint16(R.ref_half_round(bits)).view(np.float16) == np.float16(w)


# ----------------------------------------------------------------------------- symmetric quantize

@pytest.mark.parametrize('w', [32, 64])
@pytest.mark.parametrize('dtype', ['int8', 'int16'])
@pytest.mark.parametrize('dims', [[-1], [0]])
def test_symmetric_quant_round_trip_reference_recipe(w, dtype, dims):
    # tests/operators_core/test_symmetric_quant.py:19-26
    x = np.random.default_rng(w).standard_normal((w, w)).astype(np.float32)
    q, s = O.symmetric_quantize(x, dtype, dims)
    x1 = O.symmetric_dequantize(q, s, dims)
    assert q.dtype == np.dtype(dtype) and s.shape == (w,)
    assert np.allclose(x, x1, atol=1e-1, rtol=1e-1)


@pytest.mark.parametrize('quant_type', ['int8', 'int16'])
@pytest.mark.parametrize('axis', [0, 1])
def test_symmetric_quantize_invariants_and_c_restatement(quant_type, axis):
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((96, 80)) * 0.02).astype(np.float32)
    w[:, 7] = 0 if axis == 0 else w[:, 7]
    w[9, :] = 0 if axis == 1 else w[9, :]
    qmax = O.INT_MAX[quant_type]
    q, s = O.symmetric_quantize(w, quant_type, dims=axis)
    amax = np.abs(w).max(axis=axis)
    assert np.array_equal(s.view(np.uint32), (amax / np.float32(qmax)).astype(np.float32).view(np.uint32))
    nz = amax > 0
    assert np.all(np.abs(q.astype(np.int32)).max(axis=axis)[nz] == qmax)
    assert np.all(np.abs(q.astype(np.int32)) <= qmax)
    assert np.all(q.take(np.flatnonzero(~nz), axis=1 - axis) == 0) and np.all(s[~nz] == 0)
    qn, sn = O.symmetric_quantize(-w, quant_type, dims=axis)  # odd symmetry
    assert np.array_equal(qn, -q) and np.array_equal(sn, s)
    qc, sc = clib.symmetric_quantize_f32(w, axis, quant_type)
    assert np.array_equal(qc, q) and np.array_equal(sc.view(np.uint32), s.view(np.uint32))
    # dims given as a list, negative, or covering both axes
    q2, s2 = O.symmetric_quantize(w, quant_type, dims=[axis - 2])
    assert np.array_equal(q2, q) and np.array_equal(s2, s)
    q3, s3 = O.symmetric_quantize(w, quant_type, dims=[0, 1])
    assert s3.shape == () and s3 == np.float32(np.abs(w).max() / np.float32(qmax))


def test_symmetric_quantize_constructed_ties_round_away():
    # a column whose amax is 127 has scale exactly 1, so the quotient is the value itself
    col = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -126.5, 0.49999997], dtype=np.float32)
    q, s = O.symmetric_quantize(col[:, None], 'int8', dims=0)
    assert s[0] == 1.0
    assert q[:, 0].tolist() == [127, 1, 2, 3, -1, -2, -3, 64, -127, 0]
    qc, _ = clib.symmetric_quantize_f32(col[:, None], 0)
    assert qc[:, 0].tolist() == q[:, 0].tolist()


@pytest.mark.parametrize('dtype', ['float16', 'bfloat16'])
def test_symmetric_quantize_tie_rule_per_target(dtype):
    # the reference lowers round() per target: ties away on the CPU for every dtype, ties to even (hrint) on the GPU for
    # float16 / bfloat16, ties away (roundf) on the GPU for float32. Scale is exactly 1 here.
    col = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, 64.5, -100.5, -101.5, 3.25, 3.75], dtype=np.float32)
    away = [127, 1, 2, 3, -1, -2, -3, 64, 65, -101, -102, 3, 4]
    even = [127, 0, 2, 2, 0, -2, -2, 64, 64, -100, -102, 3, 4]
    q_cpu, s = O.symmetric_quantize(col[:, None], 'int8', 0, dtype=dtype, target='cpu')
    q_gpu, _ = O.symmetric_quantize(col[:, None], 'int8', 0, dtype=dtype, target='gpu')
    assert float(s[0]) == 1.0 and q_cpu[:, 0].tolist() == away and q_gpu[:, 0].tolist() == even
    q32_cpu, _ = O.symmetric_quantize(col[:, None], 'int8', 0, target='cpu')
    q32_gpu, _ = O.symmetric_quantize(col[:, None], 'int8', 0, target='gpu')
    assert q32_cpu[:, 0].tolist() == away and q32_gpu[:, 0].tolist() == away
    # away from exact ties the two targets agree
    rng = np.random.default_rng(3)
    x = rng.standard_normal((64, 8)).astype(np.float32)
    qa, _ = O.symmetric_quantize(x, 'int8', 0, dtype=dtype, target='cpu')
    qb, _ = O.symmetric_quantize(x, 'int8', 0, dtype=dtype, target='gpu')
    assert np.abs(qa.astype(np.int32) - qb.astype(np.int32)).max() <= 1
    with pytest.raises(ValueError):
        O.symmetric_quantize(x, 'int8', 0, target='tpu')


@pytest.mark.skipif(clib.ref_lib() is None, reason='oracle/_ref not built (reference checkout absent)')
def test_symmetric_quantize_f16_brute_force_against_reference_half_type():
    # every finite positive float16 pattern in one column (the largest value fixes the scale),
    # evaluated with the reference's own half operators
    R = clib.ref_lib()
    pat = np.arange(0, 0x7C00, 37, dtype=np.uint16)
    rng = np.random.default_rng(7)
    for top in (0x7BFF, 0x5BF0, 0x3C00, 0x2E66, 0x0400, 0x0011):
        col = pat[pat <= top].copy()
        col = np.concatenate([col, np.array([top], dtype=np.uint16)])
        sign = (rng.integers(0, 2, col.size).astype(np.uint16) << 15)
        bits = (col | sign).astype(np.uint16)
        w16 = bits.view(np.float16).reshape(-1, 1)
        q, s = O.symmetric_quantize(w16, 'int8', dims=0)
        codes = np.empty((col.size, 1), dtype=np.int8)
        scale = np.empty(1, dtype=np.uint16)
        R.ref_symmetric_quantize_f16_axis0(bits.ctypes.data, col.size, 1, codes.ctypes.data, scale.ctypes.data)
        assert s.view(np.uint16)[0] == scale[0], hex(top)
        assert np.array_equal(codes, q), hex(top)


def test_symmetric_quantize_bf16_carrier():
    rng = np.random.default_rng(8)
    w = O.to_bf16(rng.standard_normal((64, 48)).astype(np.float32))
    q, s = O.symmetric_quantize(w, 'int8', dims=0, dtype='bfloat16')
    tw = torch.from_numpy(w).to(torch.bfloat16)
    ts = (tw.abs().amax(0) / torch.tensor(127.0, dtype=torch.bfloat16))  # bf16 division: f32 op then RNE
    assert np.array_equal(O.bf16_bits(s), ts.view(torch.int16).numpy().view(np.uint16))
    quot = (tw / ts).float().numpy()
    assert np.array_equal(q, np.clip(O.round_half_away(quot), -128, 127).astype(np.int8))
    back = O.symmetric_dequantize(q, s, dims=0, dtype='bfloat16')
    assert np.allclose(back, w, atol=1e-1, rtol=1e-1)


def test_to_bf16_matches_torch():
    rng = np.random.default_rng(9)
    x = (rng.standard_normal(50000) * 10.0 ** rng.uniform(-20, 20, 50000)).astype(np.float32)
    x = np.concatenate([x, np.array([1.00390625, 1.01171875, 3.3895314e38, 0.0, -0.0], dtype=np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(O.to_bf16(x).view(np.uint32), want.view(np.uint32))
    assert np.array_equal(O.bf16_from_bits(O.bf16_bits(want)), want)


def test_symmetric_dequantize_closed_form():
    q = np.arange(-127, 128, dtype=np.int8).reshape(-1, 1).repeat(3, axis=1)
    s = np.array([0.001, 0.25, 3.0], dtype=np.float16)
    w = O.symmetric_dequantize(q, s, dims=0)
    assert w.dtype == np.float16
    want = (q.astype(np.float32) * s.astype(np.float32)[None, :]).astype(np.float16)
    assert np.array_equal(w.view(np.uint16), want.view(np.uint16))
    # dims=-1: one scale per row
    w2 = O.symmetric_dequantize(q.T.copy(), s, dims=-1)
    assert np.array_equal(w2, w.T)


# ----------------------------------------------------------------------------- W8A16 matmul

def _small_int_case(m, k, n, seed):
    rng = np.random.default_rng(seed)
    a = rng.integers(-4, 5, (m, k)).astype(np.float16)
    q = rng.integers(-127, 128, (k, n)).astype(np.int8)
    s = (2.0 ** rng.integers(-6, -2, n)).astype(np.float16)  # power-of-two scales keep everything exact
    return a, q, s


def test_quant_matmul_exact_on_small_integers():
    # tests/cute_kernel/test_quant_linear.py:35-49 recipe: small integers make every product and
    # fp32 partial sum exact, so the answer is an integer computable in int64
    a, q, s = _small_int_case(5, 96, 24, 11)
    want = (a.astype(np.int64) @ q.astype(np.int64)).astype(np.float64) * s.astype(np.float64)[None, :]
    got = O.symmetric_quant_matmul(a, q, s)
    assert np.array_equal(got.astype(np.float64), want.astype(np.float16).astype(np.float64))
    assert np.array_equal(clib.quant_matmul_f32acc(a, q, s), got)
    # the dropped-term / transposed-operand mistakes fail this case
    assert not np.array_equal(O.symmetric_quant_matmul(a, q, s[::-1].copy()), got)


@pytest.mark.parametrize(['x_shape', 'w_shape'], [[[2, 32, 32], [32, 32]], [[1, 64, 64], [64, 128]]])
def test_quant_matmul_reference_recipe(x_shape, w_shape):
    # tests/operators_core/test_quantization.py:39-47: against the UNquantized matmul at 2e-1
    rng = np.random.default_rng(12)
    x = rng.standard_normal(x_shape).astype(np.float16)
    w = rng.standard_normal(w_shape).astype(np.float16)
    wq, scale = O.symmetric_quantize(w, 'int8', dims=0)
    yq = O.symmetric_quant_matmul(x, wq, scale)
    y = np.matmul(x.astype(np.float32), w.astype(np.float32))
    assert yq.shape == tuple(x_shape[:-1] + [w_shape[1]])
    assert np.allclose(y, yq.astype(np.float32), atol=2e-1, rtol=2e-1)


def test_quant_matmul_equals_library_matmul_on_dequantized_weights():
    a32, w32 = O.make_inputs(0, 16, 512, 256)
    a = a32.astype(np.float16)
    q, s32 = O.symmetric_quantize(w32, 'int8', dims=0)
    s = s32.astype(np.float16)
    wd = torch.from_numpy(O.symmetric_dequantize(q, s, dims=0)).double()
    want = (torch.from_numpy(a).double() @ wd).numpy()
    got = O.symmetric_quant_matmul(a, q, s)
    got64 = O.symmetric_quant_matmul(a, q, s, acc='f64')
    assert O.max_rel_err(got, want) < 1e-3 and O.max_rel_err(got64, want) < 6e-4
    gotc = clib.quant_matmul_f32acc(a, q, s)
    assert O.max_rel_err(gotc, want) < 1e-3
    # numpy-f32 and C-f32 accumulate in different orders: equal to within an ulp or two of f16
    assert O.max_rel_err(gotc, got) < 2e-3


def test_reference_cpu_route_three_ways():
    a32, w32 = O.make_inputs(3, 4, 192, 40)
    a = a32.astype(np.float16)
    q, s32 = O.symmetric_quantize(w32, 'int8', dims=0)
    s = s32.astype(np.float16)
    py = O.reference_cpu_quant_matmul(a, q, s)
    c = clib.quant_matmul_ref_cpu(a, q, s)
    fast = clib.baseline_quant_matmul(a, q, s)
    assert np.array_equal(py.view(np.uint16), c.view(np.uint16))
    assert np.array_equal(fast.view(np.uint16), c.view(np.uint16))
    R = clib.ref_lib()
    if R is not None:
        out = np.empty((4, 40), dtype=np.float16)
        R.ref_quant_matmul_cpu(a.ctypes.data, q.ctypes.data, s.ctypes.data, out.ctypes.data, 4, 192, 40)
        assert np.array_equal(out.view(np.uint16), c.view(np.uint16))
    # the fp16-accumulating route stays within the reference's own tolerance of the fp32 one
    assert np.allclose(c.astype(np.float32), O.symmetric_quant_matmul(a, q, s).astype(np.float32), atol=2e-1,
                       rtol=2e-1)


def test_split_k_parts_sum_to_full_and_pad_with_zero():
    # 100 is not a multiple of 8 parts: the last part is ragged.  |sum| <= 100*2*7 < 2048 keeps every
    # part and the total exactly representable in float16
    rng = np.random.default_rng(13)
    a = rng.integers(-2, 3, (3, 100)).astype(np.float16)
    q = rng.integers(-7, 8, (100, 16)).astype(np.int8)
    s = (2.0 ** rng.integers(-6, -2, 16)).astype(np.float16)
    full = O.symmetric_quant_matmul(a, q, s).astype(np.float64)
    for parts in (1, 2, 3, 7, 8, 16, 128):
        c = O.quant_matmul_split_k(a, q, s, parts)
        assert c.shape == (parts, 3, 16)
        assert np.array_equal(c.astype(np.float64).sum(0), full), parts
    c = O.quant_matmul_split_k(a, q, s, 128)  # ceil(100/128) = 1: parts 100.. are all zero
    assert not c[100:].any()


def test_resolve_k_parts_table():
    # graph/ops/quant/resolve.py:42-48 evaluated by hand
    assert O.resolve_k_parts('disabled', 1, 1, 11008, 4096) == 1
    assert O.resolve_k_parts('default', 1, 1, 11008, 4096) == 3      # 172 blocks -> ceil(400/172)
    assert O.resolve_k_parts('default', 1, 1, 4096, 11008) == 7      # 64 blocks -> ceil(400/64)
    assert O.resolve_k_parts('default', 1, 16, 4096, 4096) == 7
    assert O.resolve_k_parts('default', 1, 2048, 11008, 4096) == 1   # 5504 blocks
    assert O.resolve_k_parts('default', 1, 1, 64, 128) == 2          # capped by ceil(K/64)
    assert O.resolve_k_parts(0, 1, 1, 1, 1) == 1 and O.resolve_k_parts(99, 1, 1, 1, 1) == 32
    with pytest.raises(ValueError):
        O.resolve_k_parts('bogus', 1, 1, 1, 1)


# ----------------------------------------------------------------------------- int4 groups

def test_int4_pack_order_and_round_trip():
    q = np.array([[1, -2, 7, -7, 0, -8]], dtype=np.int8)
    p = O.pack_int4(q)
    # element o -> byte o//2, bits (o%2)*4: low nibble first (transforms/lower_integer_subbyte.py:103-113)
    assert p.tolist() == [[0x01 | (0xE << 4), 0x07 | (0x9 << 4), 0x00 | (0x8 << 4)]]
    assert np.array_equal(O.unpack_int4(p), q)
    allq = np.array([[a, b] for a in range(-8, 8) for b in range(-8, 8)], dtype=np.int8)
    assert np.array_equal(O.unpack_int4(O.pack_int4(allq)), allq)


def test_group_quantize_int4_invariants():
    _, w = O.make_inputs(0, 1, 512, 64)
    w[128:256, 5] = 0
    packed, scales, q = O.group_quantize_int4(w, 128, 'bfloat16')
    assert packed.shape == (512, 32) and scales.shape == (4, 64) and packed.dtype == np.uint8
    amax = np.abs(w.reshape(4, 128, 64)).max(axis=1)
    assert np.array_equal(scales, O.to_bf16((amax / np.float32(7)).astype(np.float32)))
    g = np.abs(q.astype(np.int32)).reshape(4, 128, 64).max(axis=1)
    assert np.all(g[amax > 0] == 7) and np.all(g[amax == 0] == 0) and np.abs(q).max() <= 7
    assert np.array_equal(O.unpack_int4(packed), q)
    # dequantized weights stay within half a step of their own group's scale of the original, plus the bf16 rounding of
    # that scale (relative 2^-8 at most) on codes of magnitude 7 at most
    step = np.repeat(scales, 128, axis=0)
    assert np.all(np.abs(step * q - w) <= step * (0.5 + 7 * 2.0 ** -8) * (1 + 2.0 ** -8))


def test_group_quantize_int4_constructed_ties_and_clamp():
    # a group whose amax is 7 has scale32 exactly 1: the codes are round_half_away of the values themselves
    col = np.zeros(128, dtype=np.float32)
    vals = np.array([7.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 6.5, -6.5, 3.49, -3.51], dtype=np.float32)
    col[:vals.size] = vals
    w = np.stack([col, -col, 2 * col], axis=1).astype(np.float32)
    w = np.concatenate([w, w[:, :1]], axis=1)  # an even number of columns
    packed, scales, q = O.group_quantize_int4(w, 128, 'float16')
    want = [7, 1, 2, 3, -1, -2, -3, 7, -7, 3, -4]
    assert q[:vals.size, 0].tolist() == want and q[:vals.size, 1].tolist() == [-v for v in want]
    assert q[:vals.size, 2].tolist() == want  # scale 2: the same quotients
    assert scales[0].astype(np.float32).tolist() == [1.0, 1.0, 2.0, 1.0]
    assert np.array_equal(O.unpack_int4(packed), q)


def test_w4a16_matmul_exact_on_small_integers():
    rng = np.random.default_rng(21)
    a = rng.integers(-3, 4, (4, 256)).astype(np.float32)
    q = rng.integers(-7, 8, (256, 16)).astype(np.int8)
    scales = (2.0 ** rng.integers(-3, 1, (2, 16))).astype(np.float32)
    got = O.w4a16_matmul(a, O.pack_int4(q), scales, 128, 'bfloat16')
    want = np.zeros((4, 16))
    for g in range(2):
        want += (a[:, g * 128:(g + 1) * 128].astype(np.int64) @ q[g * 128:(g + 1) * 128].astype(np.int64)) * scales[g]
    assert np.array_equal(got, O.to_bf16(want.astype(np.float32)))


# ----------------------------------------------------------------------------- fp8 e4m3

def test_e4m3_decode_exhaustive_against_torch():
    codes = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    got = O.e4m3_decode(codes)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])
    assert got[0x7E] == 448.0 and got[0x01] == 2.0 ** -9 and np.isnan(got[0x7F]) and np.isnan(got[0xFF])


def test_e4m3_encode_against_torch_in_range_and_saturation():
    tab = O.e4m3_decode(np.arange(0, 0x7F, dtype=np.uint8)).astype(np.float64)
    mids = ((tab[:-1] + tab[1:]) / 2).astype(np.float32)
    rng = np.random.default_rng(31)
    x = np.concatenate([tab.astype(np.float32), mids, np.nextafter(mids, np.float32(1e9)),
                        np.nextafter(mids, np.float32(-1e9)), rng.uniform(-448, 448, 50000).astype(np.float32),
                        (rng.standard_normal(50000) * 10.0 ** rng.uniform(-5, 1, 50000)).astype(np.float32)])
    x = np.concatenate([x, -x])
    x = x[np.abs(x) <= 448]
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = O.e4m3_encode(x)
    assert np.array_equal(got, want)
    # saturating beyond the range, sign kept, NaN preserved
    assert O.e4m3_encode(np.array([1e9, -1e9, 449.0, 464.0, 480.0], dtype=np.float32)).tolist() == \
        [0x7E, 0xFE, 0x7E, 0x7E, 0x7E]
    assert O.e4m3_encode(np.array([np.nan], dtype=np.float32))[0] & 0x7F == 0x7F
    # round trip of every finite code
    codes = np.array([c for c in range(256) if c & 0x7F != 0x7F], dtype=np.uint8)
    assert np.array_equal(O.e4m3_encode(O.e4m3_decode(codes)), codes)


def test_e4m3_reference_known_answers():
    # tests/ir/dtypes/test_fp8e4m3.py:19-20: inputs 9, 96, 112, 10, 4 -> 104, -8, 8, 80, 20 where every
    # operator result is rounded to e4m3
    rt = lambda v: float(O.e4m3_decode(O.e4m3_encode(np.array([v], dtype=np.float32)))[0])
    i = [rt(v) for v in (9, 96, 112, 10, 4)]
    o = rt(i[0] + i[1])
    o2 = rt(o - i[2])
    o3 = rt(-o2)
    o4 = rt(o3 * i[3])
    o5 = rt(o4 / i[4])
    assert [o, o2, o3, o4, o5] == [104.0, -8.0, 8.0, 80.0, 20.0]
    # tests/ir/dtypes/test_fp8e4m3.py increment/decrement literals
    assert rt(rt(9.0) + 1) == 10.0 and rt(rt(-4.0) - 1) == -5.0


@pytest.mark.parametrize('a_shape, b_shape', [[[256, 128], [256, 128]], [[512, 256], [128, 256]]])
def test_matmul_f8_reference_recipe(a_shape, b_shape):
    # tests/operators_core/test_matmul.py:250-288: randint(-3, 3) inputs, output in e4m3
    rng = np.random.default_rng(41)
    ai = rng.integers(-3, 3, a_shape)
    bi = rng.integers(-3, 3, b_shape)
    ac, bc = O.e4m3_encode(ai.astype(np.float32)), O.e4m3_encode(bi.astype(np.float32))
    exact = (ai.astype(np.int64) @ bi.astype(np.int64).T)
    got32 = O.matmul_f8(ac, bc, out_dtype='float32')
    assert np.array_equal(got32.astype(np.int64), exact)
    got8 = O.matmul_f8(ac, bc)  # default output dtype: the fp8 input type
    want8 = torch.from_numpy(np.clip(exact, -448, 448).astype(np.float32)).to(torch.float8_e4m3fn).view(torch.uint8)
    assert np.array_equal(got8, want8.numpy())


def test_matmul_f8_scaled_reference_recipe():
    # tests/operators_core/test_matmul.py:291-373: integer inputs in [-5, 4], integer scales 1..4, expected
    # value built by pre-multiplying the scales into the operands
    rng = np.random.default_rng(42)
    m, n, k = 64, 256, 384
    ai = rng.integers(-5, 5, (m, k))
    bi = rng.integers(-5, 5, (n, k))
    sa = rng.integers(1, 5, (k // 128, m)).astype(np.float32)
    sb = rng.integers(1, 5, (n // 128, k // 128)).astype(np.float32)
    got = O.matmul_f8_scaled(O.e4m3_encode(ai.astype(np.float32)), O.e4m3_encode(bi.astype(np.float32)), sa, sb,
                             out_dtype='float32')
    a2 = ai.astype(np.int64) * np.repeat(sa.T.astype(np.int64), 128, axis=1)
    b2 = bi.astype(np.int64) * np.repeat(np.repeat(sb.astype(np.int64), 128, axis=0), 128, axis=1)
    assert np.array_equal(got.astype(np.int64), a2 @ b2.T)


def test_matmul_f8_scaled_e5m2_reference_recipe():
    # the same recipe on float8_e5m2 codes (both operands e5m2: matmul_f8.py:386-389, 709-712); integers up to 4 and the
    # integer scales are exact in e5m2, so the pre-multiplied integer product pins the decode and the block indexing
    rng = np.random.default_rng(43)
    m, n, k = 48, 256, 384
    ai = rng.integers(-4, 5, (m, k))
    bi = rng.integers(-4, 5, (n, k))
    sa = rng.integers(1, 5, (k // 128, m)).astype(np.float32)
    sb = rng.integers(1, 5, (n // 128, k // 128)).astype(np.float32)
    ac, bc = O.e5m2_encode(ai.astype(np.float32)), O.e5m2_encode(bi.astype(np.float32))
    got = O.matmul_f8_scaled(ac, bc, sa, sb, out_dtype='float32', in_dtype='float8_e5m2')
    a2 = ai.astype(np.int64) * np.repeat(sa.T.astype(np.int64), 128, axis=1)
    b2 = bi.astype(np.int64) * np.repeat(np.repeat(sb.astype(np.int64), 128, axis=0), 128, axis=1)
    assert np.array_equal(got.astype(np.int64), a2 @ b2.T)
    # the same bytes read as e4m3 are other numbers: the format argument is not ignored
    assert not np.array_equal(O.matmul_f8_scaled(ac, bc, sa, sb, out_dtype='float32'), got)


def test_e5m2_codec_against_torch_and_float16():
    # decode: every code against torch.float8_e5m2 and against "upper byte of the float16 of the same value"
    codes = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(codes).view(torch.float8_e5m2).float().numpy()
    got = O.e5m2_decode(codes)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])
    assert got[0x7B] == 57344.0 and np.isinf(got[0x7C]) and got[0x01] == 2.0 ** -16 and got[0x04] == 2.0 ** -14
    # encode: round to nearest even against torch inside the finite range (torch overflows to infinity beyond it, the
    # reference's type saturates: checked separately), every midpoint between neighbouring codes included
    tab = got[:0x7C].astype(np.float64)
    mids = (tab[:-1] + tab[1:]) / 2
    rng = np.random.default_rng(2)
    xs = np.concatenate([tab, mids, np.nextafter(mids.astype(np.float32), np.float32(0)).astype(np.float64),
                         np.nextafter(mids.astype(np.float32), np.float32(1e9)).astype(np.float64),
                         rng.standard_normal(4000) * 100, rng.standard_normal(4000) * 1e-4]).astype(np.float32)
    xs = np.concatenate([xs, -xs])
    xs = xs[np.abs(xs) <= 57344]
    want = torch.from_numpy(xs).to(torch.float8_e5m2).view(torch.uint8).numpy()
    assert np.array_equal(O.e5m2_encode(xs), want)
    # saturation and NaN of the reference's conversion
    sat = O.e5m2_encode(np.array([57344.0, 60000.0, 65504.0, 1e9, np.inf, -1e9, -np.inf, 61439.9], dtype=np.float32))
    assert sat.tolist() == [0x7B, 0x7B, 0x7B, 0x7B, 0x7B, 0xFB, 0xFB, 0x7B]
    assert (O.e5m2_encode(np.array([np.nan], dtype=np.float32))[0] & 0x7F) == 0x7F
    assert O.e5m2_encode(np.array([2.0 ** -17, 2.0 ** -17 * 1.0001, 3 * 2.0 ** -17], dtype=np.float32)).tolist() == [0, 1, 2]


def test_matmul_f8_e5m2_reference_recipe():
    # tests/operators_core/test_matmul.py:250-288 with float8_e5m2 operands: small integers, exact result
    rng = np.random.default_rng(43)
    ai, bi = rng.integers(-3, 3, (20, 96)), rng.integers(-3, 3, (12, 96))
    ac, bc = O.e5m2_encode(ai.astype(np.float32)), O.e5m2_encode(bi.astype(np.float32))
    assert np.array_equal(O.e5m2_decode(ac), ai) and np.array_equal(O.e5m2_decode(bc), bi)
    exact = ai.astype(np.int64) @ bi.astype(np.int64).T
    assert np.array_equal(O.matmul_f8(ac, bc, out_dtype='float32', in_dtype='float8_e5m2').astype(np.int64), exact)
    got8 = O.matmul_f8(ac, bc, in_dtype='float8_e5m2')  # default output: the input type
    assert np.array_equal(got8, O.e5m2_encode(exact.astype(np.float32)))
    # the same codes read as e4m3 are different numbers: the decode table matters
    assert not np.array_equal(O.matmul_f8(ac, bc, out_dtype='float32'), exact)


def test_fp8_per_tensor_quantize_and_matmul():
    a32, b32 = O.make_inputs(0, 32, 256, 48)
    b32 = b32.T.copy()  # [N, K]
    ac, sa = O.fp8_quantize_per_tensor(a32)
    bc, sb = O.fp8_quantize_per_tensor(b32)
    assert sa == np.float32(np.abs(a32).max() / np.float32(448)) and O.e4m3_decode(ac).max() <= 448
    assert np.abs(O.e4m3_decode(ac)).max() == 448.0  # the amax element maps onto the largest code
    out = O.fp8_matmul_per_tensor(ac, bc, sa, sb, 'bfloat16')
    want = a32.astype(np.float64) @ b32.astype(np.float64).T
    assert O.max_rel_err(out, want) < 6e-2  # quantization error of two e4m3 operands
    ref = (O.e4m3_decode(ac).astype(np.float64) @ O.e4m3_decode(bc).astype(np.float64).T) * float(sa) * float(sb)
    assert O.max_rel_err(out, ref) < 5e-3  # only the bf16 output rounding remains
    zc, zs = O.fp8_quantize_per_tensor(np.zeros((2, 2), dtype=np.float32))
    assert zs == 0 and not zc.any()


def test_fp8_per_tensor_matmul_exact_case():
    # integer-valued e4m3 codes and power-of-two scales: every product, the sum and the rescaling are exact in fp32,
    # so a dropped scale, a transposed operand or a wrong accumulation shows as a whole-number difference
    rng = np.random.default_rng(17)
    ai = rng.integers(-8, 9, (6, 128))
    bi = rng.integers(-8, 9, (10, 128))
    ac, bc = O.e4m3_encode(ai.astype(np.float32)), O.e4m3_encode(bi.astype(np.float32))
    assert np.array_equal(O.e4m3_decode(ac), ai) and np.array_equal(O.e4m3_decode(bc), bi)
    for sa, sb in ((0.5, 4.0), (2.0 ** -6, 2.0 ** 3), (1.0, 1.0)):
        want = (ai.astype(np.int64) @ bi.astype(np.int64).T).astype(np.float64) * sa * sb
        got = O.fp8_matmul_per_tensor(ac, bc, np.float32(sa), np.float32(sb), 'float32')
        assert np.array_equal(got.astype(np.float64), want)
        gotb = O.fp8_matmul_per_tensor(ac, bc, np.float32(sa), np.float32(sb), 'bfloat16')
        assert np.array_equal(gotb, O.to_bf16(want.astype(np.float32)))
    # per-tensor quantization of a tensor whose amax is 448 * 2^j leaves every representable value unchanged
    x = np.array([[448.0, -3.0, 0.25, 9.0 / 8.0]], dtype=np.float32) * np.float32(4.0)
    codes, scale = O.fp8_quantize_per_tensor(x)
    assert scale == np.float32(4.0) and np.array_equal(O.e4m3_decode(codes) * scale, x)


def test_max_rel_err_definition():
    assert O.max_rel_err(np.array([1.0, 10.0]), np.array([1.1, 10.0])) == pytest.approx(0.01)
    assert O.max_rel_err(np.array([0.5]), np.array([0.0])) == 0.5


def test_make_inputs_is_reproducible():
    import hashlib
    a, w = O.make_inputs(0, 1, 4096, 64)
    # digests of the generated float32 bytes: guards against drift of numpy's generator across versions
    assert hashlib.sha256(a.tobytes()).hexdigest()[:16] == _DIGESTS['a']
    assert hashlib.sha256(w.tobytes()).hexdigest()[:16] == _DIGESTS['w']


_DIGESTS = {'a': '69d00c4eb4c2d624', 'w': 'c64162dabba6a903'}


# ----------------------------------------------------------------------------- golden vectors of the reference's half type

def test_oracle_against_golden_vectors_of_reference_half_type():
    # tests/golden/ref_half_vectors.npz holds operand bit patterns and the results the reference's own CPU half type
    # (include/hidet/runtime/cpu/float16.h, compiled by oracle/Makefile's `ref` target) produced for them; written by
    # tests/golden/make_ref_half_vectors.py. This test needs neither the reference checkout nor the built driver.
    import os

    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'ref_half_vectors.npz'), allow_pickle=False)
    fa = g['op_a'].view(np.float16).astype(np.float32)
    fb = g['op_b'].view(np.float16).astype(np.float32)
    with np.errstate(over='ignore', divide='ignore', invalid='ignore'):
        for name, exact in (('mul', fa * fb), ('add', fa + fb), ('div', fa / fb)):
            # every operator of the type is: widen to float32, operate, round to nearest even
            assert np.array_equal(exact.astype(np.float32).astype(np.float16).view(np.uint16), g['op_' + name]), name
    r = O.round_half_away(g['round_in'].view(np.float16).astype(np.float32)).astype(np.float16)
    assert np.array_equal(r.view(np.uint16), g['round_out'])
    with np.errstate(over='ignore'):
        assert np.array_equal(g['cvt_f32'].astype(np.float16).view(np.uint16), g['cvt_f16'])
        L = clib.lib()
        ours = np.array([L.oracle_f32_to_f16(float(x)) for x in g['cvt_f32']], dtype=np.uint16)  # the C restatement's own conversion
        assert np.array_equal(ours, g['cvt_f16'])
    # symmetric_quantize on float16 columns, every operator in the reference's half arithmetic. The oracle saturates
    # where the reference's cast wraps (a quotient that rounds to 128): those codes read -128 in the fixture.
    w16 = g['quant_w_bits'].view(np.float16)
    q, s = O.symmetric_quantize(w16, 'int8', dims=0)
    assert np.array_equal(s.view(np.uint16), g['quant_scale_bits'])
    differs = q != g['quant_codes']
    assert np.all(g['quant_codes'][differs] == -128) and np.all(q[differs] == 127) and differs.sum() <= 4
    # the reference's CPU route of the matmul (float16 accumulator), restated in numpy and in C
    a = g['mm_a_bits'].view(np.float16)
    sc = g['mm_scale_bits'].view(np.float16)
    want = g['mm_c_bits'].view(np.float16)
    assert np.array_equal(O.reference_cpu_quant_matmul(a, g['mm_w'], sc).view(np.uint16), g['mm_c_bits'])
    assert np.array_equal(clib.quant_matmul_ref_cpu(a, g['mm_w'], sc).view(np.uint16), want.view(np.uint16))
