"""Seeded random shapes through every matmul entry point against the oracle: the launchers choose among several kernels
by shape (row count, tile fit, alignment, K depth), and this walks those choices at sizes the oracle finishes in
seconds. Exactness: small-integer operands with power-of-two scales make every product and every fp32 partial sum
exact, so any dropped tile, row block, K range or column shows as a whole-number difference."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from hidet_amd.graph.ops import quant
from hidet_amd.graph.ops.matmul import matmul_f8 as F8
from gpu_util import announce, dev, host

pytestmark = pytest.mark.gpu


def _pick(rng, choices):
    return choices[int(rng.integers(0, len(choices)))]


@pytest.mark.parametrize('seed', range(6))
def test_w8a16_random_shapes_exact(seed):
    rng = np.random.default_rng(1000 + seed)
    for _ in range(8):
        m = int(_pick(rng, [1, 2, 7, 9, 15, 16, 17, 31, 33, 64, 65, 97, 128, 129, 200, 300, 520]))
        k = int(_pick(rng, [8, 64, 72, 128, 512, 1000, 1024, 2048, 4096]))
        n = int(_pick(rng, [2, 16, 100, 256, 260, 512, 1000, 2048, 4096, 8448]))
        announce('w8a16 random', m, k, n)
        a = rng.integers(-2, 3, (m, k)).astype(np.float16)
        q = rng.integers(-127, 128, (k, n)).astype(np.int8)
        s = (2.0 ** rng.integers(-12, -9, n)).astype(np.float16)
        want = (a.astype(np.int64) @ q.astype(np.int64)).astype(np.float64) * s.astype(np.float64)[None, :]
        got = host(quant.symmetric_quant_matmul(dev(a), dev(q), dev(s)))
        assert np.array_equal(got, want.astype(np.float32).astype(np.float16)), (m, k, n)
        # the same weight stored K-contiguous: up to 16 rows run the kernels for that layout, more rows a row-major copy
        got = host(quant.symmetric_quant_matmul(dev(a), quant.to_decode_layout(dev(q)), dev(s)))
        assert np.array_equal(got, want.astype(np.float32).astype(np.float16)), ('k-contiguous', m, k, n)


@pytest.mark.parametrize('seed', range(4))
@pytest.mark.parametrize('dtype', ['bfloat16', 'float16'])
def test_w4a16_random_shapes_exact(seed, dtype):
    rng = np.random.default_rng(2000 + seed)
    tdt = torch.bfloat16 if dtype == 'bfloat16' else torch.float16
    for _ in range(6):
        g = int(_pick(rng, [32, 64, 128]))
        m = int(_pick(rng, [1, 3, 16, 17, 33, 64, 100, 129, 256, 257, 300, 513, 600]))
        k = g * int(_pick(rng, [1, 2, 4, 8, 16, 32]))
        n = int(_pick(rng, [2, 48, 256, 264, 512, 544, 1024, 2080]))
        announce('w4a16 random', m, k, n, g, dtype)
        a = rng.integers(-3, 4, (m, k)).astype(np.float32)
        q = rng.integers(-8, 8, (k, n)).astype(np.int8)
        scales = (2.0 ** rng.integers(-3, 1, (k // g, n))).astype(np.float32)
        want = np.zeros((m, n))
        for gi in range(k // g):
            want += (a[:, gi * g:(gi + 1) * g].astype(np.int64) @ q[gi * g:(gi + 1) * g].astype(np.int64)) * scales[gi]
        got = host(quant.symmetric_quant_matmul_w4a16(dev(a, tdt), dev(O.pack_int4(q)), dev(scales, tdt), g))
        exp = O.to_bf16(want.astype(np.float32)) if dtype == 'bfloat16' else want.astype(np.float32).astype(np.float16)
        assert np.array_equal(got, exp), (m, k, n, g)
        if k % 128 == 0 and g == 128 and m <= 40:  # the decode layout of the same codes
            nk = quant.to_decode_layout_int4(dev(O.pack_int4(q)))
            got = host(quant.symmetric_quant_matmul_w4a16_decode(dev(a, tdt), nk, dev(scales, tdt), g))
            assert np.array_equal(got, exp), ('decode layout', m, k, n, g)


@pytest.mark.parametrize('seed', range(5))
def test_fp8_random_shapes_exact(seed):
    rng = np.random.default_rng(3000 + seed)
    for _ in range(6):
        m = int(_pick(rng, [1, 5, 16, 17, 40, 100, 128, 200, 256, 300, 512, 700, 1100]))
        k = int(_pick(rng, [16, 48, 128, 272, 384, 1024, 2048, 4096]))
        n = int(_pick(rng, [4, 36, 128, 260, 512, 1024, 1152, 2048]))
        announce('fp8 random', m, k, n)
        ai = rng.integers(-3, 3, (m, k))
        bi = rng.integers(-3, 3, (n, k))
        ta = torch.from_numpy(O.e4m3_encode(ai.astype(np.float32))).cuda().view(torch.float8_e4m3fn)
        tb = torch.from_numpy(O.e4m3_encode(bi.astype(np.float32))).cuda().view(torch.float8_e4m3fn)
        exact = (ai.astype(np.float64) @ bi.astype(np.float64).T).astype(np.int64)
        got = F8.matmul_f8(ta, tb, output_dtype='float32')
        assert np.array_equal(host(got).astype(np.int64), exact), (m, k, n)
        if k % 128 == 0 and n % 128 == 0:
            sa = rng.integers(1, 5, (k // 128, m)).astype(np.float32)
            sb = rng.integers(1, 5, (n // 128, k // 128)).astype(np.float32)
            a2 = ai.astype(np.int64) * np.repeat(sa.T.astype(np.int64), 128, axis=1)
            b2 = bi.astype(np.int64) * np.repeat(np.repeat(sb.astype(np.int64), 128, axis=0), 128, axis=1)
            exact2 = (a2.astype(np.float64) @ b2.astype(np.float64).T).astype(np.int64)
            got2 = F8.matmul_f8_scaled(ta, tb, scale_a=dev(sa), scale_b=dev(sb), output_dtype='float32')
            assert np.array_equal(host(got2).astype(np.int64), exact2), ('scaled', m, k, n)
