"""A wider seeded walk over random shapes than test_gpu_random_shapes.py, with the fused bias and tall matrices, on
operands whose exact result is known.

Small integers, power-of-two (or small integer) scales: every partial sum is an integer below 2^24 times a power of two,
so fp32 accumulation is exact whatever the tiling, the K ranges or the order of an exchange, and the kernel's output
must equal integer arithmetic followed by the one (two, with a bias) rounding of the definition - bit for bit. The
shapes are drawn around the boundaries where the launchers change kernel or plan (16 / 32 / 64 / 128 / 256 / 512 rows,
ragged K and N), and a few tall ones reach the plans of whole rounds, K ranges of tail tiles and runs across tiles.
A failure prints the family, the shape and the index of the case (the generator is seeded, so it reproduces)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from hidet_amd.graph.ops import quant
from hidet_amd.graph.ops.matmul import matmul_f8 as F8
from gpu_util import announce, dev

pytestmark = pytest.mark.gpu

EDGE_ROWS = [31, 32, 33, 63, 64, 65, 96, 97, 127, 128, 129, 255, 256, 257, 383, 384, 385, 511, 512, 513]


def _rows(rng):
    r = rng.integers(0, 10)
    if r < 4:
        return int(rng.integers(1, 17))
    if r < 6:
        return int(rng.integers(17, 130))
    if r < 8:
        return int(rng.choice(EDGE_ROWS))
    return int(rng.integers(130, 1100))


def _f16(x):
    with np.errstate(over='ignore'):
        return x.astype(np.float32).astype(np.float16)


def _w8_case(rng, kind, tall):
    m = _rows(rng)
    k = int(rng.choice([32, 64, 96, 128, 192, 256, 320, 512, 1000, 1024, 2048, 4096, 4100, 11008]))
    if rng.integers(0, 4) == 0:
        k = 2 * int(rng.integers(1, 300))  # the operator asks for an even K, as the reference does
    n = int(rng.choice([4, 8, 16, 64, 128, 256, 260, 272, 512, 516, 1024, 2048, 4096, 11008]))
    if rng.integers(0, 4) == 0:
        n = 4 * int(rng.integers(1, 300))
    if tall:
        m, n, k = int(rng.integers(513, 2100)), int(rng.choice([4096, 5504, 8192, 11008, 12288])), 64 * int(rng.integers(4, 65))
    elif m * k * n > 3e9:
        m = max(1, int(3e9 / (k * n)))
    a = rng.integers(-3, 4, (m, k)).astype(np.float32)
    w = rng.integers(-127, 128, (k, n)).astype(np.int8)
    s = (2.0 ** rng.integers(-6, 1, n)).astype(np.float32)
    want = _f16((a.astype(np.float64) @ w.astype(np.float64)) * s)
    tw, bias = dev(w), None
    if kind == 'w8a16, K-contiguous weights':
        tw = quant.to_decode_layout(tw)
    if kind == 'w8a16 with bias':
        b = (rng.integers(-64, 65, n) / 8.0).astype(np.float16)
        bias = dev(b)
        with np.errstate(over='ignore'):
            want = (want.astype(np.float32) + b.astype(np.float32)).astype(np.float16)
    got = quant.symmetric_quant_matmul(dev(a, torch.float16), tw, dev(s, torch.float16), bias).cpu().numpy()
    return (m, k, n), np.array_equal(got.view(np.uint16), want.view(np.uint16))


def _w4_case(rng, kind, tall):
    m = _rows(rng)
    g = int(rng.choice([32, 64, 128, 128, 128, 256]))
    k = g * int(rng.integers(1, max(2, 4096 // g + 1)))
    if rng.integers(0, 3) == 0:
        k = int(rng.choice([g, 2 * g, 1024, 2048, 4096]))
    k = max(g, (k // g) * g)
    n = int(rng.choice([16, 32, 64, 128, 256, 264, 272, 512, 544, 1024, 2048, 4096, 11008]))
    if rng.integers(0, 4) == 0:
        n = 8 * int(rng.integers(1, 200))
    if tall:
        m, n = int(rng.integers(513, 1800)), int(rng.choice([4096, 5504, 8192, 11008, 11040]))
        k = max(g, (128 * int(rng.integers(4, 33)) // g) * g)
    elif m * k * n > 3e9:
        m = max(1, int(3e9 / (k * n)))
    if kind == 'w4a16, decode layout' and (k % 128 or g % 128 or n % 16):
        g, k, n = 128, 128 * (k // 128 + 1), 16 * (n // 16 + 1)
    dt = torch.bfloat16 if rng.integers(0, 2) else torch.float16
    a = rng.integers(-3, 4, (m, k)).astype(np.float32)
    q = rng.integers(-8, 8, (k, n)).astype(np.int8)
    sc = (2.0 ** rng.integers(-3, 1, (k // g, n))).astype(np.float32)
    want = np.zeros((m, n))
    for gi in range(k // g):
        want += (a[:, gi * g:(gi + 1) * g].astype(np.float64) @ q[gi * g:(gi + 1) * g].astype(np.float64)) * sc[gi]
    packed = dev(O.pack_int4(q))
    bias = None
    if kind == 'w4a16 with bias':
        bias = (rng.integers(-40, 41, n) / 8.0).astype(np.float32)
    if kind == 'w4a16, decode layout':
        got = quant.symmetric_quant_matmul_w4a16_decode(dev(a, dt), quant.to_decode_layout_int4(packed), dev(sc, dt), g)
    else:
        got = quant.symmetric_quant_matmul_w4a16(dev(a, dt), packed, dev(sc, dt), g, bias=None if bias is None else dev(bias, dt))
    exp = O.to_bf16(want.astype(np.float32)) if dt == torch.bfloat16 else _f16(want).astype(np.float32)
    if bias is not None:  # the second rounding
        exp = O.to_bf16(exp + bias) if dt == torch.bfloat16 else _f16(exp + bias).astype(np.float32)
    return (m, k, n, g, str(dt)), np.array_equal(got.float().cpu().numpy(), exp.astype(np.float32))


def _f8_case(rng, kind, tall):
    m = _rows(rng)
    if kind == 'matmul_f8_scaled':
        k, n = 128 * int(rng.integers(1, 40)), 128 * int(rng.integers(1, 24))
    else:
        k, n = 16 * int(rng.integers(1, 300)), int(rng.choice([16, 64, 128, 256, 272, 512, 1024, 1152, 2048, 4096, 8192]))
        if rng.integers(0, 4) == 0:
            n = 16 * int(rng.integers(1, 100))
    if tall:
        m, n, k = int(rng.integers(513, 4200)), 128 * int(rng.integers(8, 65)), 128 * int(rng.integers(2, 33))
    elif m * k * n > 3e9:
        m = max(1, int(3e9 / (k * n)))
    ai, bi = rng.integers(-3, 3, (m, k)), rng.integers(-3, 3, (n, k))
    ta = dev(O.e4m3_encode(ai.astype(np.float32))).view(torch.float8_e4m3fn)
    tb = dev(O.e4m3_encode(bi.astype(np.float32))).view(torch.float8_e4m3fn)
    if kind == 'matmul_f8_scaled':
        sa = rng.integers(1, 5, (k // 128, m)).astype(np.float32)
        sb = rng.integers(1, 5, (n // 128, k // 128)).astype(np.float32)
        a2 = ai.astype(np.float64) * np.repeat(sa.T.astype(np.float64), 128, axis=1)
        b2 = bi.astype(np.float64) * np.repeat(np.repeat(sb.astype(np.float64), 128, axis=0), 128, axis=1)
        exact = a2 @ b2.T
        got = F8.matmul_f8_scaled(ta, tb, scale_a=dev(sa), scale_b=dev(sb), output_dtype='float32')
    else:
        exact = ai.astype(np.float64) @ bi.astype(np.float64).T
        got = F8.matmul_f8(ta, tb, output_dtype='float32')
    return (m, k, n), np.array_equal(got.cpu().numpy().astype(np.int64), exact.astype(np.int64))


FAMILIES = [('w8a16', _w8_case, 11), ('w8a16, K-contiguous weights', _w8_case, 12), ('w8a16 with bias', _w8_case, 13),
            ('w4a16', _w4_case, 14), ('w4a16, decode layout', _w4_case, 15), ('w4a16 with bias', _w4_case, 18), ('matmul_f8', _f8_case, 16),
            ('matmul_f8_scaled', _f8_case, 17)]


@pytest.mark.parametrize('kind,case,seed', FAMILIES, ids=[f[0] for f in FAMILIES])
def test_random_shapes_exact(kind, case, seed):
    rng = np.random.default_rng(seed)
    for i in range(70):
        shape, ok = case(rng, kind, False)
        assert ok, (kind, shape, 'case', i)
    announce(kind, '70 random shapes exact')


@pytest.mark.parametrize('kind,case,seed', [f for f in FAMILIES if 'contiguous' not in f[0] and 'decode' not in f[0]],
                         ids=[f[0] for f in FAMILIES if 'contiguous' not in f[0] and 'decode' not in f[0]])
def test_random_tall_shapes_exact(kind, case, seed):
    rng = np.random.default_rng(100 + seed)
    for i in range(6):
        shape, ok = case(rng, kind, True)
        assert ok, (kind, shape, 'case', i)
    announce(kind, '6 random tall shapes exact')
