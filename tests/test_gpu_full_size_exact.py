"""Every output element of every benchmark configuration, at full size, against integer arithmetic.

The parity tests compare the full-size configurations with the oracle on samples of rows (the oracle's float arithmetic
takes minutes on whole prefill matrices). Here the operands are small integers with power-of-two (or small integer)
scales: every product and every fp32 partial sum is exact whatever the tiling, so the expected result is an integer
matrix product (float64 BLAS, exact on these values) followed by the one rounding of the output type - and the whole
output must match it bit for bit: a dropped tile, row block, K range, column or exchange slot anywhere shows."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from hidet_amd.graph.ops import quant
from hidet_amd.graph.ops.matmul import matmul_f8 as F8
from gpu_util import announce, dev

pytestmark = pytest.mark.gpu


def _f16(x):
    with np.errstate(over='ignore'):
        return x.astype(np.float32).astype(np.float16)


@pytest.mark.parametrize('m,k,n', [(16, 4096, 4096),                       # C1
                                   (1, 4096, 11008), (1, 11008, 4096),      # C2 up and down
                                   (2048, 4096, 11008), (2048, 4096, 12288)])  # C3
def test_w8a16_whole_output_exact(m, k, n):
    announce('w8a16 full size exact', m, k, n)
    rng = np.random.default_rng(k + n + m)
    a = rng.integers(-3, 4, (m, k)).astype(np.float32)
    w = rng.integers(-127, 128, (k, n)).astype(np.int8)
    s = (2.0 ** rng.integers(-8, -3, n)).astype(np.float32)
    want = _f16((a.astype(np.float64) @ w.astype(np.float64)) * s)
    ta, tw, ts = dev(a, torch.float16), dev(w), dev(s, torch.float16)
    got = quant.symmetric_quant_matmul(ta, tw, ts).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    if m <= 16:  # the same weight stored K-contiguous (the decode layout)
        got = quant.symmetric_quant_matmul(ta, quant.to_decode_layout(tw), ts).cpu().numpy()
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize('m', [1, 16, 512])  # C4
def test_w4a16_whole_output_exact(m):
    k, n, g = 4096, 11008, 128
    announce('w4a16 full size exact', m, k, n)
    rng = np.random.default_rng(40 + m)
    a = rng.integers(-3, 4, (m, k)).astype(np.float32)
    q = rng.integers(-8, 8, (k, n)).astype(np.int8)
    sc = (2.0 ** rng.integers(-3, 1, (k // g, n))).astype(np.float32)
    want = np.zeros((m, n))
    for gi in range(k // g):
        want += (a[:, gi * g:(gi + 1) * g].astype(np.float64) @ q[gi * g:(gi + 1) * g].astype(np.float64)) * sc[gi]
    want = O.to_bf16(want.astype(np.float32))
    packed = dev(O.pack_int4(q))
    got = quant.symmetric_quant_matmul_w4a16(dev(a, torch.bfloat16), packed, dev(sc, torch.bfloat16), g)
    assert np.array_equal(got.float().cpu().numpy(), want)
    if m <= 16:
        got = quant.symmetric_quant_matmul_w4a16_decode(dev(a, torch.bfloat16), quant.to_decode_layout_int4(packed), dev(sc, torch.bfloat16), g)
        assert np.array_equal(got.float().cpu().numpy(), want)


@pytest.mark.parametrize('m', [1, 4096])  # C5
def test_fp8_whole_output_exact(m):
    k, n = 8192, 8192
    announce('fp8 full size exact', m, k, n)
    rng = np.random.default_rng(50 + m)
    ai, bi = rng.integers(-3, 3, (m, k)), rng.integers(-3, 3, (n, k))
    ta = dev(O.e4m3_encode(ai.astype(np.float32))).view(torch.float8_e4m3fn)
    tb = dev(O.e4m3_encode(bi.astype(np.float32))).view(torch.float8_e4m3fn)
    exact = ai.astype(np.float64) @ bi.astype(np.float64).T
    got = F8.matmul_f8(ta, tb, output_dtype='float32').cpu().numpy()
    assert np.array_equal(got.astype(np.int64), exact.astype(np.int64))
    got = F8.matmul_f8(ta, tb, output_dtype='bfloat16').float().cpu().numpy()
    assert np.array_equal(got, O.to_bf16(exact.astype(np.float32)))
