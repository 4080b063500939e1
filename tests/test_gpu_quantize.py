"""GPU parity of symmetric_quantize / symmetric_dequantize: codes and scales bit-exact against the oracle."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from hidet_amd.graph.ops import quant
from gpu_util import announce, dev, host

pytestmark = pytest.mark.gpu


def _bits(x):
    return x.view(np.uint32) if x.dtype == np.float32 else x.view(np.uint16)


@pytest.mark.parametrize('w', [32, 64])
@pytest.mark.parametrize('dtype', ['int8', 'int16'])
@pytest.mark.parametrize('dims', [[-1], [0]])
def test_round_trip_reference_recipe(w, dtype, dims):
    # tests/operators_core/test_symmetric_quant.py:19-26 on the GPU, plus bit-exactness against the oracle
    announce('quantize round trip', w, dtype, dims)
    x = np.random.default_rng(w).standard_normal((w, w)).astype(np.float32)
    wq, scale = quant.symmetric_quantize(dev(x), dtype, dims)
    x1 = quant.symmetric_dequantize(wq, scale, dims)
    assert np.allclose(x, host(x1), atol=1e-1, rtol=1e-1)
    q0, s0 = O.symmetric_quantize(x, dtype, dims)
    assert np.array_equal(host(wq), q0) and np.array_equal(_bits(host(scale)), _bits(s0))
    assert np.array_equal(_bits(host(x1)), _bits(O.symmetric_dequantize(q0, s0, dims)))


@pytest.mark.parametrize('shape,dim', [([32, 32], 0), ([64, 64], 1), ([48, 200], 0), ([200, 48], 1)])
@pytest.mark.parametrize('atype', ['float16', 'bfloat16'])
def test_narrow_float_inputs_bit_exact(shape, dim, atype):
    # tests/operators_core/test_quantization.py:21-36 (fp16/bf16 -> int8 round trip) + oracle parity
    announce('quantize narrow', shape, dim, atype)
    rng = np.random.default_rng(shape[1] + dim)
    x32 = rng.standard_normal(shape).astype(np.float32)
    if atype == 'float16':
        x = x32.astype(np.float16)
        tx = dev(x)
        q0, s0 = O.symmetric_quantize(x, 'int8', dim, target='gpu')
        s0b = s0.view(np.uint16)
    else:
        x = O.to_bf16(x32)
        tx = dev(x, torch.bfloat16)
        q0, s0 = O.symmetric_quantize(x, 'int8', dim, dtype='bfloat16', target='gpu')
        s0b = O.bf16_bits(s0)
    wq, scale = quant.symmetric_quantize(tx, dims=dim, quant_type='int8')
    assert np.array_equal(host(wq), q0)
    assert np.array_equal(scale.view(torch.int16).cpu().numpy().view(np.uint16), s0b)
    back = quant.symmetric_dequantize(wq, scale, dims=dim)
    assert back.dtype == tx.dtype
    assert np.allclose(host(back).astype(np.float32), np.asarray(x, dtype=np.float32), atol=1e-1, rtol=1e-1)


def test_ties_zero_columns_and_saturation():
    announce('quantize ties / zero columns')
    col = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -126.5, 0.49999997], dtype=np.float32)
    w = np.stack([col, np.zeros_like(col), -col], axis=1)
    wq, scale = quant.symmetric_quantize(dev(w), 'int8', dims=0)
    q = host(wq)
    assert q[:, 0].tolist() == [127, 1, 2, 3, -1, -2, -3, 64, -127, 0]
    assert not q[:, 1].any() and host(scale)[1] == 0
    assert np.array_equal(q[:, 2], -q[:, 0])
    # subnormal float16 scale: the quotient of the amax element reaches 128 and the cast saturates
    bits = np.array([0x0400, 0x8400, 0x0123, 0x0200], dtype=np.uint16).view(np.float16).reshape(-1, 1)
    q0, s0 = O.symmetric_quantize(bits, 'int8', 0, target='gpu')
    wq, scale = quant.symmetric_quantize(dev(bits), 'int8', dims=0)
    assert np.array_equal(host(wq), q0) and np.array_equal(host(scale).view(np.uint16), s0.view(np.uint16))


@pytest.mark.parametrize('atype', ['float16', 'bfloat16'])
def test_narrow_float_ties_round_to_even(atype):
    # the reference's GPU lowering of round() for float16 / bfloat16 is hrint (ties to even); float32 keeps roundf
    # (ties away). amax 127 makes the scale exactly 1, so the quotients are the values themselves
    announce('quantize ties to even', atype)
    col = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, 64.5, -100.5, -101.5, 3.25, 3.75], dtype=np.float32)
    want_even = [127, 0, 2, 2, 0, -2, -2, 64, 64, -100, -102, 3, 4]
    want_away = [127, 1, 2, 3, -1, -2, -3, 64, 65, -101, -102, 3, 4]
    w = np.stack([col, -col], axis=1)
    tw = dev(w.astype(np.float16)) if atype == 'float16' else dev(O.to_bf16(w), torch.bfloat16)
    wq, scale = quant.symmetric_quantize(tw, 'int8', dims=0)
    assert host(wq)[:, 0].tolist() == want_even and host(wq)[:, 1].tolist() == [-v for v in want_even]
    assert host(scale.float()).tolist() == [1.0, 1.0]
    q_gpu, _ = O.symmetric_quantize(w, 'int8', 0, dtype=atype, target='gpu')
    q_cpu, _ = O.symmetric_quantize(w, 'int8', 0, dtype=atype, target='cpu')
    assert q_gpu[:, 0].tolist() == want_even and q_cpu[:, 0].tolist() == want_away
    wq32, _ = quant.symmetric_quantize(dev(w), 'int8', dims=0)  # float32 input: ties away on every target
    assert host(wq32)[:, 0].tolist() == want_away


@pytest.mark.parametrize('shape,dims', [([4, 6, 10], [1]), ([4, 6, 10], [0, 2]), ([4, 6, 10], [0, 1, 2]), ([3, 5, 7, 2], [-1, -2]),
                                        ([5, 0, 3], [1]), ([1, 1], [0])])
def test_general_dims(shape, dims):
    announce('quantize dims', shape, dims)
    x = np.random.default_rng(7).standard_normal(shape).astype(np.float32)
    q0, s0 = O.symmetric_quantize(x, 'int8', dims)
    wq, scale = quant.symmetric_quantize(dev(x), 'int8', dims)
    assert tuple(scale.shape) == s0.shape and tuple(wq.shape) == q0.shape
    assert np.array_equal(host(wq), q0) and np.array_equal(_bits(host(scale)), _bits(s0))
    back = quant.symmetric_dequantize(wq, scale, dims)
    assert np.array_equal(_bits(host(back)), _bits(O.symmetric_dequantize(q0, s0, dims)))


@pytest.mark.parametrize('k,n', [(4096, 4096), (4096, 11008), (11008, 4096), (4096, 12288)])
def test_benchmark_weight_shapes_bit_exact(k, n):
    announce('quantize benchmark shape', k, n)
    _, w = O.make_inputs(0, 1, k, n)
    wq, scale = quant.symmetric_quantize(dev(w), 'int8', dims=0)
    q0, s0 = O.symmetric_quantize(w, 'int8', dims=0)
    assert int((host(wq) != q0).sum()) == 0
    assert int((_bits(host(scale)) != _bits(s0)).sum()) == 0
    # full-size invariants: every column hits +-127, codes are odd-symmetric in w
    assert np.all(np.abs(host(wq).astype(np.int32)).max(axis=0) == 127)
    wq2, _ = quant.symmetric_quantize(dev(-w), 'int8', dims=0)
    assert torch.equal(wq2, -wq)


@pytest.mark.parametrize('rows,cols,qt,atype', [(1000, 4096, 'int8', 'float32'), (50, 5000, 'int8', 'float32'),
                                               (33, 16384, 'int16', 'float32'), (9, 16388, 'int8', 'float32'),
                                               (64, 4096, 'int8', 'float16'), (7, 1028, 'int16', 'bfloat16'),
                                               (5, 4094, 'int8', 'float32')])
def test_one_scale_per_row_bit_exact(rows, cols, qt, atype):
    # embedding tables (dims=-1): rows short enough for a workgroup's registers take the one-pass kernel, longer or
    # ragged ones the two-pass kernels; a zero row and tie values are planted
    announce('quantize rows', rows, cols, qt, atype)
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
    x[1] = 0.0
    x[2, :8] = x[2].max() * np.array([0.5, -0.5, 1.5, -1.5, 2.5, 100.5, -100.5, 126.5], dtype=np.float32) / 127
    if atype == 'float32':
        t = dev(x)
        q0, s0 = O.symmetric_quantize(x, qt, dims=-1)
        s0b = s0.view(np.uint32)
        view = torch.int32
    elif atype == 'float16':
        xh = x.astype(np.float16)
        t = dev(xh)
        q0, s0 = O.symmetric_quantize(xh, qt, dims=-1, target='gpu')
        s0b = s0.view(np.uint16)
        view = torch.int16
    else:
        xb = O.to_bf16(x)
        t = dev(xb, torch.bfloat16)
        q0, s0 = O.symmetric_quantize(xb, qt, dims=-1, dtype='bfloat16', target='gpu')
        s0b = O.bf16_bits(s0)
        view = torch.int16
    wq, scale = quant.symmetric_quantize(t, qt, dims=-1)
    assert int((host(wq) != q0).sum()) == 0
    got = scale.view(view).cpu().numpy()
    assert np.array_equal(got.view(np.uint32 if view == torch.int32 else np.uint16), s0b)
