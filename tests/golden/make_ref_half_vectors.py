"""Writes tests/golden/ref_half_vectors.npz: inputs and outputs of the reference's own CPU half type.

The outputs come from oracle/_ref/libref_half.so, i.e. from the reference's include/hidet/runtime/cpu/float16.h compiled
here by `make -C oracle ref` (only possible where the reference checkout is present). The file holds data only - operand
bit patterns and the bit patterns the reference type produced - so that the oracle can be pinned against the reference's
arithmetic on machines that have neither the checkout nor the built driver.

    python tests/golden/make_ref_half_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import clib  # noqa: E402


def main():
    R = clib.ref_lib()
    if R is None:
        raise SystemExit('oracle/_ref/libref_half.so is not built: run `make -C oracle ref` with the reference checkout present')
    rng = np.random.default_rng(20240607)
    out = {}

    # binary operators and round() on random finite halves (plus a few hand-picked ties)
    n = 4096
    a = (rng.integers(0, 0x7C00, n) | (rng.integers(0, 2, n) << 15)).astype(np.uint16)
    b = (rng.integers(1, 0x7C00, n) | (rng.integers(0, 2, n) << 15)).astype(np.uint16)
    out['op_a'], out['op_b'] = a, b
    for name in ('mul', 'add', 'div'):
        fn = getattr(R, 'ref_half_' + name)
        out['op_' + name] = np.array([fn(int(x), int(y)) for x, y in zip(a, b)], dtype=np.uint16)
    ties = np.array([100.5, 2.5, -2.5, 0.5, -0.5, 1.5, 1.4990234375, 126.5, -126.5, 127.5, 0.0, 65504.0], dtype=np.float16)
    r_in = np.concatenate([a[:1024], ties.view(np.uint16)])
    out['round_in'] = r_in
    out['round_out'] = np.array([R.ref_half_round(int(x)) for x in r_in], dtype=np.uint16)

    # float32 -> half conversion, including values that round to subnormals, ties and overflow
    f = np.concatenate([rng.standard_normal(2048).astype(np.float32) * np.float32(10.0) ** rng.integers(-8, 5, 2048).astype(np.float32),
                        np.array([65504.0, 65519.9, 65520.0, 1e-8, 5.9604645e-8, 2.9802322e-8, 1.0009766, 1.0004883, 1.0014648],
                                 dtype=np.float32)]).astype(np.float32)
    out['cvt_f32'] = f
    out['cvt_f16'] = np.array([R.ref_f32_to_f16(float(x)) for x in f], dtype=np.uint16)

    # symmetric_quantize of float16 columns (graph/ops/quant/symmetric.py:23-47 on the reference's half type)
    cols = []
    pat = np.arange(0, 0x7C00, 37, dtype=np.uint16)
    for top in (0x7BFF, 0x5BF0, 0x3C00, 0x2E66, 0x0400, 0x0011):
        col = np.concatenate([pat[pat <= top], np.array([top], dtype=np.uint16)])
        sign = (rng.integers(0, 2, col.size).astype(np.uint16) << 15)
        cols.append((col | sign).astype(np.uint16))
    rows = max(c.size for c in cols)
    mat = np.zeros((rows, len(cols)), dtype=np.uint16)
    for j, c in enumerate(cols):
        mat[: c.size, j] = c
    codes = np.empty(mat.shape, dtype=np.int8)
    scale = np.empty(mat.shape[1], dtype=np.uint16)
    R.ref_symmetric_quantize_f16_axis0(mat.ctypes.data, mat.shape[0], mat.shape[1], codes.ctypes.data, scale.ctypes.data)
    out['quant_w_bits'], out['quant_codes'], out['quant_scale_bits'] = mat, codes, scale

    # the reference's CPU route of symmetric_quant_matmul (half accumulator), small case
    m, k, nn = 5, 96, 12
    am = (rng.standard_normal((m, k))).astype(np.float16)
    wq = rng.integers(-127, 128, (k, nn)).astype(np.int8)
    sc = (rng.random(nn) * 0.02 + 0.001).astype(np.float16)
    c = np.empty((m, nn), dtype=np.uint16)
    R.ref_quant_matmul_cpu(am.ctypes.data, wq.ctypes.data, sc.ctypes.data, c.ctypes.data, m, k, nn)
    out['mm_a_bits'], out['mm_w'], out['mm_scale_bits'], out['mm_c_bits'] = am.view(np.uint16), wq, sc.view(np.uint16), c

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'ref_half_vectors.npz')
    np.savez_compressed(path, **out)
    print('wrote', path, os.path.getsize(path), 'bytes')


if __name__ == '__main__':
    main()
