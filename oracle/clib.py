"""ctypes access to the oracle's C restatement (liboracle.so) and, where it was built, to the
driver around the reference's own CPU half type (oracle/_ref/libref_half.so).

TEST INFRASTRUCTURE ONLY: imported by tests, the smoke check and the benchmark's CPU-baseline
leg; never by the product package."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_REF = None

_i64, _i32, _f32, _u16, _vp = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_uint16, ctypes.c_void_p


def build():
    subprocess.check_call(['make', '-s', '-C', _HERE, 'all'])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, 'liboracle.so')
        if not os.path.exists(path):
            build()
        L = ctypes.CDLL(path)
        L.oracle_f32_to_f16.argtypes, L.oracle_f32_to_f16.restype = [_f32], _u16
        L.oracle_f16_to_f32.argtypes, L.oracle_f16_to_f32.restype = [_u16], _f32
        L.oracle_roundf.argtypes, L.oracle_roundf.restype = [_f32], _f32
        L.oracle_symmetric_quantize_f32.argtypes = [_vp, _i64, _i64, _i32, _i32, _i32, _vp, _vp]
        L.oracle_symmetric_quantize_f32.restype = None
        for name in ('oracle_quant_matmul_f32acc', 'oracle_quant_matmul_ref_cpu'):
            getattr(L, name).argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64]
            getattr(L, name).restype = None
        L.oracle_baseline_quant_matmul.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64]
        L.oracle_baseline_quant_matmul.restype = None
        L.oracle_baseline_threads.restype = _i32
        _LIB = L
    return _LIB


def ref_lib():
    """The driver around the reference's half type, or None when it was not built."""
    global _REF
    if _REF is None:
        path = os.path.join(_HERE, '_ref', 'libref_half.so')
        if not os.path.exists(path):
            return None
        R = ctypes.CDLL(path)
        R.ref_f32_to_f16.argtypes, R.ref_f32_to_f16.restype = [_f32], _u16
        R.ref_f16_to_f32.argtypes, R.ref_f16_to_f32.restype = [_u16], _f32
        for name in ('ref_half_mul', 'ref_half_add', 'ref_half_div'):
            getattr(R, name).argtypes, getattr(R, name).restype = [_u16, _u16], _u16
        R.ref_half_round.argtypes, R.ref_half_round.restype = [_u16], _u16
        R.ref_quant_matmul_cpu.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64]
        R.ref_quant_matmul_cpu.restype = None
        R.ref_symmetric_quantize_f16_axis0.argtypes = [_vp, _i64, _i64, _vp, _vp]
        R.ref_symmetric_quantize_f16_axis0.restype = None
        _REF = R
    return _REF


def _p(x):
    return x.ctypes.data_as(_vp)


def symmetric_quantize_f32(w, reduce_axis, quant_type='int8'):
    w = np.ascontiguousarray(w, dtype=np.float32)
    rows, cols = w.shape
    qmax, nbytes, npdt = (127, 1, np.int8) if quant_type == 'int8' else (32767, 2, np.int16)
    codes = np.empty((rows, cols), dtype=npdt)
    scale = np.empty(cols if reduce_axis == 0 else rows, dtype=np.float32)
    lib().oracle_symmetric_quantize_f32(_p(w), rows, cols, reduce_axis, qmax, nbytes, _p(codes), _p(scale))
    return codes, scale


def _mm(fn, a, w, scale):
    a = np.ascontiguousarray(a, dtype=np.float16)
    w = np.ascontiguousarray(w, dtype=np.int8)
    scale = np.ascontiguousarray(scale, dtype=np.float16)
    m, k = a.shape
    n = w.shape[1]
    c = np.empty((m, n), dtype=np.float16)
    fn(_p(a), _p(w), _p(scale), _p(c), m, k, n)
    return c


def quant_matmul_f32acc(a, w, scale):
    return _mm(lib().oracle_quant_matmul_f32acc, a, w, scale)


def quant_matmul_ref_cpu(a, w, scale):
    return _mm(lib().oracle_quant_matmul_ref_cpu, a, w, scale)


def baseline_quant_matmul(a, w, scale, col_begin=0, col_end=None):
    """Reference-flag build of the reference's CPU loop nest over columns [col_begin, col_end)."""
    a = np.ascontiguousarray(a, dtype=np.float16)
    w = np.ascontiguousarray(w, dtype=np.int8)
    scale = np.ascontiguousarray(scale, dtype=np.float16)
    m, k = a.shape
    n = w.shape[1]
    col_end = n if col_end is None else col_end
    c = np.zeros((m, n), dtype=np.float16)
    lib().oracle_baseline_quant_matmul(_p(a), _p(w), _p(scale), _p(c), m, k, n, col_begin, col_end)
    return c
