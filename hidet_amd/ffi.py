"""ctypes boundary to libhidet_qmm.so.

Mirrors how the reference calls a compiled task library: convert arguments to raw pointers and fixed-width
integers (python/hidet/ffi/convert.py:56-89), make the ctypes call, then poll `hidet_get_last_error` and raise
`BackendException` naming the function, its arguments and the library (python/hidet/runtime/compiled_module.py:56-104,
python/hidet/ffi/ffi.py:46-60).  There is no CPU fallback: if the library is missing or the tensors are not on
a GPU the call fails.
"""
import ctypes
import os
from typing import Dict, Optional, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'lib', 'libhidet_qmm.so')

_vp, _i64, _i32, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float

ABI_VERSION = 2  # HIDET_QMM_ABI_VERSION of include/hidet_qmm.h

# dtype codes of include/hidet_qmm.h
F32, F16, BF16, I8, I16, E4M3, E5M2 = 0, 1, 2, 3, 4, 5, 6
DTYPE_CODE = {
    torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.int8: I8, torch.int16: I16,
    torch.float8_e4m3fn: E4M3, torch.float8_e5m2: E5M2,
}

# name -> (restype, argtypes): every symbol include/hidet_qmm.h and include/hidet_qmm_bench.h declare
SIGNATURES = {
    'hidet_set_last_error': (None, [ctypes.c_char_p]),
    'hidet_get_last_error': (ctypes.c_char_p, []),
    'hidet_qmm_abi_version': (_i32, []),
    'hidet_qmm_arch': (ctypes.c_char_p, []),
    'hidet_qmm_min_workspace_bytes': (_i64, []),
    'hidet_qmm_workspace_bytes_for_scratch': (_i64, [_i64]),
    'hidet_qmm_exchange_status': (_i32, [_vp, _i64, _vp]),
    'hidet_qmm_exchange_reset': (None, [_vp, _i64, _vp]),
    'hidet_qmm_event_create': (_vp, []),
    'hidet_qmm_event_destroy': (None, [_vp]),
    'hidet_qmm_event_record': (None, [_vp, _vp]),
    'hidet_qmm_event_synchronize': (None, [_vp]),
    'hidet_qmm_event_elapsed_ms': (_f32, [_vp, _vp]),
    'hidet_qmm_arm_timing': (None, [_vp, _vp]),
    'hidet_qmm_gemv_ring_timed': (None, [_vp, _vp, _vp, _vp, _i32, _i32, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _vp, _vp]),
    'hidet_qmm_read_probe': (None, [_vp, _i64, _vp, _vp]),
    'hidet_qmm_pattern_probe': (None, [_vp, _i64, _i64, _i32, _i32, _vp, _vp]),
    'hidet_qmm_set_exchange_spin_limit': (None, [_i32]),
    'hidet_symmetric_quantize': (None, [_vp, _vp, _vp, _i64, _i64, _i64, _i32, _i32, _vp, _i64, _vp]),
    'hidet_symmetric_dequantize': (None, [_vp, _vp, _vp, _i64, _i64, _i64, _i32, _i32, _vp]),
    'hidet_symmetric_quant_matmul_f16_i8': (None, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _vp, _i64, _vp]),
    'hidet_symmetric_quant_matmul_f16_i8_bias': (None, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _vp, _i64, _vp]),
    'hidet_symmetric_quant_matmul_f16_i8_nk_bias': (None, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _vp]),
    'hidet_qmm_static_scratch_bytes': (_i64, []),
    'hidet_symmetric_quant_matmul_f16_i8_static': (None, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _vp]),
    'hidet_symmetric_quant_matmul_f16_i8_nk': (None, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _vp]),
    'hidet_group_quantize_int4': (None, [_vp, _vp, _vp, _i64, _i64, _i32, _i32, _i32, _vp]),
    'hidet_symmetric_quant_matmul_w4a16': (None, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _vp, _i64, _vp]),
    'hidet_symmetric_quant_matmul_w4a16_bias': (None, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _vp, _i64, _vp]),
    'hidet_symmetric_quant_matmul_w4a16_nk': (None, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _vp]),
    'hidet_fp8_quantize_per_tensor': (None, [_vp, _vp, _vp, _i64, _i32, _vp, _i64, _vp]),
    'hidet_matmul_f8': (None, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i32, _vp, _vp, _vp, _i64, _vp]),
    'hidet_matmul_f8_e5m2': (None, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i32, _vp, _vp, _vp]),
    'hidet_matmul_f8_scaled': (None, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp, _i64, _vp]),
    'hidet_matmul_f8_scaled_e5m2': (None, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp, _i64, _vp]),
}


class BackendException(Exception):
    """Raised when an entry point reported an error (same name as hidet.ffi.ffi.BackendException)."""


_LIB: Optional[ctypes.CDLL] = None


def load_library() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise OSError('{} not found: build it with `python -m hidet_amd.build` (hipcc, gfx950)'.format(LIB_PATH))
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = restype, argtypes
        if lib.hidet_qmm_abi_version() != ABI_VERSION:
            raise OSError('{} has ABI version {}, expected {}'.format(LIB_PATH, lib.hidet_qmm_abi_version(), ABI_VERSION))
        _LIB = lib
    return _LIB


def get_last_error() -> Optional[str]:
    ret = load_library().hidet_get_last_error()
    return ret.decode('utf-8') if isinstance(ret, bytes) else None


def _describe(arg) -> str:
    if isinstance(arg, torch.Tensor):
        return 'torch.Tensor(shape={}, dtype={}, device={})'.format(tuple(arg.shape), arg.dtype, arg.device)
    return str(arg)


_FUNCS: Dict[str, object] = {}
_Tensor = torch.Tensor


def call(name: str, *args):
    """Call `name` with torch tensors (passed as data pointers) and Python scalars; raise on a reported error.

    This sits on the decode path of an eager caller (one call per linear layer and token), so it is kept short: bound
    function objects are cached, and the error string is polled through a cached function object as well.
    """
    fn = _FUNCS.get(name)
    if fn is None:
        lib = load_library()
        fn = _FUNCS[name] = getattr(lib, name)
        _FUNCS.setdefault('hidet_get_last_error', lib.hidet_get_last_error)
    cargs = []
    for a in args:
        if isinstance(a, _Tensor):
            if not a.is_cuda:  # a host pointer must never reach a kernel
                raise BackendException('{}: tensor argument is on {}, the kernels run on the GPU only'.format(name, a.device))
            cargs.append(a.data_ptr())
        else:
            cargs.append(a)
    ret = fn(*cargs)
    status = _FUNCS['hidet_get_last_error']()
    if status is not None:
        raise BackendException('Calling {} with arguments ({}) failed. error:\n{}\nFunction @ {}'.format(
            name, ', '.join(_describe(a) for a in args), status.decode('utf-8'), LIB_PATH))
    return ret


def require_gpu(*tensors: torch.Tensor):
    """Every operand must live on one GPU; there is no CPU path."""
    dev = None
    for t in tensors:
        if not t.is_cuda:
            raise BackendException('tensor operand is on {}: the quantized-matmul kernels run on the GPU only '
                                   '(no CPU fallback)'.format(t.device))
        if dev is not None and t.device != dev:
            raise BackendException('operands are on different devices: {} and {}'.format(dev, t.device))
        dev = t.device


_RAW_STREAM = getattr(torch._C, '_cuda_getCurrentRawStream', None)


def current_stream(device: torch.device) -> int:
    """Handle (hipStream_t as an integer) of torch's current stream on `device`."""
    if _RAW_STREAM is not None:  # the same value as torch.cuda.current_stream(device).cuda_stream, without building a Stream object
        return _RAW_STREAM(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


_WORKSPACES: Dict[Tuple[int, int], torch.Tensor] = {}


def workspace(device: torch.device, nbytes: int = 0) -> torch.Tensor:
    """Zero-initialised scratch buffer for (device, current stream); grows, never shrinks.

    Stands in for the reference's grow-only request_hip_workspace (src/hidet/runtime/hip/context.cpp:43-57).
    One buffer per stream, because two calls that overlap in time must not share it.
    """
    key = (device.index if device.index is not None else torch.cuda.current_device(), current_stream(device))
    ws = _WORKSPACES.get(key)
    if ws is None or ws.numel() < nbytes:
        need = max(int(nbytes), int(load_library().hidet_qmm_min_workspace_bytes()))
        ws = torch.zeros(need, dtype=torch.uint8, device=device)
        _WORKSPACES[key] = ws
    return ws
