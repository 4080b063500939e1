"""matmul_f8 / matmul_f8_scaled with the reference's signatures and checks
(python/hidet/graph/ops/matmul/matmul_f8.py:132-175, 357-454, 644-775), executed by `hidet_matmul_f8` and
`hidet_matmul_f8_scaled`, plus the per-tensor quantize / matmul pair of the benchmark configuration.

A is [..., M, K] and B is [..., N, K], both K-major, both float8_e4m3 or both float8_e5m2 (OCP formats, the MFMA's
fp8 and bf8 operand types).  The e4m3 path has the tuned kernels; e5m2 runs the unscaled matmul on plainer ones and
the block-scaled matmul on the same kernels as e4m3 (`hidet_matmul_f8_scaled_e5m2`)."""
from typing import List, Optional, Tuple

import torch

from hidet_amd import ffi
from hidet_amd.graph.operator import Operator, Task, TensorSpec, data_type, input_like, DTYPE_NAMES

f8e4m3 = torch.float8_e4m3fn
f8e5m2 = torch.float8_e5m2
_OUT_TYPES = (torch.float32, torch.float16, torch.bfloat16, f8e4m3, f8e5m2)


def _broadcast_heads(a_head, b_head) -> Tuple[int, ...]:
    try:
        return tuple(torch.broadcast_shapes(tuple(a_head), tuple(b_head)))
    except RuntimeError:
        raise ValueError('Matrix multiplication expects tensor A and B with compatible broadcast shapes')


class MatmulF8Task(Task):
    """w8a8 matmul task: A is (M, K) K-major, B is (N, K) K-major, C is (M, N) N-major."""

    def __init__(self, a: TensorSpec, b: TensorSpec, acc_dtype: torch.dtype, output_dtype: torch.dtype):
        assert a.dtype == b.dtype
        self._assert(a.shape[-1] == b.shape[-1],
                     'Expected A and B with shapes [...,M,K] and [...,N,K], got {} and {}'.format(list(a.shape), list(b.shape)))
        head = _broadcast_heads(a.shape[:-2], b.shape[:-2])
        acc, ad = DTYPE_NAMES[acc_dtype], a.dtype
        super().__init__(name='matmul_{}.{}.{}.{}'.format(acc, ad, ad, acc), inputs=[a, b],
                         outputs=[TensorSpec('c', DTYPE_NAMES[output_dtype], head + (a.shape[-2], b.shape[-2]))],
                         attrs={'acc_dtype': acc_dtype, 'output_dtype': output_dtype})


class MatmulF8ScaledTask(Task):
    """w8a8 block-scaled matmul task: scale_a is (K/128, M) M-major, scale_b is (N/128, K/128)."""

    def __init__(self, a: TensorSpec, b: TensorSpec, scale_a: TensorSpec, scale_b: TensorSpec, acc_dtype: torch.dtype,
                 output_dtype: torch.dtype):
        self._assert(a.dtype == b.dtype)
        self._assert(a.shape[-1] == b.shape[-1],
                     'Expected A and B with shapes [...,M,K] and [...,N,K], got {} and {}'.format(list(a.shape), list(b.shape)))
        head = _broadcast_heads(a.shape[:-2], b.shape[:-2])
        self._assert(len(scale_a.shape) >= 2 and len(scale_b.shape) >= 2 and scale_a.shape[-2] == scale_b.shape[-1],
                     'Incompatible shapes for scale_a and scale_b')
        self._assert(tuple(scale_a.shape[:-2]) == tuple(a.shape[:-2]) and tuple(scale_b.shape[:-2]) == tuple(b.shape[:-2]),
                     'Incompatible shapes for scale_a and scale_b')
        m, n, k = a.shape[-2], b.shape[-2], a.shape[-1]
        self.group_MNK = (m // max(scale_a.shape[-1], 1), n // max(scale_b.shape[-2], 1), k // max(scale_a.shape[-2], 1))
        acc, ad = DTYPE_NAMES[acc_dtype], a.dtype
        super().__init__(name='scaled_mm_{}.{}.{}.{}'.format(acc, ad, ad, acc), inputs=[a, b, scale_a, scale_b],
                         outputs=[TensorSpec('c', DTYPE_NAMES[output_dtype], head + (m, n))],
                         attrs={'acc_dtype': acc_dtype, 'output_dtype': output_dtype})


def _rows(x: torch.Tensor) -> torch.Tensor:
    """2-D operand the kernels can address as base + row * stride + column: the last axis contiguous and, with more
    than one row, a row stride of at least the row length. Anything else (a transposed view, a row expanded with
    stride 0, overlapping rows) is copied; rows that are merely strided are passed as they are."""
    rows, cols = x.shape
    if (cols > 1 and x.stride(1) != 1) or (rows > 1 and x.stride(0) < cols):
        x = x.contiguous()
    return x


def _row_stride(x: torch.Tensor) -> int:
    return x.stride(0) if x.shape[0] > 1 else x.shape[1]


def _launch_f8(a2: torch.Tensor, b2: torch.Tensor, c2: torch.Tensor, scale_a, scale_b):
    m, k = a2.shape
    n = b2.shape[0]
    if a2.dtype == f8e5m2:  # the bf8 format of the MFMA, on the plainer kernels (no workspace)
        ffi.call('hidet_matmul_f8_e5m2', a2, b2, c2, m, n, k, _row_stride(a2), _row_stride(b2), ffi.DTYPE_CODE[c2.dtype],
                 scale_a, scale_b, ffi.current_stream(a2.device))
        return
    ws = ffi.workspace(a2.device)
    ffi.call('hidet_matmul_f8', a2, b2, c2, m, n, k, _row_stride(a2), _row_stride(b2), ffi.DTYPE_CODE[c2.dtype], scale_a, scale_b,
             ws, ws.numel(), ffi.current_stream(a2.device))


def _run_f8(a: torch.Tensor, b: torch.Tensor, output_dtype: torch.dtype, scale_a=None, scale_b=None) -> torch.Tensor:
    ffi.require_gpu(a, b)
    m, k = a.shape[-2], a.shape[-1]
    n = b.shape[-2]
    if b.dim() == 2:  # fold the batch axes of a into M
        a2 = _rows(a.reshape(-1, k))
        c = torch.empty((a2.shape[0], n), dtype=output_dtype, device=a.device)
        _launch_f8(a2, _rows(b), c, scale_a, scale_b)
        return c.reshape(tuple(a.shape[:-1]) + (n,))
    head = _broadcast_heads(a.shape[:-2], b.shape[:-2])
    ae = a.expand(head + (m, k)).reshape((-1, m, k))
    be = b.expand(head + (n, k)).reshape((-1, n, k))
    c = torch.empty((ae.shape[0], m, n), dtype=output_dtype, device=a.device)
    for i in range(ae.shape[0]):
        _launch_f8(_rows(ae[i]), _rows(be[i]), c[i], scale_a, scale_b)
    return c.reshape(head + (m, n))


class MatmulF8Operator(Operator):
    def __init__(self, a: torch.Tensor, b: torch.Tensor, acc_dtype: torch.dtype, output_dtype: torch.dtype):
        super().__init__(inputs=[a, b], attributes={'acc_dtype': acc_dtype, 'output_dtype': output_dtype},
                         task=MatmulF8Task(input_like(a, 'a'), input_like(b, 'b'), acc_dtype, output_dtype))

    def run(self) -> List[torch.Tensor]:
        a, b = self.inputs
        return [_run_f8(a, b, self.attrs['output_dtype'])]


class MatmulF8ScaledOperator(Operator):
    def __init__(self, a, b, scale_a, scale_b, acc_dtype: torch.dtype, output_dtype: torch.dtype, bias: Optional[torch.Tensor] = None):
        if bias is not None:
            raise ValueError('bias is not supported for scaled matmul f8')
        super().__init__(
            inputs=[a, b, scale_a, scale_b], attributes={'acc_dtype': acc_dtype, 'output_dtype': output_dtype},
            task=MatmulF8ScaledTask(input_like(a, 'a'), input_like(b, 'b'), input_like(scale_a, 'scale_a'),
                                    input_like(scale_b, 'scale_b'), acc_dtype, output_dtype))

    def run(self) -> List[torch.Tensor]:
        a, b, scale_a, scale_b = self.inputs
        ffi.require_gpu(a, b, scale_a, scale_b)
        gm, gn, gk = self.task.group_MNK
        if (gm, gn, gk) != (1, 128, 128):
            # the reference supports exactly this configuration too (matmul_f8.py:478-480)
            raise ValueError('only per-token (group_M = 1) x 128 x 128 block scaling is supported, got groups {}'.format((gm, gn, gk)))
        if scale_a.dtype != torch.float32 or scale_b.dtype != torch.float32:
            raise ValueError('scale_a and scale_b must be float32')
        out = self.attrs['output_dtype']
        a3, b3, sa3, sb3, head = scaled_operands(a, b, scale_a, scale_b)
        m, k = a3.shape[-2], a3.shape[-1]
        n = b3.shape[-2]
        c = torch.empty((a3.shape[0], m, n), dtype=out, device=a.device)
        ws = ffi.workspace(a.device)
        for i in range(a3.shape[0]):
            ffi.call('hidet_matmul_f8_scaled_e5m2' if a.dtype == f8e5m2 else 'hidet_matmul_f8_scaled', a3[i], b3[i], sa3[i], sb3[i],
                     c[i], m, n, k, ffi.DTYPE_CODE[out],
                     ws, ws.numel(), ffi.current_stream(a.device))
        return [c.reshape(head + (a.shape[-2], n))]


def scaled_operands(a, b, scale_a, scale_b):
    """Operands of the block-scaled matmul as dense 3-D tensors with one common batch axis, plus the head shape of the
    result. The task accepts any mutually broadcastable heads (matmul_f8.py:372-376 of the reference): with a 2-D b
    the batch axes of a are folded into M - scale_a [..., K/128, M] becomes [K/128, B * M] - and one launch serves
    the whole batch; otherwise the heads are broadcast against each other."""
    m, k = a.shape[-2], a.shape[-1]
    n = b.shape[-2]
    if b.dim() == 2 and a.dim() > 2:
        head = tuple(a.shape[:-2])
        a3 = a.reshape((1, -1, k)).contiguous()
        kb = scale_a.shape[-2]
        sa3 = scale_a.reshape((-1, kb, m)).permute(1, 0, 2).reshape((1, kb, -1)).contiguous()
        return a3, b.reshape((1, n, k)).contiguous(), sa3, scale_b.reshape((1,) + tuple(scale_b.shape)).contiguous(), head
    head = _broadcast_heads(a.shape[:-2], b.shape[:-2])
    a3 = a.expand(head + (m, k)).reshape((-1, m, k)).contiguous()
    b3 = b.expand(head + (n, k)).reshape((-1, n, k)).contiguous()
    sa3 = scale_a.expand(head + tuple(scale_a.shape[-2:])).reshape((-1,) + tuple(scale_a.shape[-2:])).contiguous()
    sb3 = scale_b.expand(head + tuple(scale_b.shape[-2:])).reshape((-1,) + tuple(scale_b.shape[-2:])).contiguous()
    return a3, b3, sa3, sb3, head


_VALIDATED = {}  # operand signature of an unscaled call that passed every check -> its output dtype


def _matmul_f8(a, b, is_scaled: bool, scale_a=None, scale_b=None, bias=None, acc_dtype='float32', output_dtype=None):
    if not is_scaled:  # checked before: skip building the operator and task records (host time of a decode call)
        out = _VALIDATED.get((a.shape, a.dtype, b.shape, b.dtype, acc_dtype, output_dtype))
        if out is not None:
            return _run_f8(a, b, out)
    if len(a.shape) < 2 or len(b.shape) < 2:
        raise ValueError('a and b must have at least 2 dimensions, got shape {} and {}'.format(list(a.shape), list(b.shape)))
    if (a.dtype != f8e4m3 or b.dtype != f8e4m3) and (a.dtype != f8e5m2 or b.dtype != f8e5m2):
        raise ValueError('matmul_f8 only supports both operands being f8e4m3 or f8e5m2, got {} and {}'.format(a.dtype, b.dtype))
    signature = (a.shape, a.dtype, b.shape, b.dtype, acc_dtype, output_dtype)  # as the caller passed them
    if output_dtype is None:
        output_dtype = a.dtype
    acc_dtype, output_dtype = data_type(acc_dtype), data_type(output_dtype)
    if acc_dtype != torch.float32:
        raise ValueError('matmul_f8 accumulates in float32 only, got acc_dtype {}'.format(acc_dtype))
    if output_dtype not in _OUT_TYPES or (output_dtype in (f8e4m3, f8e5m2) and output_dtype != a.dtype):
        raise ValueError('unsupported output dtype {} for operands of {}'.format(output_dtype, a.dtype))
    if is_scaled:
        return MatmulF8ScaledOperator(a, b, scale_a, scale_b, acc_dtype, output_dtype, bias).outputs[0]
    c = MatmulF8Operator(a, b, acc_dtype, output_dtype).outputs[0]
    _VALIDATED[signature] = output_dtype
    return c


def matmul_f8(a: torch.Tensor, b: torch.Tensor, acc_dtype='float32', output_dtype=None) -> torch.Tensor:
    """Matrix multiplication for f8e4m3: a (..., M, K) K-major, b (..., N, K) K-major; the output dtype
    defaults to the dtype of a and b."""
    return _matmul_f8(a, b, False, acc_dtype=acc_dtype, output_dtype=output_dtype)


def matmul_f8_scaled(a, b, scale_a, scale_b, bias=None, acc_dtype='float32', output_dtype=None) -> torch.Tensor:
    """Block-scaled matrix multiplication for f8e4m3: scale_a (K/128, M), scale_b (N/128, K/128), float32."""
    return _matmul_f8(a, b, True, scale_a, scale_b, bias, acc_dtype, output_dtype)


# ---- per-tensor scaling (benchmark configuration; the reference has only the unscaled and the block-scaled task)

def fp8_quantize_per_tensor(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(codes float8_e4m3 of x.shape, scale float32 [1]) with scale = max|x| / 448 and codes = e4m3(x / scale)."""
    ffi.require_gpu(x)
    if x.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise ValueError('fp8_quantize_per_tensor expects float32, float16 or bfloat16, got {}'.format(x.dtype))
    x = x.contiguous()
    codes = torch.empty(x.shape, dtype=f8e4m3, device=x.device)
    scale = torch.empty(1, dtype=torch.float32, device=x.device)
    ws = ffi.workspace(x.device)
    ffi.call('hidet_fp8_quantize_per_tensor', x, codes, scale, x.numel(), ffi.DTYPE_CODE[x.dtype], ws, ws.numel(),
             ffi.current_stream(x.device))
    return codes, scale


def matmul_f8_per_tensor(a: torch.Tensor, b: torch.Tensor, scale_a: torch.Tensor, scale_b: torch.Tensor,
                         output_dtype='bfloat16') -> torch.Tensor:
    """cast((a @ b^T) * (scale_a * scale_b)) with fp32 accumulation; the scales are float32 tensors of one
    element on the GPU (as returned by fp8_quantize_per_tensor)."""
    if a.dtype != f8e4m3 or b.dtype != f8e4m3:
        raise ValueError('matmul_f8 only supports both operands being f8e4m3 or f8e5m2, got {} and {}'.format(a.dtype, b.dtype))
    if len(a.shape) < 2 or len(b.shape) < 2:
        raise ValueError('a and b must have at least 2 dimensions, got shape {} and {}'.format(list(a.shape), list(b.shape)))
    if a.shape[-1] != b.shape[-1]:
        raise ValueError('Expected A and B with shapes [...,M,K] and [...,N,K], got {} and {}'.format(list(a.shape), list(b.shape)))
    for s in (scale_a, scale_b):
        if s.dtype != torch.float32 or s.numel() != 1:
            raise ValueError('per-tensor scales must be float32 tensors with one element')
    ffi.require_gpu(scale_a, scale_b)
    return _run_f8(a, b, data_type(output_dtype), scale_a, scale_b)
