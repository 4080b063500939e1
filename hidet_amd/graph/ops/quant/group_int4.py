"""Group-wise symmetric int4 weights (W4A16).  The reference has no operator for this; the conventions are
the reference's own: signed int4 with max 7 (python/hidet/ir/dtypes/integer_subbyte.py:49), two codes per
byte along the innermost axis, low nibble first (python/hidet/transforms/lower_integer_subbyte.py:103-113),
scales shaped [K / group, N] (tests/cute_kernel/quantized_linear.py:692-699)."""
from typing import List, Optional, Tuple

import torch

from hidet_amd import ffi
from hidet_amd.graph.operator import Operator, Task, TensorSpec, data_type, input_like, DTYPE_NAMES


class SymmetricGroupQuantizationInt4Task(Task):
    def __init__(self, w: TensorSpec, group_size: int, scale_dtype: torch.dtype):
        self._assert(len(w.shape) == 2, 'expect a 2-D weight [K, N], got {}'.format(list(w.shape)))
        k, n = w.shape
        self._assert(group_size > 0 and k % group_size == 0, 'K ({}) must be a multiple of the group size ({})'.format(k, group_size))
        self._assert(n % 2 == 0, 'N ({}) must be even: two codes are packed per byte'.format(n))
        super().__init__(
            name='symmetric_group_quantization_int4',
            inputs=[w],
            outputs=[TensorSpec('packed', 'uint8', (k, n // 2)), TensorSpec('scaling', DTYPE_NAMES[scale_dtype], (k // group_size, n))],
            attrs={'group_size': group_size, 'scale_dtype': scale_dtype},
        )


class SymmetricGroupQuantizationInt4Op(Operator):
    def __init__(self, w: torch.Tensor, group_size: int, scale_dtype: torch.dtype):
        super().__init__(inputs=[w], attributes={'group_size': group_size, 'scale_dtype': scale_dtype},
                         task=SymmetricGroupQuantizationInt4Task(input_like(w, 'w'), group_size, scale_dtype))

    def run(self) -> List[torch.Tensor]:
        (w,) = self.inputs
        ffi.require_gpu(w)
        group_size, scale_dtype = self.attrs['group_size'], self.attrs['scale_dtype']
        k, n = w.shape
        w = w.contiguous()
        packed = torch.empty((k, n // 2), dtype=torch.uint8, device=w.device)
        scales = torch.empty((k // group_size, n), dtype=scale_dtype, device=w.device)
        ffi.call('hidet_group_quantize_int4', w, packed, scales, k, n, group_size, ffi.DTYPE_CODE[w.dtype],
                 ffi.DTYPE_CODE[scale_dtype], ffi.current_stream(w.device))
        return [packed, scales]


def symmetric_group_quantize_int4(w: torch.Tensor, group_size: int = 128, scale_dtype='bfloat16') -> Tuple[torch.Tensor, torch.Tensor]:
    """w float32 [K, N] -> (packed uint8 [K, N/2], scales [K/group, N]); scale = amax / 7 per (group, column)."""
    scale_dtype = data_type(scale_dtype)
    if w.dtype != torch.float32:
        raise ValueError('symmetric_group_quantize_int4 expects float32 weights, got {}'.format(w.dtype))
    if scale_dtype not in (torch.bfloat16, torch.float16):
        raise ValueError('scale dtype must be bfloat16 or float16, got {}'.format(scale_dtype))
    op = SymmetricGroupQuantizationInt4Op(w, group_size, scale_dtype)
    return op.outputs[0], op.outputs[1]


class SymmetricQuantizedMatmulW4A16Task(Task):
    def __init__(self, a: TensorSpec, packed: TensorSpec, scales: TensorSpec, group_size: int):
        self._assert(a.dtype in ('bfloat16', 'float16') and packed.dtype == 'uint8' and scales.dtype == a.dtype,
                     'Expect a and scales to be bfloat16 or float16 (same type) and the packed weight to be uint8')
        if len(a.shape) < 2 or len(packed.shape) != 2 or len(scales.shape) != 2:
            raise ValueError('SymmetricQuantizedMatmulW4A16 expect a[..., M, K], packed[K, N/2], scales[K/g, N], got {}, {} and {}'.format(
                list(a.shape), list(packed.shape), list(scales.shape)))
        k, n = packed.shape[0], packed.shape[1] * 2
        self._assert(a.shape[-1] == k, 'Matrix multiplication expect tensor A and B with shape [..., M, K] and [..., K, N]'
                                       ', got {} and {}'.format(list(a.shape), [k, n]))
        self._assert(k % group_size == 0 and tuple(scales.shape) == (k // group_size, n),
                     'scales must be [K / group, N] = {}, got {}'.format([k // max(group_size, 1), n], list(scales.shape)))
        super().__init__(name='symmetric_quantized_matmul_w4a16', inputs=[a, packed, scales],
                         outputs=[TensorSpec('c', a.dtype, tuple(a.shape[:-1]) + (n,))], attrs={'group_size': group_size})


def _check_bias(bias: torch.Tensor, n: int, dtype: torch.dtype) -> torch.Tensor:
    if bias.dtype != dtype or bias.dim() != 1 or bias.shape[0] != n:
        raise ValueError('bias must be a {} vector of {} elements, got {} {}'.format(dtype, n, bias.dtype, list(bias.shape)))
    return bias.contiguous()


class SymmetricQuantizedMatmulW4A16Op(Operator):
    def __init__(self, a: torch.Tensor, packed: torch.Tensor, scales: torch.Tensor, group_size: int, bias: Optional[torch.Tensor] = None):
        task = SymmetricQuantizedMatmulW4A16Task(input_like(a, 'a'), input_like(packed, 'b'), input_like(scales, 'scale'), group_size)
        if bias is not None:
            _check_bias(bias, packed.shape[1] * 2, a.dtype)
        self.bias = bias
        super().__init__(inputs=[a, packed, scales], attributes={'group_size': group_size}, task=task)

    def run(self) -> List[torch.Tensor]:
        a, packed, scales = self.inputs
        return [_run_w4a16(a, packed, scales, self.attrs['group_size'], self.bias)]


_VALIDATED = set()  # operand signatures that have passed the task's checks once


def _run_w4a16(a: torch.Tensor, packed: torch.Tensor, scales: torch.Tensor, group_size: int,
               bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    ffi.require_gpu(a, packed, scales)
    k, n = packed.shape[0], packed.shape[1] * 2
    if bias is not None:
        ffi.require_gpu(bias)
        bias = _check_bias(bias, n, a.dtype)
    a2 = a.reshape(-1, k)
    if a2.stride(-1) != 1 or (a2.shape[0] > 1 and a2.stride(0) < k):
        a2 = a2.contiguous()
    m = a2.shape[0]
    lda = a2.stride(0) if m > 1 else k
    c = torch.empty((m, n), dtype=a.dtype, device=a.device)
    ws = ffi.workspace(a.device)
    if bias is None:
        ffi.call('hidet_symmetric_quant_matmul_w4a16', a2, packed.contiguous(), scales.contiguous(), c, m, k, n, lda,
                 group_size, ffi.DTYPE_CODE[a.dtype], 0, ws, ws.numel(), ffi.current_stream(a.device))
    else:
        ffi.call('hidet_symmetric_quant_matmul_w4a16_bias', a2, packed.contiguous(), scales.contiguous(), bias, c, m, k, n, lda,
                 group_size, ffi.DTYPE_CODE[a.dtype], 0, ws, ws.numel(), ffi.current_stream(a.device))
    return c.reshape(tuple(a.shape[:-1]) + (n,))


def symmetric_quant_matmul_w4a16(a: torch.Tensor, packed: torch.Tensor, scales: torch.Tensor, group_size: int = 128,
                                 bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """c[..., M, N] = a @ dequant(packed, scales) with fp32 accumulation; a, scales and c share bfloat16 or float16.
    `bias` ([N], the same type) is added to the rounded result: the bits of the matmul followed by an add, as for the int8
    operator."""
    signature = (a.shape, a.dtype, packed.shape, packed.dtype, scales.shape, scales.dtype, group_size,
                 None if bias is None else (bias.shape, bias.dtype))
    if signature in _VALIDATED:  # checked before: skip building the operator and task records (host time of a decode call)
        return _run_w4a16(a, packed, scales, group_size, bias)
    if len(a.shape) < 2 or len(packed.shape) < 2:
        raise ValueError('a and b must have at least 2 dimensions, got shape {} and {}'.format(list(a.shape), list(packed.shape)))
    out = SymmetricQuantizedMatmulW4A16Op(a, packed, scales, group_size, bias).outputs[0]
    _VALIDATED.add(signature)
    return out


def to_decode_layout_int4(packed: torch.Tensor) -> torch.Tensor:
    """Repack `packed` uint8 [K, N/2] (two codes per byte along N, low nibble first) as uint8 [N, K/2] for the decode kernel.

    Row n of the result holds the K codes of output column n; inside every 4 bytes (8 consecutive k) nibble i is code
    k = 2i for i < 4 and code k = 2(i - 4) + 1 for i >= 4, so that a shift and a mask give the kernel a (k, k + 1) pair
    ready for the matrix instruction. K must be a multiple of 8 (the kernel itself wants 128).
    """
    if packed.dim() != 2 or packed.dtype != torch.uint8:
        raise ValueError('expected a packed uint8 weight [K, N/2], got {} {}'.format(packed.dtype, list(packed.shape)))
    k, n = packed.shape[0], packed.shape[1] * 2
    if k % 8 != 0:
        raise ValueError('K ({}) must be a multiple of 8'.format(k))
    codes = torch.stack((packed & 0xF, packed >> 4), dim=-1).reshape(k, n)   # nibble of q[k, n]
    pairs = codes.t().reshape(n, k // 8, 4, 2)                                # [n, word, i, parity]: code k = 2i + parity
    even, odd = pairs[..., 0], pairs[..., 1]
    out = torch.stack((even[..., 0] | (even[..., 1] << 4), even[..., 2] | (even[..., 3] << 4),
                       odd[..., 0] | (odd[..., 1] << 4), odd[..., 2] | (odd[..., 3] << 4)), dim=-1)
    return out.reshape(n, k // 2).contiguous()


def symmetric_quant_matmul_w4a16_decode(a: torch.Tensor, packed_nk: torch.Tensor, scales: torch.Tensor,
                                        group_size: int = 128) -> torch.Tensor:
    """`symmetric_quant_matmul_w4a16` on a weight repacked with `to_decode_layout_int4` ([N, K/2]); `scales` stay
    [K/group, N]. For decode: up to 16 rows of `a` per pass over the weights. K a multiple of 128, group size 128 times
    a power of two."""
    if len(a.shape) < 2 or len(packed_nk.shape) != 2 or len(scales.shape) != 2:
        raise ValueError('expect a[..., M, K], packed_nk[N, K/2], scales[K/g, N], got {}, {} and {}'.format(
            list(a.shape), list(packed_nk.shape), list(scales.shape)))
    if a.dtype not in (torch.bfloat16, torch.float16) or scales.dtype != a.dtype or packed_nk.dtype != torch.uint8:
        raise ValueError('Expect a and scales to be bfloat16 or float16 (same type) and the packed weight to be uint8')
    n, k = packed_nk.shape[0], packed_nk.shape[1] * 2
    if a.shape[-1] != k:
        raise ValueError('Matrix multiplication expect tensor A and B with shape [..., M, K] and [..., K, N]'
                         ', got {} and {}'.format(list(a.shape), [k, n]))
    if group_size <= 0 or k % group_size != 0 or tuple(scales.shape) != (k // group_size, n):
        raise ValueError('scales must be [K / group, N] = {}, got {}'.format([k // max(group_size, 1), n], list(scales.shape)))
    ffi.require_gpu(a, packed_nk, scales)
    a2 = a.reshape(-1, k)
    if a2.stride(-1) != 1 or (a2.shape[0] > 1 and (a2.stride(0) < k or a2.stride(0) % 8 != 0)) or a2.data_ptr() % 16 != 0:
        a2 = a2.contiguous()
    m = a2.shape[0]
    lda = a2.stride(0) if m > 1 else k
    c = torch.empty((m, n), dtype=a.dtype, device=a.device)
    packed_nk = packed_nk.contiguous()
    ffi.call('hidet_symmetric_quant_matmul_w4a16_nk', a2, packed_nk, scales.contiguous(), c, m, k, n, lda, k // 2, group_size,
             ffi.DTYPE_CODE[a.dtype], ffi.current_stream(a.device))
    return c.reshape(tuple(a.shape[:-1]) + (n,))
