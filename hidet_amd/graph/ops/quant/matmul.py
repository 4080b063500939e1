"""symmetric_quant_matmul with the reference's signature, checks and error texts
(python/hidet/graph/ops/quant/matmul.py:24-93), executed by `hidet_symmetric_quant_matmul_f16_i8`."""
from typing import List, Optional

import torch

from torch.utils.weak import WeakTensorKeyDictionary

from hidet_amd import ffi, option
from hidet_amd.graph.operator import Operator, Task, TensorSpec, input_like


def _check_task_operands(task: Task, a: TensorSpec, weight: TensorSpec, scale: TensorSpec):
    task._assert(a.dtype == 'float16' and weight.dtype == 'int8', 'Expect a to be float16 and weight to be int8')
    if len(a.shape) < 2 or len(weight.shape) != 2:
        raise ValueError('SymmetricQuantizedMatmul expect , got {} and {}'.format(list(a.shape), list(weight.shape)))
    task._assert(len(scale.shape) >= 1 and scale.shape[0] == weight.shape[1])
    task._assert(
        a.shape[-1] == weight.shape[-2],
        'Matrix multiplication expect tensor A and B with shape [..., M, K] and [..., K, N]'
        ', got {} and {}'.format(list(a.shape), list(weight.shape)),
    )


def check_matmul_args(a: torch.Tensor, weight: torch.Tensor):
    """The argument checks shared by every W8A16 entry (python/hidet/graph/ops/quant/matmul.py:83-92)."""
    if len(a.shape) < 2 or len(weight.shape) < 2:
        raise ValueError('a and b must have at least 2 dimensions, got shape {} and {}'.format(list(a.shape), list(weight.shape)))
    if a.shape[-1] % 2 != 0 or weight.shape[-1] % 2 != 0:
        raise ValueError('Expect the last dimension of the input tensors to be a multiple of 2')
    if a.dtype != torch.float16 or weight.dtype != torch.int8:
        raise ValueError('BatchMatmulF16Op only support float16, int8, got {} and {}'.format(a.dtype, weight.dtype))


class SymmetricQuantizedMatmulTask(Task):
    def __init__(self, a: TensorSpec, weight: TensorSpec, scale: TensorSpec):
        _check_task_operands(self, a, weight, scale)
        c_shape = tuple(a.shape[:-1]) + (weight.shape[-1],)
        super().__init__(name='symmetric_quantized_matmul', inputs=[a, weight, scale],
                         outputs=[TensorSpec('c', 'float16', c_shape)], attrs={})


_NK_MAX_ROWS = 16  # one pass of the bandwidth-bound kernels for K-contiguous weights; more rows go to the MFMA GEMM
# The GEMM that reads K-contiguous weights gathers 8 bytes per lane from 16 rows of the stored matrix per load and runs
# about a third slower than the row-major one at prefill sizes (2048 x 4096 x 11008: 214 against 157 us; 64 rows: 25 against
# 20 us).  Batched decode (17 to 64 rows) uses it, so a model that only decodes never makes a second copy of its weights;
# longer prompts use the row-major copy.
_NK_GEMM_MAX_ROWS = 64


def to_decode_layout(wq: torch.Tensor) -> torch.Tensor:
    """The same [K, N] int8 weight, stored K-contiguous (a view with strides (1, K) of a fresh [N, K] tensor).

    `symmetric_quant_matmul` on such a weight with up to 16 activation rows runs the kernel that
    reduces along the contiguous axis (no exchange between workgroups), with up to 64 the MFMA GEMM that reads this layout;
    it is what `nn.Linear` stores, so `linear.weight` quantized with `dims=1` and viewed with `.t()` is already in this
    layout.  A call with more rows makes a row-major copy of the weight the first time and keeps it for as long as the
    weight tensor lives.
    """
    if wq.dim() != 2:
        raise ValueError('expected a 2-D weight, got shape {}'.format(list(wq.shape)))
    return wq.t().contiguous().t()


_ROW_MAJOR_COPIES = WeakTensorKeyDictionary()  # K-contiguous weight tensor (by identity) -> its row-major copy


def _row_major(weight: torch.Tensor) -> torch.Tensor:
    """`weight` as the row-major [K, N] tensor the GEMM and the N-contiguous GEMV read.  The copy of a K-contiguous weight
    (45 MB for a 4096 x 11008 layer) is made once per tensor object and lives as long as that object does; it is made again
    when the weight has been written in place since (torch's version counter)."""
    if weight.is_contiguous():
        return weight
    if weight.dim() == 2 and weight.stride(0) == 1:
        entry = _ROW_MAJOR_COPIES.get(weight)
        if entry is None or entry[0] != weight._version or entry[1].device != weight.device:
            entry = _ROW_MAJOR_COPIES[weight] = (weight._version, weight.contiguous())
        return entry[1]
    return weight.contiguous()


def _check_bias(bias: torch.Tensor, n: int) -> torch.Tensor:
    if bias.dtype != torch.float16 or bias.dim() != 1 or bias.shape[0] != n:
        raise ValueError('bias must be a float16 vector of {} elements, got {} {}'.format(n, bias.dtype, list(bias.shape)))
    return bias.contiguous()


def run_w8a16(a: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor, parallel_k_parts: int = 0,
              bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """c[..., M, N] on the GPU.  Leading axes of `a` are folded into M: the weight is 2-D, so broadcasting
    over them is the same as one tall matmul.  `bias` (float16 [N]) is added in the kernel's epilogue."""
    ffi.require_gpu(a, weight, scale)
    k, n = weight.shape
    if bias is not None:
        ffi.require_gpu(bias)
        bias = _check_bias(bias, n)
    a2 = a.reshape(-1, k)
    if a2.stride(-1) != 1 or (a2.shape[0] > 1 and a2.stride(0) < k):
        a2 = a2.contiguous()
    m = a2.shape[0]
    lda = a2.stride(0) if m > 1 else k
    scale = scale.contiguous()
    c = torch.empty((m, n), dtype=torch.float16, device=a.device)
    # A [K, N] weight held K-contiguous (strides (1, ldw): `wq_nk.t()` of an [N, K] tensor, see `to_decode_layout`) goes to
    # the entry point for that layout: the bandwidth-bound kernels up to 16 rows, the MFMA GEMM reading the same layout up
    # to 64 (K a multiple of 64, N of 4).  What neither takes uses a row-major copy, as any non-contiguous operand does.
    if (k > 1 and n > 1 and weight.stride(0) == 1 and weight.stride(1) >= k and weight.stride(1) % 16 == 0
            and k % 16 == 0 and weight.data_ptr() % 16 == 0
            and (m <= _NK_MAX_ROWS or (m <= _NK_GEMM_MAX_ROWS and k % 64 == 0 and n % 4 == 0 and lda % 8 == 0 and a2.data_ptr() % 16 == 0
                                       and (n - 1) * weight.stride(1) + k < (1 << 31) - (1 << 20)
                                       and (m * lda + k) * 2 < (1 << 31) - (1 << 20)))):
        ws = ffi.workspace(a.device)
        if bias is None:
            ffi.call('hidet_symmetric_quant_matmul_f16_i8_nk', a2, weight, scale, c, m, k, n, lda, weight.stride(1), ws, ws.numel(),
                     ffi.current_stream(a.device))
        else:
            ffi.call('hidet_symmetric_quant_matmul_f16_i8_nk_bias', a2, weight, scale, bias, c, m, k, n, lda, weight.stride(1), ws,
                     ws.numel(), ffi.current_stream(a.device))
        return c.reshape(tuple(a.shape[:-1]) + (n,))
    weight = _row_major(weight)
    ws = ffi.workspace(a.device)
    if bias is None:
        ffi.call('hidet_symmetric_quant_matmul_f16_i8', a2, weight, scale, c, m, k, n, lda, int(parallel_k_parts), ws,
                 ws.numel(), ffi.current_stream(a.device))
    else:
        ffi.call('hidet_symmetric_quant_matmul_f16_i8_bias', a2, weight, scale, bias, c, m, k, n, lda, int(parallel_k_parts), ws,
                 ws.numel(), ffi.current_stream(a.device))
    return c.reshape(tuple(a.shape[:-1]) + (n,))


class SymmetricQuantizedMatmulOp(Operator):
    def __init__(self, a: torch.Tensor, b: torch.Tensor, scale: torch.Tensor, bias: Optional[torch.Tensor] = None):
        task = SymmetricQuantizedMatmulTask(input_like(a, 'a'), input_like(b, 'b'), input_like(scale, 'scale'))
        if bias is not None:
            _check_bias(bias, b.shape[1])
        self.bias = bias
        super().__init__(inputs=[a, b, scale], attributes={}, task=task)

    def run(self) -> List[torch.Tensor]:
        from .resolve import resolve_parallel_k_parts

        a, b, scale = self.inputs
        parts = resolve_parallel_k_parts(option.get_parallel_k(), a, b)
        return [run_w8a16(a, b, scale, parts, self.bias)]


# Operand signatures (shapes and dtypes) that have passed every check once.  A decode loop calls the operator with the same
# signature for every token and layer, and building the operator and task records again costs about as much host time as
# the kernel runs (a 4096 x 11008 GEMV: 11 to 14 us); the device checks and the launch are done on every call.
_VALIDATED = set()


def symmetric_quant_matmul(a: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor,
                           bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The reference's operator (python/hidet/graph/ops/quant/matmul.py:83-93).  `bias`, which the reference's signature
    does not have, is the fused form of the epilogue its template admits (matmul_f16_i8.py:95-99): a float16 [N] vector
    added to the float16 result (two roundings, as the reference's fused epilogue and the matmul followed by an add
    give): fused and unfused calls return the same bits."""
    signature = (a.shape, a.dtype, weight.shape, weight.dtype, scale.shape, scale.dtype,
                 None if bias is None else (bias.shape, bias.dtype))
    if signature in _VALIDATED:
        from .resolve import resolve_parallel_k_parts

        return run_w8a16(a, weight, scale, resolve_parallel_k_parts(option.get_parallel_k(), a, weight), bias)
    check_matmul_args(a, weight)
    out = SymmetricQuantizedMatmulOp(a, weight, scale, bias).outputs[0]
    _VALIDATED.add(signature)
    return out
