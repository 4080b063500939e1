"""symmetric_quant_matmul_f16_i8: the split-K form whose output keeps the K parts as a leading axis
(python/hidet/graph/ops/quant/matmul_f16_i8.py:30-93, 501-511); the caller sums over axis 0
(python/hidet/graph/ops/quant/resolve.py:99)."""
from typing import List

import torch

from hidet_amd.graph.operator import Operator, Task, TensorSpec, input_like
from .matmul import _check_task_operands, check_matmul_args, run_w8a16


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


class SymmetricQuantizedMatmulF16I8Task(Task):
    def __init__(self, a: TensorSpec, weight: TensorSpec, scale: TensorSpec, parallel_k_parts: int = 1):
        _check_task_operands(self, a, weight, scale)
        c_shape = (parallel_k_parts,) + tuple(a.shape[:-1]) + (weight.shape[-1],)
        super().__init__(name='symmetric_quantized_matmulf16', inputs=[a, weight, scale],
                         outputs=[TensorSpec('c', 'float16', c_shape)], attrs={'parallel_k_parts': parallel_k_parts})

    def allow_prologue(self) -> bool:
        return False

    def allow_epilogue(self) -> bool:
        # as in the reference (matmul_f16_i8.py:98-99). What the pre-built kernels can take into their epilogue is the bias
        # add of a linear layer (the rewrite rule SymmetricQuantizeMatmulBiasFused); any other consumer stays an operator
        # of its own
        return True


class SymmetricQuantizedMatmulF16I8Op(Operator):
    def __init__(self, a: torch.Tensor, b: torch.Tensor, scale: torch.Tensor, parallel_k_parts: int = 1):
        if not isinstance(parallel_k_parts, int) or parallel_k_parts < 1:
            raise ValueError('parallel_k_parts must be a positive integer, got {}'.format(parallel_k_parts))
        super().__init__(
            inputs=[a, b, scale],
            attributes={'parallel_k_parts': parallel_k_parts},
            task=SymmetricQuantizedMatmulF16I8Task(input_like(a, 'a'), input_like(b, 'b'), input_like(scale, 'scale'),
                                                   parallel_k_parts),
        )

    def run(self) -> List[torch.Tensor]:
        a, b, scale = self.inputs
        parts = self.attrs['parallel_k_parts']
        k, n = b.shape
        ext = _cdiv(k, parts)  # k_part_extent of the task definition (matmul_f16_i8.py:63)
        out = torch.zeros((parts,) + tuple(a.shape[:-1]) + (n,), dtype=torch.float16, device=a.device)
        for p in range(parts):
            lo, hi = min(p * ext, k), min((p + 1) * ext, k)
            if hi > lo:  # a K slice of `a` is a strided view: the kernel takes the row stride
                out[p] = run_w8a16(a[..., lo:hi], b[lo:hi], scale, 1)
        return [out]


def symmetric_quant_matmul_f16_i8(a: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor, parallel_k_parts=1) -> torch.Tensor:
    """Output [parallel_k_parts, ..., M, N]: part p sums k in [p * ceil(K / parts), (p + 1) * ceil(K / parts))."""
    check_matmul_args(a, weight)
    return SymmetricQuantizedMatmulF16I8Op(a, weight, scale, parallel_k_parts).outputs[0]
