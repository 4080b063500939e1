"""symmetric_quant_matmul_atomic_f16_i8: the split-K form that reduces its parts in place and returns
[..., M, N] (python/hidet/graph/ops/quant/matmul_f16_i8_atomic.py:31-92, 555-565).

The reference zero-fills the output and adds float16 pairs atomically, so its result depends on arrival
order.  The MI355X kernel adds the parts in a fixed order in float32, so this entry is deterministic."""
from typing import List

import torch

from hidet_amd.graph.operator import Operator, Task, TensorSpec, input_like
from .matmul import _check_task_operands, check_matmul_args, run_w8a16


class SymmetricQuantizedMatmulAtomicF16I8Task(Task):
    def __init__(self, a: TensorSpec, weight: TensorSpec, scale: TensorSpec, parallel_k_parts: int = 1):
        _check_task_operands(self, a, weight, scale)
        c_shape = tuple(a.shape[:-1]) + (weight.shape[-1],)
        super().__init__(name='symmetric_quantized_matmulf16', inputs=[a, weight, scale],
                         outputs=[TensorSpec('c', 'float16', c_shape)], attrs={'parallel_k_parts': parallel_k_parts})


class SymmetricQuantizedMatmulAtomicF16I8Op(Operator):
    def __init__(self, a: torch.Tensor, b: torch.Tensor, scale: torch.Tensor, parallel_k_parts: int = 1):
        if not isinstance(parallel_k_parts, int) or parallel_k_parts < 1:
            raise ValueError('parallel_k_parts must be a positive integer, got {}'.format(parallel_k_parts))
        super().__init__(
            inputs=[a, b, scale],
            attributes={'parallel_k_parts': parallel_k_parts},
            task=SymmetricQuantizedMatmulAtomicF16I8Task(input_like(a, 'a'), input_like(b, 'b'),
                                                         input_like(scale, 'scale'), parallel_k_parts),
        )

    def run(self) -> List[torch.Tensor]:
        a, b, scale = self.inputs
        return [run_w8a16(a, b, scale, self.attrs['parallel_k_parts'])]


def symmetric_quant_matmul_atomic_f16_i8(a: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor, parallel_k_parts=1) -> torch.Tensor:
    check_matmul_args(a, weight)
    return SymmetricQuantizedMatmulAtomicF16I8Op(a, weight, scale, parallel_k_parts).outputs[0]
