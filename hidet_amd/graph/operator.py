"""Thin mirrors of the reference's Operator / Task objects for the quantized-matmul path.

An operator keeps `.inputs / .attrs / .task / .outputs` and runs on construction
(python/hidet/graph/operator.py:59-71); a task keeps `.name / .inputs / .outputs / .attrs` and answers
`allow_prologue / allow_epilogue` (python/hidet/ir/task.py:108-124, 317-321).  Tensors are torch tensors on
the GPU; there is no IR behind a task, only the description of what the pre-built kernel computes.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Sequence, Tuple

import torch

DTYPE_NAMES = {
    torch.float32: 'float32', torch.float16: 'float16', torch.bfloat16: 'bfloat16', torch.int8: 'int8',
    torch.int16: 'int16', torch.uint8: 'uint8', torch.float8_e4m3fn: 'float8_e4m3',
    torch.float8_e5m2: 'float8_e5m2',
}
_ALIASES = {
    'float32': torch.float32, 'f32': torch.float32, 'float16': torch.float16, 'f16': torch.float16,
    'bfloat16': torch.bfloat16, 'bf16': torch.bfloat16, 'int8': torch.int8, 'i8': torch.int8,
    'int16': torch.int16, 'i16': torch.int16, 'uint8': torch.uint8, 'float8_e4m3': torch.float8_e4m3fn,
    'f8e4m3': torch.float8_e4m3fn, 'float8_e5m2': torch.float8_e5m2, 'f8e5m2': torch.float8_e5m2,
}


def data_type(dtype) -> torch.dtype:
    """Accepts a torch dtype or one of the reference's dtype names / short names (python/hidet/ir/dtypes)."""
    if isinstance(dtype, torch.dtype):
        return dtype
    name = getattr(dtype, 'name', dtype)
    if isinstance(name, str) and name in _ALIASES:
        return _ALIASES[name]
    raise ValueError('unknown data type: {}'.format(dtype))


@dataclass
class TensorSpec:
    """What the reference's TensorNode carries for a task parameter: name, dtype, shape."""
    name: str
    dtype: str
    shape: Tuple[int, ...]


def input_like(t: torch.Tensor, name: str) -> TensorSpec:
    return TensorSpec(name, DTYPE_NAMES.get(t.dtype, str(t.dtype)), tuple(t.shape))


@dataclass
class Task:
    name: str
    inputs: List[TensorSpec]
    outputs: List[TensorSpec]
    attrs: Dict[str, Any] = field(default_factory=dict)

    def allow_prologue(self) -> bool:
        return False

    def allow_epilogue(self) -> bool:
        return False

    @staticmethod
    def _assert(cond: bool, msg: str = ''):
        # the reference's Task._assert raises on a constant-false condition (python/hidet/ir/task.py:126-137)
        if not cond:
            raise ValueError(msg or 'task assertion failed')


class Operator:
    def __init__(self, inputs: Sequence[torch.Tensor], attributes: Dict[str, Any], task: Task):
        assert all(isinstance(v, torch.Tensor) for v in inputs)
        name = type(self).__name__
        self.name: str = name[:-2] if name.endswith('Op') else name
        self.inputs: List[torch.Tensor] = list(inputs)
        self.attrs: Dict[str, Any] = attributes
        self.task: Task = task
        self.outputs: List[torch.Tensor] = self.run()

    def run(self) -> List[torch.Tensor]:
        raise NotImplementedError

    def __str__(self):
        arguments = ['{}: {}{}'.format(i, DTYPE_NAMES.get(t.dtype, t.dtype), list(t.shape)) for i, t in enumerate(self.inputs)]
        attributes = ['{}={}'.format(k, v) for k, v in self.attrs.items()]
        return '{}({})'.format(self.name, ', '.join(arguments + attributes))


def normalize_dim(dims, rank: int) -> List[int]:
    """python/hidet/graph/ops/utils: negative axes wrapped, returned as a list."""
    if isinstance(dims, int):
        dims = [dims]
    out = []
    for d in dims:
        if d < 0:
            d += rank
        if not 0 <= d < rank:
            raise ValueError('Given dims {} out of range for rank {}'.format(dims, rank))
        out.append(d)
    return out
