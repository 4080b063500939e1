"""symmetric_quantize / symmetric_dequantize with the reference's signatures
(python/hidet/graph/ops/quant/symmetric.py:23-88), executed by the HIP kernels behind
`hidet_symmetric_quantize` / `hidet_symmetric_dequantize`."""
from typing import List, Sequence, Tuple, Union

import torch

from hidet_amd import ffi
from hidet_amd.graph.operator import Operator, Task, TensorSpec, data_type, input_like, normalize_dim, DTYPE_NAMES

_FLOATS = (torch.float32, torch.float16, torch.bfloat16)
_QUANTS = (torch.int8, torch.int16)


def _prod(xs: Sequence[int]) -> int:
    p = 1
    for x in xs:
        p *= int(x)
    return p


def _view_plan(shape: Sequence[int], dims: List[int]):
    """Fold `shape` into [outer, reduce, inner] when the reduced axes are adjacent; otherwise return the
    permutation that moves them last (then inner == 1)."""
    red = sorted(set(dims))
    if red == list(range(red[0], red[-1] + 1)):
        lo, hi = red[0], red[-1]
        return None, (_prod(shape[:lo]), _prod(shape[lo:hi + 1]), _prod(shape[hi + 1:]))
    kept = [i for i in range(len(shape)) if i not in red]
    perm = kept + red
    return perm, (_prod([shape[i] for i in kept]), _prod([shape[i] for i in red]), 1)


class SymmetricQuantizationTask(Task):
    def __init__(self, w: TensorSpec, quant_type: torch.dtype, dims: Union[int, List[int]] = -1):
        dims = normalize_dim(dims, len(w.shape))
        scale_shape = tuple(s for i, s in enumerate(w.shape) if i not in dims)
        super().__init__(
            name='symmetric_quantization',
            inputs=[w],
            outputs=[TensorSpec('quantize', DTYPE_NAMES[quant_type], w.shape), TensorSpec('scaling', w.dtype, scale_shape)],
            attrs={'dims': dims, 'quant_type': quant_type},
        )


class SymmetricDeQuantizationTask(Task):
    def __init__(self, wq: TensorSpec, scale: TensorSpec, dims: Union[int, List[int]] = -1):
        dims = normalize_dim(dims, len(wq.shape))
        super().__init__(
            name='symmetric_dequantization',
            inputs=[wq, scale],
            outputs=[TensorSpec('dequantize', scale.dtype, wq.shape)],
            attrs={'dims': dims},
        )


class SymmetricQuantizationOp(Operator):
    def __init__(self, w: torch.Tensor, quant_type: torch.dtype, dims: Union[int, List[int]] = -1):
        super().__init__(
            inputs=[w],
            attributes={'dims': dims, 'quant_type': quant_type},
            task=SymmetricQuantizationTask(input_like(w, 'w'), quant_type=quant_type, dims=dims),
        )

    def run(self) -> List[torch.Tensor]:
        (w,) = self.inputs
        ffi.require_gpu(w)
        quant_type = self.attrs['quant_type']
        dims = self.task.attrs['dims']
        shape = tuple(w.shape)
        perm, (outer, reduce, inner) = _view_plan(shape, dims)
        src = w.contiguous() if perm is None else w.permute(perm).contiguous()
        wq = torch.empty(src.shape, dtype=quant_type, device=w.device)
        scale_shape = [s for i, s in enumerate(shape) if i not in dims]
        scale = torch.empty(scale_shape, dtype=w.dtype, device=w.device)
        ws = ffi.workspace(w.device, (64 << 10) + 4 * outer * inner)
        ffi.call('hidet_symmetric_quantize', src, wq, scale, outer, reduce, inner, ffi.DTYPE_CODE[w.dtype],
                 ffi.DTYPE_CODE[quant_type], ws, ws.numel(), ffi.current_stream(w.device))
        if perm is not None:
            inv = [0] * len(perm)
            for i, p in enumerate(perm):
                inv[p] = i
            wq = wq.permute(inv).contiguous()
        return [wq, scale]


class SymmetricDeQuantizationOp(Operator):
    def __init__(self, wq: torch.Tensor, scale: torch.Tensor, dims: Union[int, List[int]] = -1):
        super().__init__(
            inputs=[wq, scale],
            attributes={'dims': dims},
            task=SymmetricDeQuantizationTask(input_like(wq, 'wq'), input_like(scale, 'scale'), dims=dims),
        )

    def run(self) -> List[torch.Tensor]:
        wq, scale = self.inputs
        ffi.require_gpu(wq, scale)
        dims = self.task.attrs['dims']
        shape = tuple(wq.shape)
        kept = tuple(s for i, s in enumerate(shape) if i not in dims)
        if tuple(scale.shape) != kept:
            raise ValueError('scale shape {} does not match the non-reduced axes {} of wq {}'.format(
                tuple(scale.shape), kept, shape))
        perm, (outer, reduce, inner) = _view_plan(shape, dims)
        src = wq.contiguous() if perm is None else wq.permute(perm).contiguous()
        w = torch.empty(src.shape, dtype=scale.dtype, device=wq.device)
        ffi.call('hidet_symmetric_dequantize', src, scale.contiguous(), w, outer, reduce, inner,
                 ffi.DTYPE_CODE[wq.dtype], ffi.DTYPE_CODE[scale.dtype], ffi.current_stream(wq.device))
        if perm is not None:
            inv = [0] * len(perm)
            for i, p in enumerate(perm):
                inv[p] = i
            w = w.permute(inv).contiguous()
        return [w]


def symmetric_quantize(w: torch.Tensor, quant_type='int8', dims: Union[int, List[int]] = -1) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (wq, scale); `dims` are the reduced axes and `scale` keeps the other axes, in w's dtype."""
    quant_type = data_type(quant_type)
    if quant_type not in _QUANTS:
        raise ValueError('symmetric_quantize supports int8 and int16, got {}'.format(quant_type))
    if w.dtype not in _FLOATS:
        raise ValueError('symmetric_quantize expects a float32, float16 or bfloat16 tensor, got {}'.format(w.dtype))
    op = SymmetricQuantizationOp(w, quant_type, dims=dims)
    return op.outputs[0], op.outputs[1]


def symmetric_dequantize(wq: torch.Tensor, scale: torch.Tensor, dims: Union[int, List[int]] = -1) -> torch.Tensor:
    if wq.dtype not in _QUANTS:
        raise ValueError('symmetric_dequantize expects int8 or int16 codes, got {}'.format(wq.dtype))
    if scale.dtype not in _FLOATS:
        raise ValueError('symmetric_dequantize expects a float32, float16 or bfloat16 scale, got {}'.format(scale.dtype))
    return SymmetricDeQuantizationOp(wq, scale, dims).outputs[0]
