"""Persistence of quantized weights next to a saved model.

The reference bakes quantized weights into the compiled graph and stores a graph's weights as one `.npz`
(python/hidet/runtime/compiled_graph.py:610-693). Here the (codes, scale) pairs the rewrite rules produce are kept in a
`QuantizedWeightStore`, keyed by the parameter's qualified name, which saves to / loads from one `.npz`. Handing a loaded
store to `PassContext.set_quantized_weights` makes the rules reuse those tensors instead of quantizing again, so a model
can be shipped with int8 weights only.
"""
from typing import Dict, Tuple

import numpy as np
import torch

_SCALE_DTYPES = {'float32': torch.float32, 'float16': torch.float16, 'bfloat16': torch.bfloat16}


class QuantizedWeightStore(dict):
    """name -> (wq integer codes, scale) as torch tensors."""

    def save(self, path: str) -> None:
        arrays: Dict[str, np.ndarray] = {}
        for name, (wq, scale) in self.items():
            arrays[name + '::wq'] = wq.detach().cpu().numpy()
            dtype_name = str(scale.dtype).replace('torch.', '')
            if scale.dtype == torch.bfloat16:  # numpy has no bfloat16: keep the bit pattern
                arrays[name + '::scale::bfloat16'] = scale.detach().cpu().view(torch.int16).numpy()
            else:
                arrays[name + '::scale::' + dtype_name] = scale.detach().cpu().numpy()
        with open(path, 'wb') as f:
            np.savez(f, **arrays)

    @classmethod
    def load(cls, path: str, device='cpu') -> 'QuantizedWeightStore':
        store = cls()
        pending: Dict[str, Dict[str, torch.Tensor]] = {}
        with np.load(path, allow_pickle=False) as data:
            for key in data.files:
                parts = key.split('::')
                name, kind = parts[0], parts[1]
                t = torch.from_numpy(data[key])
                if kind == 'scale':
                    dtype = _SCALE_DTYPES[parts[2]]
                    t = t.view(torch.bfloat16) if dtype == torch.bfloat16 else t.to(dtype)
                pending.setdefault(name, {})[kind] = t.to(device)
        for name, pair in pending.items():
            if 'wq' not in pair or 'scale' not in pair:
                raise ValueError('incomplete entry for {!r} in {}'.format(name, path))
            store[name] = (pair['wq'], pair['scale'])
        return store

    def nbytes(self) -> int:
        return sum(wq.numel() * wq.element_size() + s.numel() * s.element_size() for wq, s in self.values())

    def pairs(self) -> Tuple[Tuple[str, torch.Tensor, torch.Tensor], ...]:
        return tuple((name, wq, s) for name, (wq, s) in self.items())
