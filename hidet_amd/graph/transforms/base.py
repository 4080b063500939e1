"""Pass context and rewrite-rule base classes of the quantization rewrite, on torch.fx graphs.

Mirrors the part of python/hidet/graph/transforms/base.py that the quantized-matmul path uses: `PassContext` with its
stack, `set_precision` and `add_quantize_rules` (base.py:49-165), `GraphPass` (base.py:263-300), and
`SubgraphRewriteRule` (python/hidet/graph/transforms/graph_patterns/base.py: a named rule with a source pattern and a
target builder). The graph here is a `torch.fx.GraphModule` (traced by `torch.fx.symbolic_trace` or handed over by
`torch.compile`), a rule rewrites matching nodes in place.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch
from torch import fx


class SubgraphRewriteRule:
    """One rewrite: `apply` visits the graph once and returns how many sub-graphs it rewrote."""

    def __init__(self, name: str = ''):
        self.name = name

    def apply(self, gm: fx.GraphModule, ctx: 'PassContext') -> int:
        raise NotImplementedError()

    def __repr__(self):
        return '{}({})'.format(type(self).__name__, self.name)


class PassContext:
    """Options of the graph passes; `with PassContext() as ctx:` scopes them (base.py:49-110)."""

    _stack: List['PassContext'] = []

    def __init__(self):
        self.configs: Dict[str, object] = {
            'precision': None,            # target float dtype of the model: None, 'float16', 'bfloat16', 'float32'
            'quantize_patterns': [],      # selective quantization rules, applied in order
            'quantized_weights': None,    # optional QuantizedWeightStore: reuse persisted (wq, scale) instead of quantizing
            'decode_layout': False,       # keep the int8 codes of fused linears K-contiguous (see set_decode_layout)
            'verbose': False,
        }
        self.rewrites: List[Tuple[str, int]] = []  # (rule name, sub-graphs rewritten), filled by the passes

    def __enter__(self) -> 'PassContext':
        self._stack.append(self)
        return self

    def __exit__(self, exc_type, exc_val, exc_tb):
        popped = self._stack.pop()
        assert popped is self

    @classmethod
    def current(cls) -> 'PassContext':
        if len(cls._stack) == 0:
            cls._stack.append(PassContext())
        return cls._stack[-1]

    def set_precision(self, dtype: Optional[str] = None) -> 'PassContext':
        """'int8' = run the model in float16 and quantize linear / embedding weights with the default patterns
        (base.py:112-141); any other value only sets the float dtype."""
        if dtype == 'int8':
            from hidet_amd.graph import quant

            self.add_quantize_rules(quant.default_patterns())
            self.configs['precision'] = 'float16'
        else:
            if dtype not in (None, 'float16', 'bfloat16', 'float32'):
                raise ValueError("precision must be None, 'int8', 'float16', 'bfloat16' or 'float32', got {!r}".format(dtype))
            self.configs['precision'] = dtype
        return self

    def add_quantize_rules(self, patterns: Optional[List[SubgraphRewriteRule]]) -> 'PassContext':
        """Append rules (instances or classes); None clears the list (base.py:143-165)."""
        if patterns is not None:
            for pat in patterns:
                if isinstance(pat, SubgraphRewriteRule):
                    self.configs['quantize_patterns'].append(pat)
                elif isinstance(pat, type) and issubclass(pat, SubgraphRewriteRule):
                    self.configs['quantize_patterns'].append(pat())
                else:
                    raise TypeError('expected a SubgraphRewriteRule or a subclass of it, got {!r}'.format(pat))
        else:
            self.configs['quantize_patterns'] = []
        return self

    def set_quantized_weights(self, store) -> 'PassContext':
        """Weights quantized earlier (see hidet_amd.graph.frontend.torch.QuantizedWeightStore): the linear and embedding
        rules take (wq, scale) from the store when it has the parameter's name instead of quantizing again."""
        self.configs['quantized_weights'] = store
        return self

    def set_decode_layout(self, enable: bool = True) -> 'PassContext':
        """Keep the int8 codes of every fused linear layer K-contiguous (the storage order of `nn.Linear.weight`).

        Calls with a few activation rows (token-by-token decoding) then run the GEMV that reduces along the contiguous
        axis; a call with more rows makes a row-major copy of the codes the first time and keeps it, so a model that
        does both holds the int8 weights twice. No counterpart in the reference, whose quantized operator reads
        row-major `[K, N]` codes only (python/hidet/graph/ops/quant/matmul.py:24-74)."""
        self.configs['decode_layout'] = bool(enable)
        return self

    def set_verbose(self, verbose: bool = True) -> 'PassContext':
        self.configs['verbose'] = bool(verbose)
        return self


class GraphPass:
    """A pass over a GraphModule (base.py:263-300); `__call__` returns the rewritten module."""

    def __init__(self):
        self.name = type(self).__name__

    @staticmethod
    def current_context() -> PassContext:
        return PassContext.current()

    def __call__(self, gm: fx.GraphModule) -> fx.GraphModule:
        return self.process_graph(gm)

    def process_graph(self, gm: fx.GraphModule) -> fx.GraphModule:
        raise NotImplementedError()


# ---- helpers shared by the rules -------------------------------------------------------------------------------------

def fetch_attr(gm: torch.nn.Module, target: str):
    obj = gm
    for atom in target.split('.'):
        obj = getattr(obj, atom)
    return obj


def constant_of(gm: fx.GraphModule, node) -> Optional[torch.Tensor]:
    """The tensor behind a `get_attr` node (a parameter or buffer = a constant of the graph), else None."""
    if isinstance(node, fx.Node) and node.op == 'get_attr':
        value = fetch_attr(gm, node.target)
        if isinstance(value, torch.Tensor):
            return value
    return None


def node_value(node) -> Optional[torch.Tensor]:
    """Shape/dtype carrier recorded on the node by torch.compile ('example_value'), FakeTensorProp ('val') or ShapeProp
    ('tensor_meta'); None when the graph carries no such annotation."""
    if not isinstance(node, fx.Node):
        return None
    for key in ('example_value', 'val'):
        v = node.meta.get(key)
        if isinstance(v, torch.Tensor):
            return v
    return node.meta.get('tensor_meta')


def add_constant(gm: fx.GraphModule, base: str, tensor: torch.Tensor) -> str:
    """Register `tensor` as a buffer under a fresh attribute name derived from `base`; returns the name."""
    stem = base.replace('.', '_')
    name, i = stem, 0
    while hasattr(gm, name):
        i += 1
        name = '{}_{}'.format(stem, i)
    gm.register_buffer(name, tensor)
    return name
