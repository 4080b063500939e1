"""`torch.compile(model, backend='hidet')` for the quantized-matmul path.

The reference's backend (python/hidet/graph/frontend/torch/dynamo_backends.py:144-178) turns the fx graph into a
FlowGraph, optimizes it under a fresh PassContext and runs the compiled graph; weights are constants of that graph
(:107-113). This backend keeps the fx graph, applies the *current* PassContext - so
`with PassContext() as ctx: ctx.set_precision('int8')` around the first call selects quantization, which the reference's
fresh context never does - and returns the rewritten GraphModule. Linear layers that meet the conditions of the fused
rule run on the HIP W8A16 kernels; everything else stays on torch's own operators.
"""
import copy
from typing import Callable, List, Optional, Sequence

import torch
from torch import fx

from hidet_amd.graph.transforms import PassContext, selective_quantize_pass

_PRECISIONS = {'float16': torch.float16, 'bfloat16': torch.bfloat16, 'float32': torch.float32}


def _freeze_parameters(gm: fx.GraphModule, example_inputs: Sequence) -> int:
    """torch.compile hands parameters over as graph inputs; the quantization rules want constants (`get_attr`), as in the
    reference where weights are constants of the compiled graph. Every placeholder fed by an nn.Parameter is rebound to an
    attribute holding that parameter's tensor (shared storage, no copy); the placeholder stays, unused, so the calling
    convention does not change."""
    placeholders = [n for n in gm.graph.nodes if n.op == 'placeholder']
    frozen = 0
    for node, value in zip(placeholders, example_inputs):
        if isinstance(value, torch.nn.Parameter) and len(node.users) > 0:
            name = 'frozen_' + str(node.target)
            while hasattr(gm, name):
                name += '_'
            gm.register_buffer(name, value.detach(), persistent=False)
            with gm.graph.inserting_after(node):
                const = gm.graph.get_attr(name)
            const.meta = dict(node.meta)
            node.replace_all_uses_with(const)
            frozen += 1
    if frozen:
        gm.recompile()
    return frozen


def _cast_constants(gm: fx.GraphModule, dtype: torch.dtype) -> None:
    for node in gm.graph.nodes:
        if node.op == 'get_attr':
            owner, _, leaf = node.target.rpartition('.')
            mod = gm.get_submodule(owner) if owner else gm
            value = getattr(mod, leaf)
            if isinstance(value, torch.Tensor) and value.dtype.is_floating_point and value.dtype != dtype:
                cast = value.detach().to(dtype)
                if isinstance(value, torch.nn.Parameter):
                    setattr(mod, leaf, torch.nn.Parameter(cast, requires_grad=False))
                else:
                    setattr(mod, leaf, cast)
    # sub-modules the graph calls may be the caller's own objects: cast copies, never the originals
    for name, child in list(gm.named_children()):
        if any(t.dtype.is_floating_point and t.dtype != dtype for t in list(child.parameters()) + list(child.buffers())):
            setattr(gm, name, copy.deepcopy(child).to(dtype))


class CompiledModule:
    """The callable handed back to torch.compile: casts floating inputs to the model precision, runs the rewritten graph,
    casts floating outputs back to the dtype the caller's graph produced."""

    def __init__(self, gm: fx.GraphModule, precision: Optional[torch.dtype], out_dtypes: Optional[List[Optional[torch.dtype]]]):
        self.graph_module = gm
        self.precision = precision
        self.out_dtypes = out_dtypes

    def __call__(self, *args):
        if self.precision is not None:
            args = tuple(a.to(self.precision) if isinstance(a, torch.Tensor) and a.dtype.is_floating_point
                         and a.dtype != self.precision else a for a in args)
        out = self.graph_module(*args)
        if self.precision is None or self.out_dtypes is None:
            return out
        if isinstance(out, (tuple, list)):
            return type(out)(o.to(d) if isinstance(o, torch.Tensor) and d is not None and o.dtype != d else o
                             for o, d in zip(out, self.out_dtypes))
        d = self.out_dtypes[0]
        return out.to(d) if isinstance(out, torch.Tensor) and d is not None and out.dtype != d else out


def _output_dtypes(gm: fx.GraphModule) -> Optional[List[Optional[torch.dtype]]]:
    out_node = next(n for n in reversed(gm.graph.nodes) if n.op == 'output')
    outs = out_node.args[0]
    outs = outs if isinstance(outs, (tuple, list)) else (outs,)
    dtypes = []
    for o in outs:
        val = o.meta.get('example_value', o.meta.get('val')) if isinstance(o, fx.Node) else None
        dtypes.append(val.dtype if isinstance(val, torch.Tensor) and val.dtype.is_floating_point else None)
    return dtypes


def hidet_backend(graph_module: fx.GraphModule, example_inputs, **kwargs) -> Callable:
    assert isinstance(graph_module, fx.GraphModule)
    ctx = PassContext.current()
    out_dtypes = _output_dtypes(graph_module)
    _freeze_parameters(graph_module, example_inputs)
    precision = _PRECISIONS.get(ctx.configs['precision']) if ctx.configs['precision'] else None
    if precision is not None:
        _cast_constants(graph_module, precision)
    graph_module = selective_quantize_pass()(graph_module)
    return CompiledModule(graph_module, precision, out_dtypes)


def quantize_module(module: torch.nn.Module, ctx: Optional[PassContext] = None) -> fx.GraphModule:
    """Ahead-of-time form of the same rewrite: symbolic-trace `module`, cast its constants to the context's precision and
    apply the context's quantize rules. The result is an ordinary GraphModule (inputs are not cast for the caller)."""
    ctx = ctx if ctx is not None else PassContext.current()
    # the rewrite casts and replaces constants: it works on a copy, the caller's module keeps its parameters and dtypes
    # (the reference's from_torch leaves the torch model untouched as well)
    module = copy.deepcopy(module)
    gm = module if isinstance(module, fx.GraphModule) else fx.symbolic_trace(module)
    precision = _PRECISIONS.get(ctx.configs['precision']) if ctx.configs['precision'] else None
    if precision is not None:
        _cast_constants(gm, precision)
    with ctx:
        gm = selective_quantize_pass()(gm)
    return gm


def register_dynamo_backends() -> None:
    """Make `torch.compile(..., backend='hidet')` (and 'hidet_amd') resolve to this backend. The reference registers
    'hidet' through an entry point (python/hidet/graph/frontend/torch/__init__.py:71-75); a name that is already taken
    is left alone."""
    try:
        from torch._dynamo import register_backend, list_backends
    except ImportError:  # torch without dynamo
        return
    taken = set(list_backends(None))
    for name in ('hidet', 'hidet_amd'):
        if name not in taken:
            register_backend(compiler_fn=hidet_backend, name=name)
