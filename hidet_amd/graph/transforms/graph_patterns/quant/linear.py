"""Rewrite rules that quantize linear layers (python/hidet/graph/transforms/graph_patterns/quant/linear.py).

As in the reference a linear layer is "a matmul one of whose operands is a constant with two dimensions"
(linear.py:21-22). On a torch.fx graph that is an `nn.Linear` module call, `F.linear(x, w, b)` or a
`matmul(x, w)` / `matmul(w, x)` whose `w` is a `get_attr` node. Two steps, as in the reference:

  1. SymmetricLinearQuantizePatternR / L   linear(x, w) => matmul(x, dequant(wq, scale))      (linear.py:25-78)
     the weight is quantized once, at rewrite time, and (wq, scale) become constants of the graph;
  2. SymmetricQuantizeMatmulFused          matmul(x, dequant(wq, scale)) => symmetric_quant_matmul(x, wq, scale)
     under the same conditions as linear.py:104-124 (float16 activations, int8 2-D codes, dims = 0, one scale per
     output column, N a multiple of 4).

A linear layer that fails the conditions of step 2 keeps running as matmul over the dequantized weight.
"""
import operator
from typing import List, Optional, Union

import torch
import torch.nn.functional as F
from torch import fx

from hidet_amd.graph.operator import normalize_dim
from ...base import SubgraphRewriteRule, PassContext, constant_of, node_value, add_constant, fetch_attr

_MATMUL_FUNCTIONS = (torch.matmul, operator.matmul)


def _quant_ops():
    from hidet_amd.graph.ops import quant

    return quant


def _is_matmul(node: fx.Node) -> bool:
    if node.op == 'call_function' and node.target in _MATMUL_FUNCTIONS:
        return True
    return node.op == 'call_method' and node.target == 'matmul'


def _quantized_constants(gm: fx.GraphModule, ctx: PassContext, name: str, w_kn: torch.Tensor, quant_type: str, dims):
    """(wq, scale) of the constant `w_kn`, from the context's store of persisted weights when it has `name`."""
    store = ctx.configs.get('quantized_weights')
    if store is not None and name in store:
        wq, scale = store[name]
        return wq.to(w_kn.device), scale.to(w_kn.device)
    wq, scale = _quant_ops().symmetric_quantize(w_kn.contiguous(), quant_type=quant_type, dims=dims)
    if store is not None:
        store[name] = (wq, scale)
    return wq, scale


def _insert_dequant(gm: fx.GraphModule, before: fx.Node, name: str, wq: torch.Tensor, scale: torch.Tensor, dims) -> fx.Node:
    wq_name = add_constant(gm, name + '_wq', wq)
    scale_name = add_constant(gm, name + '_scale', scale)
    with gm.graph.inserting_before(before):
        wq_node = gm.graph.get_attr(wq_name)
        scale_node = gm.graph.get_attr(scale_name)
        return gm.graph.call_function(_quant_ops().symmetric_dequantize, (wq_node, scale_node), {'dims': dims})


class SymmetricLinearQuantizePatternR(SubgraphRewriteRule):
    """linear(x, w) => matmul(x, dequant(wq, scale)) with w the right operand (linear.py:25-50)."""

    def __init__(self, quant_type: str = 'int8', dims: Union[int, List[int]] = 0):
        super().__init__('linear(x, w) => linear(x, dequant(wq, scale, {}, dims={}))'.format(quant_type, dims))
        self.quant_type = quant_type
        self.dims = dims

    def apply(self, gm: fx.GraphModule, ctx: PassContext) -> int:
        count = 0
        for node in list(gm.graph.nodes):
            x = bias = None
            if node.op == 'call_module':
                mod = fetch_attr(gm, node.target)
                if type(mod) is not torch.nn.Linear:
                    continue
                x, name = node.args[0], node.target + '.weight'
                w_kn = mod.weight.detach().t()
                bias_t = None if mod.bias is None else mod.bias.detach()
            elif node.op == 'call_function' and node.target is F.linear:
                w = constant_of(gm, node.args[1] if len(node.args) > 1 else node.kwargs.get('weight'))
                if w is None or w.dim() != 2:
                    continue
                x, name = node.args[0], (node.args[1] if len(node.args) > 1 else node.kwargs['weight']).target
                w_kn = w.detach().t()
                bias = node.args[2] if len(node.args) > 2 else node.kwargs.get('bias')
                bias_t = None
            elif _is_matmul(node) and len(node.args) == 2:
                w = constant_of(gm, node.args[1])
                if w is None or w.dim() != 2:  # only two-dimensional constants are linear-layer weights (linear.py:38-39)
                    continue
                x, name, w_kn, bias_t = node.args[0], node.args[1].target, w.detach(), None
            else:
                continue
            if not w_kn.dtype.is_floating_point:
                continue
            wq, scale = _quantized_constants(gm, ctx, name, w_kn, self.quant_type, self.dims)
            w_dq = _insert_dequant(gm, node, name, wq, scale, self.dims)
            with gm.graph.inserting_before(node):
                out = gm.graph.call_function(torch.matmul, (x, w_dq))
                if node.op == 'call_module' and bias_t is not None:
                    bias = gm.graph.get_attr(add_constant(gm, node.target + '_bias', bias_t))
                if bias is not None:
                    out = gm.graph.call_function(torch.add, (out, bias))
            out.meta = dict(node.meta)
            node.replace_all_uses_with(out)
            gm.graph.erase_node(node)
            count += 1
        return count


class SymmetricLinearQuantizePatternL(SubgraphRewriteRule):
    """matmul(w, x) => matmul(dequant(wq, scale), x) with w the left operand (linear.py:53-78)."""

    def __init__(self, quant_type: str = 'int8', dims: Union[int, List[int]] = 0):
        super().__init__('matmul(w, x) => matmul(dequant(wq, scale, {}, dims={}), x)'.format(quant_type, dims))
        self.quant_type = quant_type
        self.dims = dims

    def apply(self, gm: fx.GraphModule, ctx: PassContext) -> int:
        count = 0
        for node in list(gm.graph.nodes):
            if not (_is_matmul(node) and len(node.args) == 2):
                continue
            w = constant_of(gm, node.args[0])
            if w is None or w.dim() != 2 or not w.dtype.is_floating_point:
                continue
            name = node.args[0].target
            wq, scale = _quantized_constants(gm, ctx, name, w.detach(), self.quant_type, self.dims)
            w_dq = _insert_dequant(gm, node, name, wq, scale, self.dims)
            with gm.graph.inserting_before(node):
                out = gm.graph.call_function(torch.matmul, (w_dq, node.args[1]))
            out.meta = dict(node.meta)
            node.replace_all_uses_with(out)
            gm.graph.erase_node(node)
            count += 1
        return count


def symmetric_linear_quantize_patterns(quant_type: str = 'int8', dims=0) -> List[SubgraphRewriteRule]:
    return [SymmetricLinearQuantizePatternR(quant_type=quant_type, dims=dims),
            SymmetricLinearQuantizePatternL(quant_type=quant_type, dims=dims)]


class SymmetricQuantizeMatmulFused(SubgraphRewriteRule):
    """matmul(x, dequant(wq, scale)) => symmetric_quant_matmul(x, wq, scale) (linear.py:88-124)."""

    def __init__(self):
        super().__init__('matmul(x, dequant(wq, scale)) => fused_matmulf16(x, wq, scale)')

    def apply(self, gm: fx.GraphModule, ctx: PassContext) -> int:
        quant = _quant_ops()
        count = 0
        for node in list(gm.graph.nodes):
            if not (_is_matmul(node) and len(node.args) == 2):
                continue
            x, w_dequant = node.args
            if not (isinstance(w_dequant, fx.Node) and w_dequant.op == 'call_function'
                    and w_dequant.target is quant.symmetric_dequantize):
                continue
            wq = constant_of(gm, w_dequant.args[0])
            scale = constant_of(gm, w_dequant.args[1])
            if wq is None or scale is None:
                continue
            dims = w_dequant.kwargs.get('dims', w_dequant.args[2] if len(w_dequant.args) > 2 else -1)
            dim = normalize_dim(dims, wq.dim())
            # the conditions of linear.py:104-122
            if wq.dim() != 2 or wq.dtype != torch.int8:
                continue
            if list(dim) != [0]:
                continue
            if scale.shape[0] != wq.shape[1]:
                continue
            if wq.shape[-1] % 4 != 0:
                continue
            # the fused operator is float16 x int8 -> float16 (linear.py:114-115). The activation dtype is the context's
            # precision when one is set (the graph's annotations predate that cast), else the graph's annotation, else
            # the dtype the weight was quantized in.
            precision = ctx.configs.get('precision')
            if precision is not None:
                x_dtype = {'float16': torch.float16, 'bfloat16': torch.bfloat16, 'float32': torch.float32}[precision]
            else:
                x_dtype = getattr(node_value(x), 'dtype', None) or scale.dtype
            if x_dtype != torch.float16 or scale.dtype != torch.float16:
                continue
            with gm.graph.inserting_before(node):
                wq_node = w_dequant.args[0]
                if ctx.configs.get('decode_layout'):
                    # same [K, N] operand, stored K-contiguous; the row-major constant loses its last user below
                    wq_node = gm.graph.get_attr(add_constant(gm, wq_node.target + '_kc', quant.to_decode_layout(wq)))
                out = gm.graph.call_function(quant.symmetric_quant_matmul, (x, wq_node, w_dequant.args[1]))
            out.meta = dict(node.meta)
            node.replace_all_uses_with(out)
            gm.graph.erase_node(node)
            count += 1
        return count


class SymmetricQuantizeMatmulBiasFused(SubgraphRewriteRule):
    """add(symmetric_quant_matmul(x, wq, scale), bias) => symmetric_quant_matmul(x, wq, scale, bias) for a constant float16
    bias of one element per output column: the bias of an nn.Linear rides in the kernel's epilogue instead of a separate
    element-wise launch per layer. The reference gets the same effect from its fusion pass, which folds the add into the
    template's epilogue (matmul_f16_i8.py:95-99, allow_epilogue); there is no rule of this name there. The fused kernel adds
    the bias to the float16 product with a second rounding, so the rewritten graph returns the bits of the unfused one."""

    def __init__(self):
        super().__init__('add(fused_matmulf16(x, wq, scale), bias) => fused_matmulf16(x, wq, scale, bias)')

    def apply(self, gm: fx.GraphModule, ctx: PassContext) -> int:
        import operator as py_operator

        quant = _quant_ops()
        count = 0
        for node in list(gm.graph.nodes):
            if not (node.op == 'call_function' and node.target in (torch.add, py_operator.add) and len(node.args) == 2
                    and not node.kwargs):
                continue
            for mm, other in ((node.args[0], node.args[1]), (node.args[1], node.args[0])):
                if not (isinstance(mm, fx.Node) and mm.op == 'call_function' and mm.target is quant.symmetric_quant_matmul
                        and len(mm.args) == 3 and not mm.kwargs and len(mm.users) == 1 and isinstance(other, fx.Node)):
                    continue
                bias = constant_of(gm, other)
                wq = constant_of(gm, mm.args[1])
                if bias is None or wq is None or bias.dim() != 1 or bias.shape[0] != wq.shape[1] or bias.dtype != torch.float16:
                    continue
                with gm.graph.inserting_before(node):
                    out = gm.graph.call_function(quant.symmetric_quant_matmul, tuple(mm.args) + (other,))
                out.meta = dict(node.meta)
                node.replace_all_uses_with(out)
                gm.graph.erase_node(node)
                gm.graph.erase_node(mm)
                count += 1
                break
        return count


def matmul_specialization_rules() -> List[SubgraphRewriteRule]:
    """Rules that replace generic sub-graphs by fused operators where those apply (linear.py:127-129)."""
    return [SymmetricQuantizeMatmulFused()]


def epilogue_fusion_rules() -> List[SubgraphRewriteRule]:
    """What the reference leaves to its operator-fusion pass, which runs after the quantize rules: here the quantize pass
    applies these once the context's own rules are done."""
    return [SymmetricQuantizeMatmulBiasFused()]
