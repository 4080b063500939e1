"""Rewrite rule that quantizes embedding tables (python/hidet/graph/transforms/graph_patterns/quant/embedding.py).

An embedding layer is a row gather (axis 0) from a constant 2-D table with integer indices (embedding.py:20-34): an
`nn.Embedding` module call or `F.embedding(ind, w)` with `w` a `get_attr` node. The table is quantized once with one
scale per row (`dims=[-1]`, embedding.py:38); at run time the gathered rows are dequantized,
`dequant(wq[ind], scale[ind])`, which is element for element `take(dequant(wq, scale), ind)` of embedding.py:39
without dequantizing the whole table on every call.
"""
from typing import List

import torch
import torch.nn.functional as F
from torch import fx

from ...base import SubgraphRewriteRule, PassContext, constant_of, add_constant, fetch_attr


class SymmetricEmbeddingQuantizePattern(SubgraphRewriteRule):
    def __init__(self, quant_type: str = 'int8'):
        super().__init__('embedding(w, ind) => embedding(dequant(wq, scale, {}), ind)'.format(quant_type))
        self.quant_type = quant_type

    def apply(self, gm: fx.GraphModule, ctx: PassContext) -> int:
        from hidet_amd.graph.ops import quant
        from .linear import _quantized_constants

        count = 0
        for node in list(gm.graph.nodes):
            if node.op == 'call_module':
                mod = fetch_attr(gm, node.target)
                if type(mod) is not torch.nn.Embedding or mod.max_norm is not None:
                    continue
                ind, name, w = node.args[0], node.target + '.weight', mod.weight.detach()
            elif node.op == 'call_function' and node.target is F.embedding:
                w_node = node.args[1] if len(node.args) > 1 else node.kwargs.get('weight')
                w = constant_of(gm, w_node)
                # F.embedding(input, weight, padding_idx, max_norm, ...): max_norm renormalizes the table in place, which a
                # quantized table cannot follow; the other options do not change the forward result
                max_norm = node.args[3] if len(node.args) > 3 else node.kwargs.get('max_norm')
                if w is None or max_norm is not None:
                    continue
                ind, name = node.args[0], w_node.target
            else:
                continue
            if w.dim() != 2 or not w.dtype.is_floating_point:
                continue
            wq, scale = _quantized_constants(gm, ctx, name, w, self.quant_type, [-1])
            wq_name = add_constant(gm, name + '_wq', wq)
            scale_name = add_constant(gm, name + '_scale', scale)
            with gm.graph.inserting_before(node):
                wq_node = gm.graph.get_attr(wq_name)
                scale_node = gm.graph.get_attr(scale_name)
                rows = gm.graph.call_function(F.embedding, (ind, wq_node))                       # int8 [..., D]
                row_scale = gm.graph.call_function(_take_rows, (scale_node, ind))                      # [...]
                out = gm.graph.call_function(quant.symmetric_dequantize, (rows, row_scale), {'dims': [-1]})
            out.meta = dict(node.meta)
            node.replace_all_uses_with(out)
            gm.graph.erase_node(node)
            count += 1
        return count


def _take_rows(values: torch.Tensor, ind: torch.Tensor) -> torch.Tensor:
    """values[ind] for a 1-D `values`: the scale of every gathered row."""
    return values[ind]


def symmetric_embedding_quantize_patterns(quant_type: str = 'int8') -> List[SubgraphRewriteRule]:
    return [SymmetricEmbeddingQuantizePattern(quant_type=quant_type)]
