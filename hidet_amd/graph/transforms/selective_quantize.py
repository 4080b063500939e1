"""Selective quantization pass: apply the context's quantize rules, in order, until none of them matches
(python/hidet/graph/transforms/selective_quantize.py:23-40: one SubgraphRewrite pass per rule)."""
from torch import fx

from .base import GraphPass, PassContext


class SelectiveQuantizePass(GraphPass):
    def process_graph(self, gm: fx.GraphModule) -> fx.GraphModule:
        ctx = PassContext.current()
        for rule in ctx.configs['quantize_patterns']:
            count = rule.apply(gm, ctx)
            ctx.rewrites.append((rule.name, count))
            if ctx.configs['verbose']:
                print('[selective_quantize] {}: {} rewrite(s)'.format(rule.name, count))
            if count:
                gm.graph.eliminate_dead_code()
                gm.graph.lint()
                gm.recompile()
        return gm


def selective_quantize_pass() -> GraphPass:
    return SelectiveQuantizePass()
