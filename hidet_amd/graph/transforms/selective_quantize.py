"""Selective quantization pass: apply the context's quantize rules, in order, until none of them matches
(python/hidet/graph/transforms/selective_quantize.py:23-40: one SubgraphRewrite pass per rule)."""
from torch import fx

from .base import GraphPass, PassContext


class SelectiveQuantizePass(GraphPass):
    def process_graph(self, gm: fx.GraphModule) -> fx.GraphModule:
        from .graph_patterns.quant.linear import epilogue_fusion_rules

        ctx = PassContext.current()
        rules = list(ctx.configs['quantize_patterns'])
        if rules:  # the fused operators those rules leave behind take their layer's bias into the epilogue
            rules += epilogue_fusion_rules()
        for rule in rules:
            count = rule.apply(gm, ctx)
            ctx.rewrites.append((rule.name, count))
            if ctx.configs['verbose']:
                print('[selective_quantize] {}: {} rewrite(s)'.format(rule.name, count))
            if count:
                gm.graph.eliminate_dead_code()
                gm.graph.lint()
                gm.recompile()
        _release_unused_constants(gm)
        return gm


def _release_unused_constants(gm: fx.GraphModule):
    """Drop what the rewritten graph no longer reads: sub-modules that are not called any more (the float weights of
    quantized linear layers and embeddings) and buffers of the root module that no `get_attr` node names (codes that a
    later rule replaced by another layout)."""
    gm.delete_all_unused_submodules()
    used = {str(n.target) for n in gm.graph.nodes if n.op == 'get_attr'}
    for name in [n for n, _ in gm.named_buffers(recurse=False)]:
        if name not in used:
            delattr(gm, name)


def selective_quantize_pass() -> GraphPass:
    return SelectiveQuantizePass()
