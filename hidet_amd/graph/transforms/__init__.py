from .base import PassContext, SubgraphRewriteRule, GraphPass
from .selective_quantize import selective_quantize_pass, SelectiveQuantizePass
from . import graph_patterns

__all__ = ['PassContext', 'SubgraphRewriteRule', 'GraphPass', 'selective_quantize_pass', 'SelectiveQuantizePass',
           'graph_patterns']
