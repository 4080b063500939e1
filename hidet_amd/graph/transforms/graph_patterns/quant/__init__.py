"""Default quantization patterns (python/hidet/graph/transforms/graph_patterns/quant/__init__.py:19-61)."""
from typing import List, Union

from ...base import SubgraphRewriteRule
from .embedding import symmetric_embedding_quantize_patterns, SymmetricEmbeddingQuantizePattern
from .linear import (symmetric_linear_quantize_patterns, matmul_specialization_rules, SymmetricLinearQuantizePatternR,
                     SymmetricLinearQuantizePatternL, SymmetricQuantizeMatmulFused)


def default_patterns() -> List[SubgraphRewriteRule]:
    """int8, one scale per output channel of every linear layer, one per row of every embedding table."""
    quant_type = 'int8'
    dims = 0
    rules = symmetric_linear_patterns(quant_type=quant_type, dims=dims)
    rules += symmetric_embedding_patterns(quant_type=quant_type)
    return rules


def symmetric_linear_patterns(quant_type: str = 'int8', dims: Union[int, List[int]] = 0) -> List[SubgraphRewriteRule]:
    """Channel-wise symmetric weight quantization of linear layers (a matmul with a constant 2-D weight), followed by
    the rule that fuses `matmul(x, dequant(wq, scale))` into the quantized-matmul operator."""
    rules = symmetric_linear_quantize_patterns(quant_type=quant_type, dims=dims)
    rules.extend(matmul_specialization_rules())
    return rules


def symmetric_embedding_patterns(quant_type: str = 'int8') -> List[SubgraphRewriteRule]:
    """Row-wise symmetric weight quantization of embedding layers (a row gather from a constant 2-D table)."""
    return symmetric_embedding_quantize_patterns(quant_type=quant_type)
