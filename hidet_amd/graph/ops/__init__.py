from . import quant
from . import matmul
from .quant import symmetric_quantize, symmetric_dequantize  # python/hidet/graph/ops/__init__.py:40
