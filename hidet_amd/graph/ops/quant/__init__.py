# the exports of python/hidet/graph/ops/quant/__init__.py:12-15, plus the resolve policy the reference forgets to import
from .symmetric import symmetric_quantize, symmetric_dequantize
from .matmul import symmetric_quant_matmul, to_decode_layout  # to_decode_layout: not in the reference
from .matmul_f16_i8 import symmetric_quant_matmul_f16_i8
from .matmul_f16_i8_atomic import symmetric_quant_matmul_atomic_f16_i8
from . import resolve
from .group_int4 import (symmetric_group_quantize_int4, symmetric_quant_matmul_w4a16,  # group-wise W4A16 (not in the reference)
                         to_decode_layout_int4, symmetric_quant_matmul_w4a16_decode)
