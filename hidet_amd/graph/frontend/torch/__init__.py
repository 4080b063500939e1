"""torch front end of the quantized-matmul path: the `torch.compile` backend and persistence of quantized weights."""
from .dynamo_backends import hidet_backend, register_dynamo_backends, quantize_module
from .persist import QuantizedWeightStore

__all__ = ['hidet_backend', 'register_dynamo_backends', 'quantize_module', 'QuantizedWeightStore']

register_dynamo_backends()
