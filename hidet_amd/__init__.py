"""MI355X-native kernels for Hidet's quantized-matmul operator path, behind Hidet's Python operator API."""
from . import option
from . import ffi
from . import graph
from .graph import ops
from .ffi import BackendException

__all__ = ['option', 'ffi', 'graph', 'ops', 'BackendException']
