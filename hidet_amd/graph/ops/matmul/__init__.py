# the reference does not re-export matmul_f8 from ops.matmul either: import it by its full path
# (python/hidet/graph/ops/matmul/__init__.py, tests/operators_core/test_matmul.py:259)
from . import matmul_f8
