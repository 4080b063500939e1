from . import ops
from . import transforms
from .transforms import PassContext
from .transforms.graph_patterns import quant  # hidet.graph.quant (python/hidet/graph/__init__.py:31)
from . import frontend
