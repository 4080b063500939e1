from . import quant
