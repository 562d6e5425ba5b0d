"""trident_amd: the attention path of kakaobrain/trident on MI355X (gfx950).

Use it where the reference is used (``import trident_amd as trident``):
``trident.function.scaled_dot_product_attention`` and ``trident.operation.Attention`` keep the
reference's signatures (trident/function/function.py:238-253, trident/operation/attention.py:23-83).
"""
from . import config, function, operation, util
from .config import *
from .module import Attention, Dropout, MaskedSoftmax, Softmax

__version__ = "0.1.0"
