from . import functional
from . import module
from .module import MultiHeadAttentionMMA
