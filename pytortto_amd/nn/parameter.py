"""``nn.Parameter`` is defined next to ``Tensor``; this module keeps the reference's import path."""
from ..tensor import Parameter

__all__ = ['Parameter']
