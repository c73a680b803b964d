"""``tt.optim``: the optimisers that consume the gradients of the path (``src/tortto/optim``)."""
from .optimizer import Optimizer
from .rules import SGD, Adam, AdamW

__all__ = ['Optimizer', 'SGD', 'Adam', 'AdamW']
