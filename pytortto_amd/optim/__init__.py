"""``tt.optim``: the optimisers that consume the gradients of the path (``src/tortto/optim``)."""
from .optimizer import Optimizer
from .adam import Adam, AdamW
from .sgd import SGD

__all__ = ['Optimizer', 'SGD', 'Adam', 'AdamW']
