"""``ReLU`` (``src/tortto/nn/modules/activation.py:24-34``)."""
from .. import functional as F
from .module import Module


class ReLU(Module):
    def __init__(self, inplace=False):
        super().__init__()
        self.inplace = inplace

    def forward(self, tensor):
        return F.relu(tensor, inplace=self.inplace)

    def extra_repr(self):
        return 'inplace=True' if self.inplace else ''
