"""``ReLU``, ``LeakyReLU`` and ``LogSoftmax`` (``src/tortto/nn/modules/activation.py:24-48``,
``:75-84``): each keeps its hyper-parameters and calls the functional of the same name."""
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


class LeakyReLU(Module):
    def __init__(self, negative_slope=1e-2, inplace=False):
        super().__init__()
        self.negative_slope, self.inplace = negative_slope, inplace

    def forward(self, tensor):
        return F.leaky_relu(tensor, self.negative_slope, self.inplace)

    def extra_repr(self):
        return f'negative_slope={self.negative_slope}' + (', inplace=True' if self.inplace else '')


class LogSoftmax(Module):
    def __init__(self, dim):
        super().__init__()
        self.dim = dim

    def forward(self, tensor):
        return F.log_softmax(tensor, self.dim)

    def extra_repr(self):
        return f'dim={self.dim}'
