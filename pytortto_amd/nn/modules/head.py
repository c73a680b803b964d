"""The modules either side of the convolution stack in the reference's ResNet examples, thin
wrappers over ``nn.functional``: ``MaxPool2d`` (``src/tortto/nn/modules/pooling.py:6-27``),
``Identity`` and ``Linear`` (``linear.py:8-43``) and ``NLLLoss`` (``loss.py:38-46``)."""
import math

from ... import VariableFunctions as _vf
from .. import functional as F
from .. import init
from ..parameter import Parameter
from .module import Module
from .utils import _pair


class MaxPool2d(Module):
    def __init__(self, kernel_size, stride=None, padding=0, dilation=1, return_indices=False, ceil_mode=False):
        super().__init__()
        self.__dict__.update(kernel_size=kernel_size, stride=kernel_size if stride is None else stride,
                             padding=padding, dilation=dilation, return_indices=return_indices, ceil_mode=ceil_mode)

    def extra_repr(self):
        return (f'kernel_size={self.kernel_size}, stride={self.stride}, padding={self.padding}, '
                f'dilation={self.dilation}, ceil_mode={self.ceil_mode}')

    def forward(self, input):
        window = [_pair(v) for v in (self.kernel_size, self.stride, self.padding, self.dilation)]
        return F.max_pool2d(input, *window, self.ceil_mode, self.return_indices)


class Identity(Module):
    def __init__(self, *args, **kwargs):
        super().__init__()

    def forward(self, x):
        return x


class Linear(Module):
    """y = x @ weight.T + bias with weight [out_features, in_features]; initialised like the
    convolutions (kaiming-uniform with a = sqrt(5), bias within +-1/sqrt(fan_in))."""

    def __init__(self, in_features, out_features, bias=True):
        super().__init__()
        self.in_feature, self.out_feature = in_features, out_features      # the reference's attribute names
        self.weight = Parameter(_vf.zeros((out_features, in_features)))
        self.bias = Parameter(_vf.zeros(out_features)) if bias else None
        self.reset_parameters()

    def reset_parameters(self):
        init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            fan_in = init._calculate_fan_in_and_fan_out(self.weight)[0]
            bound = 1 / math.sqrt(fan_in) if fan_in > 0 else 0
            init.uniform_(self.bias, -bound, bound)

    def extra_repr(self):
        return f'in_feature={self.in_feature}, out_feature={self.out_feature}, bias={self.bias is not None}'

    def forward(self, x):
        return F.linear(x, self.weight, self.bias)


class NLLLoss(Module):
    def __init__(self, weight=None, ignore_index=-100, reduction='mean'):
        super().__init__()
        self.weight, self.ignore_index, self.reduction = weight, ignore_index, reduction

    def forward(self, inpt, target):
        return F.nll_loss(inpt, target, weight=self.weight, ignore_index=self.ignore_index, reduction=self.reduction)
