"""``Conv2d`` / ``ConvTranspose2d`` modules (``src/tortto/nn/modules/conv.py``): same constructor
signatures, defaults, weight shapes, initialisation order (weight, then bias) and errors."""
import math

from ... import VariableFunctions as _vf
from .. import functional as F
from .. import init
from ..parameter import Parameter
from .module import Module
from .utils import _pair, _single


class _ConvNd(Module):
    def __init__(self, in_channels, out_channels, kernel_size, stride, padding, dilation, transposed,
                 output_padding, groups, bias, padding_mode):
        super().__init__()
        if in_channels % groups != 0:
            raise ValueError('in_channels must be divisible by groups')
        if out_channels % groups != 0:
            raise ValueError('out_channels must be divisible by groups')
        valid_padding_modes = {'zeros', 'reflect', 'replicate'}
        if padding_mode not in valid_padding_modes:
            raise ValueError("padding_mode must be one of {}, but got padding_mode='{}'".format(
                valid_padding_modes, padding_mode))
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = kernel_size
        self.stride = stride
        self.padding = padding
        self.dilation = dilation
        self.transposed = transposed
        self.output_padding = output_padding
        self.groups = groups
        self.padding_mode = padding_mode
        if transposed:
            self.weight = Parameter(_vf.zeros((in_channels, out_channels // groups, *kernel_size)))
        else:
            self.weight = Parameter(_vf.zeros((out_channels, in_channels // groups, *kernel_size)))
        if bias:
            self.bias = Parameter(_vf.zeros(out_channels))
        else:
            self.register_parameter('bias', None)
        self.reset_parameters()

    def reset_parameters(self):
        init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            fan_in, _ = init._calculate_fan_in_and_fan_out(self.weight)
            if fan_in != 0:
                bound = 1 / math.sqrt(fan_in)
                init.uniform_(self.bias, -bound, bound)

    def extra_repr(self):
        s = '{in_channels}, {out_channels}, kernel_size={kernel_size}, stride={stride}'
        if self.padding != (0,) * len(self.padding):
            s += ', padding={padding}'
        if self.dilation != (1,) * len(self.dilation):
            s += ', dilation={dilation}'
        if self.groups != 1:
            s += ', groups={groups}'
        if self.bias is None:
            s += ', bias=False'
        if self.padding_mode != 'zeros':
            s += ', padding_mode={padding_mode}'
        return s.format(**self.__dict__)


class Conv2d(_ConvNd):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 bias=True, padding_mode='zeros'):
        super().__init__(in_channels, out_channels, _pair(kernel_size), _pair(stride), _pair(padding),
                         _pair(dilation), False, _pair(0), groups, bias, padding_mode)

    def forward(self, inpt):
        if self.padding_mode != 'zeros':
            return F.conv2d(F.pad(inpt, self.padding, self.padding_mode), self.weight, self.bias, self.stride,
                            _pair(0), self.dilation, self.groups)
        return F.conv2d(inpt, self.weight, self.bias, self.stride, self.padding, self.dilation, self.groups)


class _ConvTransposeNd(_ConvNd):
    def __init__(self, in_channels, out_channels, kernel_size, stride, padding, dilation, transposed,
                 output_padding, groups, bias, padding_mode):
        if padding_mode != 'zeros':
            raise ValueError('Only "zeros" padding mode is supported for {}'.format(self.__class__.__name__))
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, transposed,
                         output_padding, groups, bias, padding_mode)

    def _output_padding(self, input, output_size, stride, padding, kernel_size, dilation=None):
        """conv.py:117-153: the extra rows/columns needed to reach a requested ``output_size``."""
        if output_size is None:
            return _single(self.output_padding)
        k = input.dim() - 2
        if len(output_size) == k + 2:
            output_size = output_size[2:]
        if len(output_size) != k:
            raise ValueError('output_size must have {} or {} elements (got {})'.format(k, k + 2, len(output_size)))
        min_sizes, max_sizes = [], []
        for d in range(k):
            dil = dilation[d] if dilation is not None else 1
            lo = (input.shape[d + 2] - 1) * stride[d] - 2 * padding[d] + dil * (kernel_size[d] - 1) + 1
            min_sizes.append(lo)
            max_sizes.append(lo + stride[d] - 1)
        for size, lo, hi in zip(output_size, min_sizes, max_sizes):
            if size < lo or size > hi:
                raise ValueError('requested an output size of {}, but valid sizes range from {} to {} '
                                 '(for an input of {})'.format(output_size, min_sizes, max_sizes, input.shape[2:]))
        return [output_size[d] - min_sizes[d] for d in range(k)]


class ConvTranspose2d(_ConvTransposeNd):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, output_padding=0, groups=1,
                 bias=True, dilation=1, padding_mode='zeros'):
        super().__init__(in_channels, out_channels, _pair(kernel_size), _pair(stride), _pair(padding),
                         _pair(dilation), True, _pair(output_padding), groups, bias, padding_mode)

    def forward(self, inpt, output_size=None):
        if self.padding_mode != 'zeros':
            raise ValueError('Only `zeros` padding mode is supported for ConvTranspose2d')
        output_padding = self._output_padding(inpt, output_size, self.stride, self.padding, self.kernel_size,
                                              self.dilation)
        return F.conv_transpose2d(inpt, self.weight, self.bias, self.stride, self.padding, output_padding,
                                  self.groups, self.dilation)
