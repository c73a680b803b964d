"""``Conv2d`` / ``ConvTranspose2d`` with the constructor signatures, defaults, attribute names,
weight layouts, initialisation order (weight first, then bias) and error texts of
``src/tortto/nn/modules/conv.py`` (:8-56 base class, :93-102 Conv2d, :117-153 and :179-188
ConvTranspose2d).  Two-dimensional only: that is the whole convolution path of this build."""
import math

from ... import VariableFunctions as _vf
from .. import functional as F
from .. import init
from ..parameter import Parameter
from .module import Module
from .utils import _pair, _single

_PADDING_MODES = {'zeros', 'reflect', 'replicate'}
# (attribute, value that extra_repr leaves out)
_REPR_OPTIONAL = (('padding', 0), ('dilation', 1))


class _ConvNd(Module):
    """Holds the hyper-parameters and the parameters; subclasses only differ in ``forward``."""

    def __init__(self, in_channels, out_channels, kernel_size, stride, padding, dilation, transposed,
                 output_padding, groups, bias, padding_mode):
        super().__init__()
        for name, count in (('in_channels', in_channels), ('out_channels', out_channels)):
            if count % groups:
                raise ValueError(f'{name} must be divisible by groups')
        if padding_mode not in _PADDING_MODES:
            raise ValueError("padding_mode must be one of {}, but got padding_mode='{}'".format(_PADDING_MODES,
                                                                                                padding_mode))
        self.__dict__.update(in_channels=in_channels, out_channels=out_channels, kernel_size=kernel_size,
                             stride=stride, padding=padding, dilation=dilation, transposed=transposed,
                             output_padding=output_padding, groups=groups, padding_mode=padding_mode)
        lead = (in_channels, out_channels // groups) if transposed else (out_channels, in_channels // groups)
        self.weight = Parameter(_vf.zeros(lead + tuple(kernel_size)))
        self.register_parameter('bias', Parameter(_vf.zeros(out_channels)) if bias else None)
        self.reset_parameters()

    def reset_parameters(self):
        """kaiming-uniform weight with a = sqrt(5), bias uniform in +-1/sqrt(fan_in) (:52-56)."""
        init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is None:
            return
        fan_in = init._calculate_fan_in_and_fan_out(self.weight)[0]
        if fan_in:
            init.uniform_(self.bias, -1 / math.sqrt(fan_in), 1 / math.sqrt(fan_in))

    def extra_repr(self):
        parts = [f'{self.in_channels}, {self.out_channels}', f'kernel_size={self.kernel_size}', f'stride={self.stride}']
        for name, neutral in _REPR_OPTIONAL:
            value = getattr(self, name)
            if value != (neutral,) * len(value):
                parts.append(f'{name}={value}')
        if self.groups != 1:
            parts.append(f'groups={self.groups}')
        if self.bias is None:
            parts.append('bias=False')
        if self.padding_mode != 'zeros':
            parts.append(f'padding_mode={self.padding_mode}')
        return ', '.join(parts)


class Conv2d(_ConvNd):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 bias=True, padding_mode='zeros'):
        super().__init__(in_channels, out_channels, _pair(kernel_size), _pair(stride), _pair(padding),
                         _pair(dilation), False, _pair(0), groups, bias, padding_mode)

    def forward(self, inpt):
        padding = self.padding
        if self.padding_mode != 'zeros':       # explicit padding first, then an unpadded convolution (:96-100)
            inpt, padding = F.pad(inpt, self.padding, self.padding_mode), _pair(0)
        return F.conv2d(inpt, self.weight, self.bias, self.stride, padding, self.dilation, self.groups)


class ConvTranspose2d(_ConvNd):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, output_padding=0, groups=1,
                 bias=True, dilation=1, padding_mode='zeros'):
        if padding_mode != 'zeros':
            raise ValueError('Only "zeros" padding mode is supported for {}'.format(self.__class__.__name__))
        super().__init__(in_channels, out_channels, _pair(kernel_size), _pair(stride), _pair(padding),
                         _pair(dilation), True, _pair(output_padding), groups, bias, padding_mode)

    def _output_padding(self, input, output_size, stride, padding, kernel_size, dilation=None):
        """Extra rows / columns that make the output exactly ``output_size`` (:117-153): each axis
        may be anything from the size without output padding up to ``stride - 1`` more."""
        if output_size is None:
            return _single(self.output_padding)     # the reference keeps the first entry only (:121)
        spatial = input.dim() - 2
        wanted = list(output_size)
        if len(wanted) == spatial + 2:
            wanted = wanted[2:]
        if len(wanted) != spatial:
            raise ValueError('output_size must have {} or {} elements (got {})'.format(spatial, spatial + 2,
                                                                                       len(output_size)))
        smallest = [(input.shape[2 + d] - 1) * stride[d] - 2 * padding[d] +
                    (1 if dilation is None else dilation[d]) * (kernel_size[d] - 1) + 1 for d in range(spatial)]
        largest = [lo + stride[d] - 1 for d, lo in enumerate(smallest)]
        if any(not lo <= size <= hi for size, lo, hi in zip(wanted, smallest, largest)):
            raise ValueError('requested an output size of {}, but valid sizes range from {} to {} (for an input of '
                             '{})'.format(wanted, smallest, largest, input.shape[2:]))
        return [size - lo for size, lo in zip(wanted, smallest)]

    def forward(self, inpt, output_size=None):
        extra = self._output_padding(inpt, output_size, self.stride, self.padding, self.kernel_size, self.dilation)
        return F.conv_transpose2d(inpt, self.weight, self.bias, self.stride, self.padding, extra, self.groups,
                                  self.dilation)
