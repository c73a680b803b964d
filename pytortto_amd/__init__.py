"""pytortto_amd -- the MI355X (gfx950) convolution / BatchNorm path behind tortto's API.

Mirrors the names of samrere/pytortto that the path sits behind: ``tensor``, ``Tensor``,
``manual_seed``, ``randn``/``zeros``/``ones``, ``no_grad``, ``nn.Conv2d``, ``nn.ConvTranspose2d``,
``nn.BatchNorm2d``, ``nn.functional.conv2d`` / ``conv_transpose2d`` / ``batch_norm``.
``.cuda()`` moves data into device arrays owned through ``libtortto_hip.so``; every computation
on them runs in hand-written HIP kernels.  Importing this package does not touch the GPU.
"""
__version__ = '0.1.0'

import numpy as np

from .xparray import nparray, hiparray
from .tensor import Tensor, float16, float32, float64, int16, int32, int64
from .VariableFunctions import (manual_seed, empty, zeros, ones, randn, tensor, transpose, swapaxes, swapdims,
                                mean, flatten, mm, matmul)
from .autograd import (no_grad, enable_grad, set_grad_enabled, is_grad_enabled, Function, AccumulateGrad,
                       ToCopy, Add, Convolution, TransposedConvolution, BatchNorm, Relu, LeakyRelu,
                       MaxPool2DWithIndices, LogSoftmax, NllLoss, View, Transpose, Mm, Mean)
from .serialization import save, load
from . import nn
from . import optim
from . import _hip

cparray = hiparray   # the reference's name for "the device array class"


class cuda:
    """``tt.cuda`` helpers."""

    @staticmethod
    def is_available():
        return _hip.is_available()

    @staticmethod
    def synchronize():
        _hip.synchronize()

    @staticmethod
    def set_conv_math(mode):
        """Not in the reference (float32 throughout): ``'f32'`` (default), ``'bf16'`` -- the three
        convolution passes with operands rounded to bfloat16 inside the kernels and float32
        accumulation; tensors stay float32, results then differ from the float32 path by a few 1e-3
        of their magnitude -- or ``'bf16x3'``: float32 arithmetic carried out on the bf16 matrix
        instructions (three exact bf16 terms per operand element), which meets the float32 path's
        tolerances and is faster on layers with at least one tile per compute unit."""
        _hip.set_conv_math(mode)

    @staticmethod
    def get_conv_math():
        return _hip.get_conv_math()
