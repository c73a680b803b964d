from .grad_mode import no_grad, enable_grad, set_grad_enabled, is_grad_enabled
from .function import Function, BackwardFunction, AccumulateGrad, FunctionBase
from .helper import build_links, toposort, inplace_precheck, inplace_update
from .grad_fcn import ToCopy, Add, Unsqueeze, Squeeze, View, Transpose, Mm, Mean
from .grad_nn import (Convolution, TransposedConvolution, BatchNorm, Relu, LeakyRelu, MaxPool2DWithIndices,
                      LogSoftmax, NllLoss)
