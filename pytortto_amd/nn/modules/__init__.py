from .module import Module
from .conv import Conv2d, ConvTranspose2d
from .batchnorm import BatchNorm1d, BatchNorm2d, BatchNorm3d
from .container import Sequential
from .activation import LeakyReLU, LogSoftmax, ReLU
from .head import Identity, Linear, MaxPool2d, NLLLoss

__all__ = ['Module', 'Conv2d', 'ConvTranspose2d', 'BatchNorm1d', 'BatchNorm2d', 'BatchNorm3d', 'Sequential', 'ReLU',
           'LeakyReLU', 'MaxPool2d', 'LogSoftmax', 'Identity', 'Linear', 'NLLLoss']
