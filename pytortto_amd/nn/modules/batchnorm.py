"""``BatchNorm1d/2d/3d`` modules with the state and behaviour of
``src/tortto/nn/modules/batchnorm.py`` (:8-57 state, :62-93 forward, :104-107 and siblings for the
input checks): gamma = 1, beta = 0, running_mean = 0, running_var = 1, ``num_batches_tracked`` a
float32 scalar buffer; ``momentum=None`` turns the running statistics into a cumulative average."""
from ... import VariableFunctions as _vf
from ...tensor import Tensor
from .. import functional as F
from .. import init
from ..parameter import Parameter
from .module import Module


class _BatchNorm(Module):
    _input_dims = ()        # admissible input ranks, set by the subclasses

    def __init__(self, num_features, eps=1e-5, momentum=0.1, affine=True, track_running_stats=True):
        super().__init__()
        self.__dict__.update(num_features=num_features, eps=eps, momentum=momentum, affine=affine,
                             track_running_stats=track_running_stats)
        for name, start in (('weight', _vf.ones), ('bias', _vf.zeros)):
            self.register_parameter(name, Parameter(start(num_features)) if affine else None)
        if track_running_stats:
            self.register_buffer('running_mean', _vf.zeros(num_features))
            self.register_buffer('running_var', _vf.ones(num_features))
            self.register_buffer('num_batches_tracked', Tensor(0))
        else:
            for name in ('running_mean', 'running_var', 'num_batches_tracked'):
                self.register_parameter(name, None)
        self.reset_parameters()

    def reset_running_stats(self):
        if self.track_running_stats:
            self.running_mean = init.zeros_(self.running_mean)
            self.running_var = init.ones_(self.running_var)
            self.num_batches_tracked = init.zeros_(self.num_batches_tracked)

    def reset_parameters(self):
        self.reset_running_stats()
        if self.affine:
            init.ones_(self.weight)
            init.zeros_(self.bias)

    def _check_input_dim(self, input):
        if input.dim() not in self._input_dims:
            wanted = ' or '.join(f'{d}D' for d in self._input_dims)
            raise ValueError(f'expected {wanted} input (got {input.dim()}D input)')

    def extra_repr(self):
        return (f'{self.num_features}, eps={self.eps}, momentum={self.momentum}, affine={self.affine}, '
                f'track_running_stats={self.track_running_stats}')

    def forward(self, inpt):
        self._check_input_dim(inpt)
        factor = None                                   # weight of the new batch in the running statistics
        count_batch = None
        if self.training and self.track_running_stats:
            if self.momentum is not None and self.num_batches_tracked.is_cuda and inpt.is_cuda:
                # the counter's `+= 1` (:66) rides along in the training kernel; nothing reads it before
                count_batch = self.num_batches_tracked
                factor = self.momentum
            else:
                self.num_batches_tracked.data += 1      # (:66)
                factor = self.momentum if self.momentum is not None else 1.0 / self.num_batches_tracked.item()
        # batch statistics are used in training mode, and in eval mode when there are no buffers (:75-78)
        no_buffers = self.running_mean is None and self.running_var is None
        batch_stats = self.training or no_buffers
        pass_buffers = self.track_running_stats or not self.training
        return F.batch_norm(inpt, self.running_mean if pass_buffers else None,
                            self.running_var if pass_buffers else None, self.weight, self.bias, batch_stats,
                            factor, self.eps, _count_batch=count_batch)


class BatchNorm1d(_BatchNorm):
    _input_dims = (2, 3)


class BatchNorm2d(_BatchNorm):
    _input_dims = (4,)


class BatchNorm3d(_BatchNorm):
    _input_dims = (5,)
