"""``BatchNorm2d`` (and the 1d/3d input checks) as in ``src/tortto/nn/modules/batchnorm.py``:
gamma=1, beta=0, running_mean=0, running_var=1, ``num_batches_tracked`` a float32 scalar tensor;
``momentum=None`` switches to a cumulative moving average."""
from ... import VariableFunctions as _vf
from ...tensor import Tensor
from .. import functional as F
from .. import init
from ..parameter import Parameter
from .module import Module


class _NormBase(Module):
    def __init__(self, num_features, eps=1e-5, momentum=0.1, affine=True, track_running_stats=True):
        super().__init__()
        self.num_features = num_features
        self.eps = eps
        self.momentum = momentum
        self.affine = affine
        self.track_running_stats = track_running_stats
        if self.affine:
            self.weight = Parameter(_vf.ones(num_features))
            self.bias = Parameter(_vf.zeros(num_features))
        else:
            self.register_parameter('weight', None)
            self.register_parameter('bias', None)
        if self.track_running_stats:
            self.register_buffer('running_mean', _vf.zeros(num_features))
            self.register_buffer('running_var', _vf.ones(num_features))
            self.register_buffer('num_batches_tracked', Tensor(0))
        else:
            self.register_parameter('running_mean', None)
            self.register_parameter('running_var', None)
            self.register_parameter('num_batches_tracked', None)
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
        raise NotImplementedError

    def extra_repr(self):
        return ('{num_features}, eps={eps}, momentum={momentum}, affine={affine}, '
                'track_running_stats={track_running_stats}'.format(**self.__dict__))


class _BatchNorm(_NormBase):
    def forward(self, inpt):
        self._check_input_dim(inpt)
        if self.training and self.track_running_stats:
            self.num_batches_tracked.data += 1
            if self.momentum is None:
                factor = 1.0 / self.num_batches_tracked.item()
            else:
                factor = self.momentum
        else:
            factor = None
        bn_training = True if self.training else (self.running_mean is None and self.running_var is None)
        use_buffers = not self.training or self.track_running_stats
        return F.batch_norm(inpt, self.running_mean if use_buffers else None,
                            self.running_var if use_buffers else None,
                            self.weight, self.bias, bn_training, factor, self.eps)


class BatchNorm1d(_BatchNorm):
    def _check_input_dim(self, input):
        if input.dim() != 2 and input.dim() != 3:
            raise ValueError('expected 2D or 3D input (got {}D input)'.format(input.dim()))


class BatchNorm2d(_BatchNorm):
    def _check_input_dim(self, input):
        if input.dim() != 4:
            raise ValueError('expected 4D input (got {}D input)'.format(input.dim()))


class BatchNorm3d(_BatchNorm):
    def _check_input_dim(self, input):
        if input.dim() != 5:
            raise ValueError('expected 5D input (got {}D input)'.format(input.dim()))
