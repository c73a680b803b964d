"""``SGD`` (``src/tortto/optim/sgd.py``)."""
from . import _functional as F
from .optimizer import Optimizer, required


class SGD(Optimizer):
    def __init__(self, params, lr=required, momentum=0, dampening=0, weight_decay=0, nesterov=False):
        if lr is not required and lr < 0.0:
            raise ValueError('Invalid learning rate: {}'.format(lr))
        if momentum < 0.0:
            raise ValueError('Invalid momentum value: {}'.format(momentum))
        if weight_decay < 0.0:
            raise ValueError('Invalid weight_decay value: {}'.format(weight_decay))
        defaults = dict(lr=lr, momentum=momentum, dampening=dampening, weight_decay=weight_decay, nesterov=nesterov)
        if nesterov and (momentum <= 0 or dampening != 0):
            raise ValueError('Nesterov momentum requires a momentum and zero dampening')
        super().__init__(params, defaults)

    def __setstate__(self, state):
        super().__setstate__(state)
        for group in self.param_groups:
            group.setdefault('nesterov', False)

    def step(self):
        for group in self.param_groups:
            with_grad, grads, bufs = [], [], []
            for p in group['params']:
                if p.grad is None or p.grad.__class__ is int:      # no gradient arrived for this parameter
                    continue
                with_grad.append(p)
                grads.append(p.grad)
                bufs.append(self.state[p].get('momentum_buffer'))
            F.sgd(with_grad, grads, bufs, group['weight_decay'], group['momentum'], group['lr'], group['dampening'],
                  group['nesterov'])
            for p, buf in zip(with_grad, bufs):
                self.state[p]['momentum_buffer'] = buf
