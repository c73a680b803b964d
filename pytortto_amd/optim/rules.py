"""``SGD`` (``src/tortto/optim/sgd.py``), ``Adam`` and ``AdamW`` (``adam.py``, ``adamw.py``): argument
checks and per-parameter state of the reference; the arithmetic is one kernel launch per parameter
(``_functional.py`` here)."""
from ..xparray import hiparray
from . import _functional as F
from .optimizer import Optimizer, required


def _check(ok, text, value):
    if not ok:
        raise ValueError(text.format(value))


class SGD(Optimizer):
    def __init__(self, params, lr=required, momentum=0, dampening=0, weight_decay=0, nesterov=False):
        _check(lr is required or lr >= 0.0, 'Invalid learning rate: {}', lr)
        _check(momentum >= 0.0, 'Invalid momentum value: {}', momentum)
        _check(weight_decay >= 0.0, 'Invalid weight_decay value: {}', weight_decay)
        if nesterov and (momentum <= 0 or dampening != 0):
            raise ValueError('Nesterov momentum requires a momentum and zero dampening')
        super().__init__(params, dict(lr=lr, momentum=momentum, dampening=dampening, weight_decay=weight_decay,
                                      nesterov=nesterov))

    def __setstate__(self, state):
        super().__setstate__(state)
        for group in self.param_groups:
            group.setdefault('nesterov', False)

    def step(self):
        for group, members in self._with_grad():
            buffers = [self.state[p].get('momentum_buffer') for p in members]
            F.sgd(members, [p.grad for p in members], buffers, group['weight_decay'], group['momentum'], group['lr'],
                  group['dampening'], group['nesterov'])
            for p, buf in zip(members, buffers):        # created by the first step when momentum != 0
                self.state[p]['momentum_buffer'] = buf


class Adam(Optimizer):
    _rule = staticmethod(F.adam)

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0, amsgrad=False):
        _check(lr >= 0.0, 'Invalid learning rate: {}', lr)
        _check(eps >= 0.0, 'Invalid epsilon value: {}', eps)
        for i in (0, 1):
            _check(0.0 <= betas[i] < 1.0, 'Invalid beta parameter at index %d: {}' % i, betas[i])
        _check(weight_decay >= 0.0, 'Invalid weight_decay value: {}', weight_decay)
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad))

    def __setstate__(self, state):
        super().__setstate__(state)
        for group in self.param_groups:
            group.setdefault('amsgrad', False)

    def _moments(self, p, amsgrad):
        """The parameter's state, created on its first step (adam.py:45-54), with the step advanced."""
        state = self.state[p]
        if not state:
            state['step'] = 0
            names = ('exp_avg', 'exp_avg_sq') + (('max_exp_avg_sq',) if amsgrad else ())
            for name in names:
                state[name] = hiparray.zeros(p.data.shape)
        state['step'] += 1
        return state

    def step(self):
        for group, members in self._with_grad():
            amsgrad = group['amsgrad']
            states = [self._moments(p, amsgrad) for p in members]
            self._rule(members, [p.grad for p in members], [s['exp_avg'] for s in states],
                       [s['exp_avg_sq'] for s in states], [s['max_exp_avg_sq'] for s in states] if amsgrad else [],
                       [s['step'] for s in states], amsgrad, *group['betas'], group['lr'], group['weight_decay'],
                       group['eps'])


class AdamW(Adam):
    _rule = staticmethod(F.adamw)

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, amsgrad=False):
        super().__init__(params, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad)
