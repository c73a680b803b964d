"""``Adam`` and ``AdamW`` (``src/tortto/optim/adam.py``, ``adamw.py``)."""
from ..xparray import hiparray
from . import _functional as F
from .optimizer import Optimizer


class Adam(Optimizer):
    _update = staticmethod(F.adam)

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0, amsgrad=False):
        if not 0.0 <= lr:
            raise ValueError('Invalid learning rate: {}'.format(lr))
        if not 0.0 <= eps:
            raise ValueError('Invalid epsilon value: {}'.format(eps))
        if not 0.0 <= betas[0] < 1.0:
            raise ValueError('Invalid beta parameter at index 0: {}'.format(betas[0]))
        if not 0.0 <= betas[1] < 1.0:
            raise ValueError('Invalid beta parameter at index 1: {}'.format(betas[1]))
        if not 0.0 <= weight_decay:
            raise ValueError('Invalid weight_decay value: {}'.format(weight_decay))
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad))

    def __setstate__(self, state):
        super().__setstate__(state)
        for group in self.param_groups:
            group.setdefault('amsgrad', False)

    def step(self):
        for group in self.param_groups:
            with_grad, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, steps = [], [], [], [], [], []
            beta1, beta2 = group['betas']
            for p in group['params']:
                if p.grad is None:
                    continue
                with_grad.append(p)
                grads.append(p.grad)
                state = self.state[p]
                if len(state) == 0:                      # lazy state initialisation (adam.py:45-54)
                    state['step'] = 0
                    state['exp_avg'] = hiparray.zeros(p.data.shape)
                    state['exp_avg_sq'] = hiparray.zeros(p.data.shape)
                    if group['amsgrad']:
                        state['max_exp_avg_sq'] = hiparray.zeros(p.data.shape)
                exp_avgs.append(state['exp_avg'])
                exp_avg_sqs.append(state['exp_avg_sq'])
                if group['amsgrad']:
                    max_exp_avg_sqs.append(state['max_exp_avg_sq'])
                state['step'] += 1
                steps.append(state['step'])
            self._update(with_grad, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, steps, group['amsgrad'], beta1,
                         beta2, group['lr'], group['weight_decay'], group['eps'])


class AdamW(Adam):
    _update = staticmethod(F.adamw)

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, amsgrad=False):
        super().__init__(params, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad)
