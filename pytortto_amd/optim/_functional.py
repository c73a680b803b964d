"""The update rules (``src/tortto/optim/_functional.py``) as one fused kernel launch per parameter.
Device parameters only: host tensors belong to tortto's NumPy path and are refused."""
import numpy as np

from .. import _hip
from ..xparray import hiparray


def _device(param, *arrays):
    for a in (param.data,) + arrays:
        if a is not None and (a.__class__ is not hiparray or a.dtype != np.float32):
            raise RuntimeError('the optimisers of pytortto_amd update float32 device parameters only; move the model '
                               'with .cuda() first')


def sgd(params, d_p_list, momentum_buffer_list, weight_decay, momentum, lr, dampening, nesterov):
    """_functional.py:4-22."""
    for i, param in enumerate(params):
        d_p, buf = d_p_list[i], momentum_buffer_list[i]
        _device(param, d_p, buf)
        first = False
        if momentum != 0 and buf is None:
            buf = hiparray.empty(param.data.shape)      # the kernel stores d_p into it (:12-13)
            momentum_buffer_list[i] = buf
            first = True
        _hip.call('tt_sgd_step_f32', param.data.ptr, d_p.ptr, None if buf is None else buf.ptr, param.data.size,
                  lr, momentum, dampening, weight_decay, int(bool(nesterov)), int(first))


def _adam(params, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, state_steps, amsgrad, beta1, beta2, lr,
          weight_decay, eps, decoupled):
    for i, param in enumerate(params):
        vmax = max_exp_avg_sqs[i] if amsgrad else None
        _device(param, grads[i], exp_avgs[i], exp_avg_sqs[i], vmax)
        _hip.call('tt_adam_step_f32', param.data.ptr, grads[i].ptr, exp_avgs[i].ptr, exp_avg_sqs[i].ptr,
                  None if vmax is None else vmax.ptr, param.data.size, state_steps[i], lr, beta1, beta2, eps,
                  weight_decay, int(bool(amsgrad)), int(decoupled))


def adam(params, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, state_steps, amsgrad, beta1, beta2, lr,
         weight_decay, eps):
    """_functional.py:25-65."""
    _adam(params, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, state_steps, amsgrad, beta1, beta2, lr,
          weight_decay, eps, False)


def adamw(params, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, state_steps, amsgrad, beta1, beta2, lr,
          weight_decay, eps):
    """_functional.py:68-119."""
    _adam(params, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, state_steps, amsgrad, beta1, beta2, lr,
          weight_decay, eps, True)
