"""The update rules (``src/tortto/optim/_functional.py``) as fused kernels, a group's parameters in a few launches.
Device parameters only: host tensors belong to tortto's NumPy path and are refused."""
import ctypes

import numpy as np

from .. import _hip
from ..xparray import hiparray


def _device(param, *arrays):
    for a in (param.data,) + arrays:
        if a is not None and (a.__class__ is not hiparray or a.dtype != np.float32):
            raise RuntimeError('the optimisers of pytortto_amd update float32 device parameters only; move the model '
                               'with .cuda() first')


def sgd(params, d_p_list, momentum_buffer_list, weight_decay, momentum, lr, dampening, nesterov):
    """_functional.py:4-22, all parameters of the group in one call (a few launches)."""
    count = len(params)
    if count == 0:
        return
    first = [0] * count
    for i, param in enumerate(params):
        _device(param, d_p_list[i], momentum_buffer_list[i])
        if momentum != 0 and momentum_buffer_list[i] is None:
            momentum_buffer_list[i] = hiparray.empty(param.data.shape)      # the kernel stores d_p into it (:12-13)
            first[i] = 1
    for param in params:            # written in place: nothing may still depend on the old values
        param.data.own()
    pointers = ctypes.c_void_p * count
    bufs = pointers(*[None if b is None else b.ptr for b in momentum_buffer_list])
    _hip.call('tt_sgd_step_multi_f32', count, pointers(*[p.data.ptr for p in params]),
              pointers(*[g.ptr for g in d_p_list]), bufs, (ctypes.c_size_t * count)(*[p.data.size for p in params]),
              (ctypes.c_int * count)(*first), lr, momentum, dampening, weight_decay, int(bool(nesterov)))


def _adam(params, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, state_steps, amsgrad, beta1, beta2, lr,
          weight_decay, eps, decoupled):
    count = len(params)
    if count == 0:
        return
    for i, param in enumerate(params):
        _device(param, grads[i], exp_avgs[i], exp_avg_sqs[i], max_exp_avg_sqs[i] if amsgrad else None)
    for param in params:            # written in place: nothing may still depend on the old values
        param.data.own()
    pointers = ctypes.c_void_p * count
    vmax = pointers(*[a.ptr for a in max_exp_avg_sqs]) if amsgrad else None
    _hip.call('tt_adam_step_multi_f32', count, pointers(*[p.data.ptr for p in params]),
              pointers(*[g.ptr for g in grads]), pointers(*[a.ptr for a in exp_avgs]),
              pointers(*[a.ptr for a in exp_avg_sqs]), vmax, (ctypes.c_size_t * count)(*[p.data.size for p in params]),
              (ctypes.c_int * count)(*state_steps), lr, beta1, beta2, eps, weight_decay, int(bool(amsgrad)),
              int(decoupled))


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
