"""Optimiser updates restated from ``src/tortto/optim/_functional.py`` -- TEST INFRASTRUCTURE ONLY.

Each function updates NumPy arrays in place with the reference's own expressions, so that the
float32 roundings (and the float64 denominator of Adam, which comes from dividing a float32
array by the float64 scalar ``np.sqrt(bias_correction2)``) are the reference's.

Pinned by (tests/test_oracle_optim.py): torch CPU ``optim.SGD`` / ``Adam`` / ``AdamW`` over
several steps (momentum, dampening, Nesterov, weight decay, AMSGrad), and closed forms (plain
SGD is p - lr * g; with a constant gradient the momentum buffer is a geometric series; Adam's
first step moves every element by lr * sign(g) up to eps).
"""
import numpy as np


def sgd(params, grads, momentum_bufs, weight_decay, momentum, lr, dampening, nesterov):
    """_functional.py:4-22.  ``momentum_bufs[i]`` is None before the first step."""
    for i, param in enumerate(params):
        d_p = grads[i]
        if weight_decay != 0:
            d_p = d_p + param * weight_decay
        if momentum != 0:
            buf = momentum_bufs[i]
            if buf is None:
                buf = d_p                       # the buffer starts as the gradient array itself (:12-13)
                momentum_bufs[i] = d_p
            else:
                buf *= momentum
                buf += d_p * (1 - dampening)
            if nesterov:
                d_p = d_p + buf * momentum
            else:
                d_p = buf
        param += d_p * -lr


def adam(params, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, steps, amsgrad, beta1, beta2, lr, weight_decay,
         eps, decoupled=False):
    """_functional.py:25-65 (Adam) and :68-119 (AdamW, ``decoupled=True``)."""
    for i, param in enumerate(params):
        grad = grads[i]
        exp_avg, exp_avg_sq, step = exp_avgs[i], exp_avg_sqs[i], steps[i]
        if decoupled:
            param *= 1 - lr * weight_decay
        bias_correction1 = 1 - beta1 ** step
        bias_correction2 = 1 - beta2 ** step
        if weight_decay != 0 and not decoupled:
            grad = grad + param * weight_decay
        exp_avg *= beta1
        exp_avg += (1 - beta1) * grad
        exp_avg_sq *= beta2
        exp_avg_sq += grad * grad.conj() * (1 - beta2)
        if amsgrad:
            np.maximum(max_exp_avg_sqs[i], exp_avg_sq, out=max_exp_avg_sqs[i])
            denom = (np.sqrt(max_exp_avg_sqs[i]) / np.sqrt(bias_correction2)) + eps
        else:
            denom = (np.sqrt(exp_avg_sq) / np.sqrt(bias_correction2)) + eps
        step_size = lr / bias_correction1
        param += -step_size * exp_avg / denom
