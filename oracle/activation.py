"""ReLU / LeakyReLU restated from ``src/tortto/autograd/grad_nn.py:33-95`` -- TEST INFRASTRUCTURE ONLY.

Pinned by closed forms on hand-picked values (signs, zero, NaN) and torch CPU
``F.relu`` / ``F.leaky_relu`` with autograd (tests/test_oracle_pool.py).
"""
import numpy as np


def relu_forward(x):
    return np.maximum(x, 0)                       # :56 / :59 -- propagates NaN


def relu_backward(grad, y):
    return grad * (y > 0)                         # :67


def leaky_relu_forward(x, negative_slope):
    return np.maximum(x * negative_slope, x)      # :82 / :85


def leaky_relu_backward(grad, x, negative_slope):
    grad = grad.copy()                            # the reference scales `grad` itself in place (:94)
    grad[x < 0] *= negative_slope
    return grad
