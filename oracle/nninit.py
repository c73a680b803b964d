"""Seeded parameter/input generation exactly as the reference's modules draw them
(test infrastructure only).

``manual_seed`` is ``np.random.seed`` (``src/tortto/VariableFunctions.py:8-9``); conv
weights are Kaiming-uniform with ``a=sqrt(5)`` => U(-1/sqrt(fan_in), 1/sqrt(fan_in)) with
``fan_in = weight.shape[1]*R*S`` and the bias uses the same bound
(``nn/modules/conv.py:48-56``, ``nn/init.py:41-52``, ``:91-96``); both are drawn with
``np.random.uniform(...).astype(float32)``, weight first (``nn/init.py:6-10``).
"""
import math

import numpy as np


def conv_parameters(c_in, c_out, ksize, groups=1, bias=True, transposed=False):
    """Draw ``(weight, bias)`` from the legacy global NumPy stream in the reference's order."""
    r, s = ksize
    shape = (c_in, c_out // groups, r, s) if transposed else (c_out, c_in // groups, r, s)
    fan_in = shape[1] * r * s
    gain = math.sqrt(2.0 / (1 + math.sqrt(5) ** 2))   # leaky_relu gain, slope sqrt(5) (init.py:76-77)
    std = gain / math.sqrt(fan_in)                    # same operation order as init.py:93-95
    bound = math.sqrt(3.0) * std
    w = np.random.uniform(low=-bound, high=bound, size=shape).astype(np.float32)
    b = None
    if bias:
        bb = 1 / math.sqrt(fan_in)
        b = np.random.uniform(low=-bb, high=bb, size=(c_out,)).astype(np.float32)
    return w, b


def bn_affine_c4(c):
    """gamma ~ U(0.5, 1.5), beta ~ N(0, 0.1), in that order (BatchNorm benchmark inputs)."""
    gamma = np.random.uniform(0.5, 1.5, size=c).astype(np.float32)
    beta = np.random.normal(0.0, 0.1, size=c).astype(np.float32)
    return gamma, beta
