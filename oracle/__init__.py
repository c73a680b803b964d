"""CPU oracle for the convolution / BatchNorm path -- TEST INFRASTRUCTURE ONLY.

This package is a NumPy restatement of the reference's CPU algorithm
(``src/tortto/autograd/grad_nn.py`` in samrere/pytortto 1.3.4).  It is the checker the
GPU kernels are compared against and the CPU baseline that ``bench.py`` times; it is
never part of the product path.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it -- ``pytortto_amd`` must not.

How each function is pinned (none of this needed an import of the reference, which
publishes no golden vectors for this path):

* ``conv2d``            brute-force nested loops, float64 evaluation, torch CPU ``F.conv2d``
* ``conv2d_backward_x`` adjoint identity <conv(x,w),g> = <x,dgrad(g,w)> in float64,
                        brute force, torch autograd (incl. uncovered bottom/right rows)
* ``conv2d_backward_w`` adjoint identity <conv(x,w),g> = <w,wgrad(x,g)>, torch autograd
* ``conv_transpose2d``  definition as dgrad of conv, torch CPU ``F.conv_transpose2d``
                        (incl. ``output_padding``), adjointness with ``conv2d``
* ``batch_norm_*``      closed forms (mean(y)=beta, var(y)=gamma^2 var/(var+eps)),
                        running-stat recurrence, sum(dx)=0, sum(dx*xhat)=0,
                        torch CPU ``F.batch_norm`` + autograd, float64 finite differences

* ``max_pool2d*``       nested-loop brute force with sequential assignment (last window wins),
                        torch CPU ``F.max_pool2d`` (forward always; backward where windows do
                        not overlap, so that assignment and summation coincide)
* ``relu*/leaky_relu*`` closed forms on signs / zero / NaN, torch CPU with autograd
* ``mean_*``, ``mm_*``, ``linear_*``, ``log_softmax_*``, ``nll_loss_*``
                        torch CPU functions with autograd (weights, ignore_index, reductions),
                        closed forms (normalisation, zero-sum gradient rows, g / count)
* ``optim.sgd``, ``optim.adam``
                        torch CPU optimisers over several steps, closed forms

The checks live in ``tests/test_oracle_*.py``.
"""
from .conv import (conv2d, conv2d_backward_w, conv2d_backward_x, conv_output_size,
                   conv_transpose_output_size, convolution_forward, convolution_backward,
                   transposed_convolution_forward, transposed_convolution_backward)
from .batchnorm import batch_norm_forward, batch_norm_backward
from .nninit import conv_parameters, bn_affine_c4
from .pool import max_pool2d, max_pool2d_backward, pool_output_size
from .head import (mean_forward, mean_backward, mm_forward, mm_backward, linear_forward, linear_backward,
                   log_softmax_forward, log_softmax_backward, nll_loss_forward, nll_loss_backward)
from . import optim
from .activation import relu_forward, relu_backward, leaky_relu_forward, leaky_relu_backward

__all__ = [
    'conv2d', 'conv2d_backward_w', 'conv2d_backward_x', 'conv_output_size',
    'conv_transpose_output_size', 'convolution_forward', 'convolution_backward',
    'transposed_convolution_forward', 'transposed_convolution_backward',
    'batch_norm_forward', 'batch_norm_backward', 'conv_parameters', 'bn_affine_c4',
    'max_pool2d', 'max_pool2d_backward', 'pool_output_size',
    'optim',
    'relu_forward', 'relu_backward', 'leaky_relu_forward', 'leaky_relu_backward',
    'mean_forward', 'mean_backward', 'mm_forward', 'mm_backward', 'linear_forward', 'linear_backward',
    'log_softmax_forward', 'log_softmax_backward', 'nll_loss_forward', 'nll_loss_backward',
]
