"""The hot-path autograd functions with the reference's names, arguments and error behaviour
(``src/tortto/autograd/grad_nn.py``): ``Convolution`` (:684-734), ``TransposedConvolution``
(:737-779), ``BatchNorm`` (:907-989), ``Relu`` (:33-69), ``LeakyRelu`` (:71-95) and
``MaxPool2DWithIndices`` (:826-864), ``LogSoftmax`` (:373-392), ``NllLoss`` (:287-349).

Where the reference evaluates NumPy/CuPy expressions, these call ``libtortto_hip.so`` through
``pytortto_amd.ops``.  Only device tensors (``hiparray``) are computed here: host tensors stay
with tortto's own NumPy path, and are refused rather than silently computed some other way.
"""
import math
from math import prod

import numpy as np

from .. import _hip, ops
from ..xparray import hiparray
from .function import Function
from .helper import build_links, inplace_precheck, inplace_update


def _device_only(name, data):
    if data.__class__ is not hiparray:
        raise RuntimeError(f'{name}: pytortto_amd implements the device (HIP) path only and got a host '
                           f'{data.__class__.__name__}; move the tensors with .cuda() first '
                           f'(host tensors belong to tortto\'s NumPy path)')


class Convolution(Function):
    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, xt1, xt2 = inputs   # input, weight, bias
        xd0, xd1 = xt0.data, xt1.data
        xd2 = None if xt2 is None else xt2.data
        stride, padding = params['stride'], params['padding']
        dilation, groups = params['dilation'], params['groups']
        if xd0.__class__ is not xd1.__class__:
            raise RuntimeError(f'Input type ({xd0.__class__.__name__}) and weight type '
                               f'({xd1.__class__.__name__}) should be the same')
        if xd2 is not None and xd0.__class__ is not xd2.__class__:
            raise RuntimeError(f'Input type ({xd0.__class__.__name__}) and bias type '
                               f'({xd2.__class__.__name__}) should be the same')
        if xd0.ndim != 4:
            raise RuntimeError(f'Expected 3D (unbatched) or 4D (batched) input to conv2d, '
                               f'but got input of size: {xd0.shape}')
        if groups * xd1.shape[-3] != xd0.shape[-3]:
            raise RuntimeError(f'Given groups={groups}, weight of size {xd1.shape}, '
                               f'expected input{xd0.shape} to have {groups * xd1.shape[-3]} channels, '
                               f'but got {xd0.shape[-3]} channels instead')
        _device_only('Convolution', xd0)
        yd0 = ops.conv2d_fwd(xd0, xd1, xd2, stride, padding, dilation, groups)
        yt0 = build_links(yd0, grad_fn=ctx)
        # the reference also keeps a zero-padded copy of the input for the weight gradient
        # (grad_nn.py:714); the kernels address padding implicitly, so the input itself suffices
        ctx.save_for_backward(xt0, xt1)
        return yt0

    @staticmethod
    def backward(ctx, *grad_outputs):
        gd0, = grad_outputs
        xd0, xd1 = ctx.saved_tensors
        stride, padding = ctx.params['stride'], ctx.params['padding']
        dilation, groups = ctx.params['dilation'], ctx.params['groups']
        grad0 = grad1 = grad2 = None
        if ctx.needs_input_grad[2]:
            grad2 = ops.channel_sum(gd0)
        if ctx.needs_input_grad[1]:
            grad1 = ops.conv2d_wgrad(xd0, gd0, xd1.shape, stride, padding, dilation, groups)
        if ctx.needs_input_grad[0]:
            grad0 = ops.conv2d_dgrad(gd0, xd1, None, xd0.shape[-2:], stride, padding, dilation, groups)
        return grad0, grad1, grad2


class TransposedConvolution(Function):
    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, xt1, xt2 = inputs   # input, weight [C_in, C_out/groups, R, S], bias
        xd0, xd1 = xt0.data, xt1.data
        stride, padding = params['stride'], params['padding']
        dilation, groups = params['dilation'], params['groups']
        output_padding = params['output_padding']
        if xd0.ndim != 4:
            raise RuntimeError(f'Expected 3D (unbatched) or 4D (batched) input to conv_transpose2d, '
                               f'but got input of size: {xd0.shape}')
        if xd1.shape[-4] != xd0.shape[-3]:
            raise RuntimeError(f'Given transposed=1, weight of size {xd1.shape}, '
                               f'expected input {xd0.shape} to have {xd1.shape[-4]} channels, '
                               f'but got {xd0.shape[-3]} channels instead')
        _device_only('TransposedConvolution', xd0)
        _device_only('TransposedConvolution', xd1)
        oph = output_padding[0]
        opw = oph if len(output_padding) == 1 else output_padding[1]
        r, s = xd1.shape[-2:]
        hy = (xd0.shape[-2] - 1) * stride[0] - 2 * padding[0] + dilation[0] * (r - 1) + oph + 1
        wy = (xd0.shape[-1] - 1) * stride[1] - 2 * padding[1] + dilation[1] * (s - 1) + opw + 1
        # the forward pass is the input gradient of the convolution that has this weight
        yd0 = ops.conv2d_dgrad(xd0, xd1, None if xt2 is None else xt2.data, (hy, wy),
                               stride, padding, dilation, groups)
        yt0 = build_links(yd0, grad_fn=ctx)
        ctx.save_for_backward(xt0, xt1)
        return yt0

    @staticmethod
    def backward(ctx, *grad_outputs):
        gd0, = grad_outputs
        xd0, xd1 = ctx.saved_tensors
        stride, padding = ctx.params['stride'], ctx.params['padding']
        dilation, groups = ctx.params['dilation'], ctx.params['groups']
        grad0 = grad1 = grad2 = None
        if ctx.needs_input_grad[2]:
            grad2 = ops.channel_sum(gd0)
        if ctx.needs_input_grad[1]:
            grad1 = ops.conv2d_wgrad(gd0, xd0, xd1.shape, stride, padding, dilation, groups)
        if ctx.needs_input_grad[0]:
            # Always the padded convolution.  The reference drops the padding here when the
            # weight needs no gradient (grad_nn.py:778), which is wrong for padding != 0.
            grad0 = ops.conv2d_fwd(gd0, xd1, None, stride, padding, dilation, groups)
        return grad0, grad1, grad2


def _verify_batch_size(size):
    """grad_nn.py:899-904"""
    if prod((size[0],) + tuple(size[2:])) == 1:
        raise ValueError(f'Expected more than 1 value per channel when training, got input size {size}')


class BatchNorm(Function):
    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, xt1, xt2 = inputs   # input, weight, bias
        xd0 = xt0.data
        running_mean, running_var = params['running_mean'], params['running_var']
        training, momentum, eps = params['training'], params['momentum'], params['eps']
        _device_only('BatchNorm', xd0)
        gamma = None if xt1 is None else xt1.data
        beta = None if xt2 is None else xt2.data
        have_running = running_mean is not None and running_var is not None
        cshape = (xd0.shape[1],) + (1,) * (xd0.ndim - 2)
        count_batch = params.get('count_batch')
        if training:
            _verify_batch_size(xd0.shape)
            # the launch is parked: a ReLU that comes next absorbs it (one pass over the tensor
            # instead of two), anything else triggers it as it is
            yd0, mean, var_eps, sd, new_rm, new_rv = ops.bn_fwd_train_deferred(
                xd0, gamma, beta, running_mean.data if have_running else None,
                running_var.data if have_running else None, momentum, eps,
                num_batches_tracked=None if count_batch is None else count_batch.data)
            if have_running:            # the buffers are re-bound to new arrays (grad_nn.py:929-930)
                running_mean.data = new_rm
                running_var.data = new_rv
        elif have_running:
            yd0, mean, var_eps, sd = ops.bn_fwd_eval(xd0, gamma, beta, running_mean.data, running_var.data, eps)
        elif xd0.size == xd0.shape[1]:
            # eval mode without buffers and one value per channel: the batch statistics are the value
            # itself and zero (grad_nn.py:935-937); only training refuses this shape (:921-922)
            yd0, mean, var_eps, sd = ops.bn_fwd_eval(xd0, gamma, beta, xd0.reshape((xd0.shape[1],)),
                                                     hiparray(np.zeros(xd0.shape[1], np.float32)), eps)
        else:
            yd0, mean, var_eps, sd, _, _ = ops.bn_fwd_train(xd0, gamma, beta, None, None, 0.0, eps)
        yt0 = build_links(yd0, grad_fn=ctx)
        ctx.save_for_backward(xt0, xt1)
        ctx.params = {'axis': (0,) + tuple(range(2, xd0.ndim)), 'shape': (xd0.shape[0],) + xd0.shape[2:],
                      'mean': mean.reshape(cshape), 'var': var_eps.reshape(cshape), 'sd': sd.reshape(cshape)}
        return yt0

    @staticmethod
    def backward(ctx, *grad_outputs):
        gd0, = grad_outputs
        xd0, xd1 = ctx.saved_tensors
        p = ctx.params
        parked = _hip.take_pending_if(lambda op: op.__class__ is ops.DeferredReluBackward and op.out._buf is gd0._buf)
        if parked is not None:
            # the gradient comes straight from a ReLU whose mask has not been applied yet: apply it
            # while reading dy (grad_nn.py:67 folded into :977-988)
            return ops.bn_relu_bwd(xd0, parked.dy, parked.y, xd1, p['mean'], p['var'], p['sd'],
                                   need=ctx.needs_input_grad)
        grad0, grad1, grad2 = ops.bn_bwd(xd0, gd0, xd1, p['mean'], p['var'], p['sd'], need=ctx.needs_input_grad)
        return grad0, grad1, grad2


class Relu(Function):
    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, = inputs
        xd0 = xt0.data
        inplace = params['inplace']
        # only a device input can be the output of a parked device operation (a host array has no buffer)
        parked = None
        if xd0.__class__ is hiparray:
            parked = _hip.take_pending_if(lambda op: (op.__class__ is ops.DeferredBatchNorm and op.y._buf is xd0._buf)
                                          or (op.__class__ is ops.DeferredAdd and op.out._buf is xd0._buf))
        if parked is not None:
            # the input is a BatchNorm output, or a residual sum, that has not been launched yet: one
            # kernel writes maximum(bn(x), 0) (grad_nn.py:942-959 and :56 in one pass) or maximum(a + b, 0)
            if inplace:
                try:
                    inplace_precheck(xt0)
                except RuntimeError:
                    parked.run()
                    raise
                parked.run_with_relu()
                yt0 = inplace_update(xt0, ctx)
            else:
                yt0 = build_links(parked.run_with_relu(hiparray.empty(xd0.shape)), grad_fn=ctx)
            if parked.__class__ is ops.DeferredBatchNorm:
                ctx.params['after_batch_norm'] = True
        elif xd0.__class__ is hiparray:
            if inplace:
                inplace_precheck(xt0)
                ops.relu_fwd(xd0, out=xd0)
                yt0 = inplace_update(xt0, ctx)
            else:
                yt0 = build_links(ops.relu_fwd(xd0), grad_fn=ctx)
        elif inplace:
            inplace_precheck(xt0)
            np.maximum(xd0, 0, out=xd0)
            yt0 = inplace_update(xt0, ctx)
        else:
            yt0 = build_links(np.maximum(xd0, 0), grad_fn=ctx)
        ctx.save_for_backward(yt0)
        return yt0

    @staticmethod
    def backward(ctx, *grad_outputs):
        gd0, = grad_outputs
        yd0, = ctx.saved_tensors
        if yd0.__class__ is hiparray:
            if ctx.params.get('after_batch_norm') and gd0.__class__ is hiparray:
                # the BatchNorm backward that follows can apply the mask itself; parked until then
                return ops.relu_bwd_deferred(gd0, yd0)
            return ops.relu_bwd(gd0, yd0)
        return gd0 * (yd0 > 0)


class LeakyRelu(Function):
    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, = inputs
        xd0 = xt0.data
        inplace = params['inplace']
        negative_slope = params['negative_slope']
        if xd0.__class__ is hiparray:
            if inplace:
                inplace_precheck(xt0)
                ops.leaky_relu_fwd(xd0, negative_slope, out=xd0)
                yt0 = inplace_update(xt0, ctx)
            else:
                yt0 = build_links(ops.leaky_relu_fwd(xd0, negative_slope), grad_fn=ctx)
        elif inplace:
            inplace_precheck(xt0)
            np.maximum(xd0 * negative_slope, xd0, out=xd0)
            yt0 = inplace_update(xt0, ctx)
        else:
            yt0 = build_links(np.maximum(xd0 * negative_slope, xd0), grad_fn=ctx)
        ctx.save_for_backward(xt0)
        return yt0

    @staticmethod
    def backward(ctx, *grad_outputs):
        # the reference scales the incoming gradient array in place and hands it on (:94-95)
        gd0, = grad_outputs
        xd0, = ctx.saved_tensors
        negative_slope = ctx.params['negative_slope']
        if xd0.__class__ is hiparray:
            return ops.leaky_relu_bwd(gd0, xd0, negative_slope, out=gd0)
        gd0[xd0 < 0] *= negative_slope
        return gd0


def pool_output_size(size, k, stride, pad, dil, ceil_mode):
    """Window count along one axis (``_sliding_window_view``, :565-579): floor rule, or the ceil
    rule less the last window when it would start beyond the input and its leading padding."""
    span = size + 2 * pad - dil * (k - 1) - 1
    if not ceil_mode:
        return math.floor(span / stride + 1)
    out = math.ceil(span / stride + 1)
    extra = (out - 1) * stride - span
    if extra + pad >= (k - 1) * dil + 1:
        out -= 1
    return out


def _reference_pos(tap, kw):
    """The index tuple the reference returns for ``return_indices=True`` (:787-803), as host arrays:
    aranges over (N, P, Q, C) and, per window, the kernel row and kernel column of its maximum."""
    t = tap.get().reshape((-1,) + tap.shape[-3:])      # [N,C,P,Q]; a 3-D input counts as N = 1
    t = np.moveaxis(t, 1, -1).astype(np.int64)         # [N,P,Q,C]
    n, p, q, c = t.shape
    return (np.arange(n)[:, None, None, None], np.arange(p)[None, :, None, None],
            np.arange(q)[None, None, :, None], np.arange(c)[None, None, None, :], t // kw, t % kw)


class MaxPool2DWithIndices(Function):
    @staticmethod
    def forward(ctx, *inputs, **params):
        (xt0,), xd0 = inputs, inputs[0].data
        kernel_size, stride, padding, dilation, ceil_mode, return_indices = (
            params[name] for name in ('kernel_size', 'stride', 'padding', 'dilation', 'ceil_mode', 'return_indices'))
        (kh, kw), (pad_h, pad_w) = kernel_size, padding
        if 2 * pad_h > kh or 2 * pad_w > kw:        # the reference's two checks and messages (grad_nn.py:835-845)
            raise RuntimeError(f'pad should be smaller than or equal to half of kernel size, '
                               f'but got padW = {pad_w}, padH = {pad_h}, kW = {kw}, kH = {kh}')
        if xd0.ndim not in (3, 4):
            raise RuntimeError('non-empty 3D or 4D (batch mode) tensor expected for input')
        _device_only('max_pool2d', xd0)
        out_hw = tuple(pool_output_size(xd0.shape[-2 + a], kernel_size[a], stride[a], padding[a], dilation[a],
                                        ceil_mode) for a in (0, 1))
        yd0, tap = ops.maxpool2d_fwd(xd0, out_hw, kernel_size, stride, padding, dilation)
        yt0 = build_links(yd0, grad_fn=ctx)
        ctx.save_for_backward(xt0)
        ctx.params['pos'] = tap
        return (yt0, _reference_pos(tap, kernel_size[1])) if return_indices else yt0

    @staticmethod
    def backward(ctx, *grad_outputs):
        gd0, *_ = grad_outputs
        xd0, = ctx.saved_tensors
        p = ctx.params
        return ops.maxpool2d_bwd(gd0, p['pos'], xd0.shape[-2:], p['kernel_size'], p['stride'], p['padding'],
                                 p['dilation'])


class LogSoftmax(Function):
    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, = inputs
        xd0 = xt0.data
        dim = params['dim']
        if xd0.__class__ is hiparray:
            if dim % xd0.ndim != xd0.ndim - 1:
                raise RuntimeError(f'device log_softmax reduces the last dimension only, got dim={dim} for shape '
                                   f'{xd0.shape}')
            yd0 = ops.log_softmax_fwd(xd0)
        else:
            aug = xd0 - np.max(xd0, axis=dim, keepdims=True)
            yd0 = aug - np.log(np.sum(np.exp(aug), axis=dim, keepdims=True))
        yt0 = build_links(yd0, grad_fn=ctx)
        ctx.save_for_backward(yt0)
        return yt0

    @staticmethod
    def backward(ctx, *grad_outputs):
        gd0, = grad_outputs
        dim = ctx.params['dim']
        yd0, = ctx.saved_tensors
        if yd0.__class__ is hiparray:
            return ops.log_softmax_bwd(gd0, yd0)
        return gd0 - gd0.sum(axis=dim, keepdims=True) * np.exp(yd0)


class NllLoss(Function):
    """Device tensors only: logp [N, C] with an int64 target [N] (the classification head)."""

    @staticmethod
    def forward(ctx, *inputs, **params):
        xt0, = inputs
        xt1 = params['target']
        xd0, xd1 = xt0.data, xt1.data
        reduction = params['reduction']
        weight = params['weight']
        ignore_index = params['ignore_index']
        _device_only('nll_loss', xd0)
        if xd1.__class__ is not hiparray or (weight is not None and weight.data.__class__ is not hiparray):
            raise RuntimeError('Expected all tensors to be on the same device')
        yd0, count = ops.nll_loss_fwd(xd0, xd1, None if weight is None else weight.data, ignore_index, reduction)
        ctx.params['N'] = count
        yt0 = build_links(yd0, grad_fn=ctx)
        ctx.save_for_backward(xt0, xt1, weight)
        return yt0

    @staticmethod
    def backward(ctx, *grad_outputs):
        gd0, = grad_outputs
        p = ctx.params
        xd0, xd1, w = ctx.saved_tensors
        return ops.nll_loss_bwd(gd0, xd0.shape, xd1, w, p['N'], p['ignore_index'], p['reduction'])
