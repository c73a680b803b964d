"""GPU: the PreAct-ResNet-18 basic-block stack (conv3x3 3->64, stages (64, 128, 256, 512) of two
blocks, block = BN-ReLU -> [conv3x3(stride) - BN - ReLU - conv3x3] + shortcut, identity or 1x1
stride-2 convolution on the block input, no biases, BatchNorm in training mode) at batch 8 through
the module API on the device, against the same stack composed from oracle calls.

Twenty convolutions and seventeen BatchNorm/ReLU pairs compound rounding differences, so the
criterion is the one of the other stack test: every tensor of the device path must be as close to a
float64 evaluation of the stack as the float32 oracle is.  ReLU's gradient is discontinuous: where a
pre-activation lies within rounding distance of zero, two correct float32 evaluations may mask
differently and the gradients then differ by a whole element.  The oracle's backward pass therefore
takes the device's masks -- after checking that every element where a device mask differs from the
float64 one has a pre-activation within 1e-4 of zero relative to the layer's magnitude, and that
there are next to none of them: a mask that is wrong anywhere else fails the test.
"""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

STAGES = ((64, 1), (128, 2), (256, 2), (512, 2))
BATCH = 8


def _build():
    import pytortto_amd as tt
    from pytortto_amd import nn
    tt.manual_seed(3)
    stem = nn.Conv2d(3, 64, 3, 1, 1, bias=False)
    blocks, cin = [], 64
    for cout, stride in STAGES:
        for s, ci in ((stride, cin), (1, cout)):
            blk = {'bn1': nn.BatchNorm2d(ci), 'conv1': nn.Conv2d(ci, cout, 3, s, 1, bias=False),
                   'bn2': nn.BatchNorm2d(cout), 'conv2': nn.Conv2d(cout, cout, 3, 1, 1, bias=False),
                   'short': None if s == 1 and ci == cout else nn.Conv2d(ci, cout, 1, s, bias=False), 'stride': s}
            for key in ('bn1', 'bn2'):     # affine parameters away from their (1, 0) initial values
                c = blk[key].num_features
                blk[key].weight.data[...] = np.random.uniform(0.5, 1.5, c).astype(np.float32)
                blk[key].bias.data[...] = (0.1 * np.random.randn(c)).astype(np.float32)
            blocks.append(blk)
        cin = cout
    return stem, blocks


def _host(t):
    return np.asarray(t.data).copy()


def test_preact_resnet18_stack_matches_oracle_composition():
    import pytortto_amd as tt
    from pytortto_amd import nn
    F = nn.functional
    stem, blocks = _build()
    x = np.random.randn(BATCH, 3, 32, 32).astype(np.float32)
    g = np.random.randn(BATCH, 512, 4, 4).astype(np.float32)
    w0 = _host(stem.weight)
    params = [{k: _host(getattr(b[k], 'weight')) for k in ('conv1', 'conv2')} |
              {'ws': None if b['short'] is None else _host(b['short'].weight),
               'g1': _host(b['bn1'].weight), 'b1': _host(b['bn1'].bias),
               'g2': _host(b['bn2'].weight), 'b2': _host(b['bn2'].bias), 'stride': b['stride']} for b in blocks]

    # ---- device: forward (keeping every ReLU output for its mask) and backward ---------------------
    stem.cuda()
    for b in blocks:
        for k in ('bn1', 'conv1', 'bn2', 'conv2', 'short'):
            if b[k] is not None:
                b[k].cuda()
    xt = tt.tensor(x, requires_grad=True)
    a = stem(xt.cuda())
    relu_outputs = []
    for b in blocks:
        r1 = F.relu(b['bn1'](a))
        r2 = F.relu(b['bn2'](b['conv1'](r1)))
        relu_outputs += [r1, r2]
        a = b['conv2'](r2) + (a if b['short'] is None else b['short'](a))
    out = a
    out.backward(tt.tensor(g).cuda())
    device_masks = [r.cpu().detach().numpy() > 0 for r in relu_outputs]
    del relu_outputs

    # ---- oracle: the same stack, forward and backward, in float32 and float64 ---------------------
    def oracle_stack(dtype, check_masks):
        one = (1, 1)
        cast = lambda v: None if v is None else v.astype(dtype)
        a, _ = oracle.convolution_forward(x.astype(dtype), cast(w0), None, one, one, one, 1)
        tape, masks = [], iter(device_masks)

        def bn_relu(t, gamma, beta):
            y, saved, _, _ = oracle.batch_norm_forward(t, cast(gamma), cast(beta), None, None, True, 0.1, 1e-5)
            mask = next(masks)
            if check_masks:
                differ = (y > 0) != mask
                assert differ.mean() < 1e-4, 'ReLU masks of device and oracle disagree beyond rounding'
                if differ.any():
                    assert np.abs(y[differ]).max() <= 1e-4 * np.abs(y).max(), \
                        'a device ReLU mask differs where the pre-activation is not within rounding distance of zero'
            return np.maximum(y, 0), saved, mask       # the forward pass is the oracle's own; `mask` serves the backward pass

        for p in params:
            st = (p['stride'],) * 2
            r1, s1, m1 = bn_relu(a, p['g1'], p['b1'])
            c1, r1pad = oracle.convolution_forward(r1, cast(p['conv1']), None, st, one, one, 1)
            r2, s2, m2 = bn_relu(c1, p['g2'], p['b2'])
            c2, r2pad = oracle.convolution_forward(r2, cast(p['conv2']), None, one, one, one, 1)
            if p['ws'] is None:
                sc, apad = a, None
            else:
                sc, apad = oracle.convolution_forward(a, cast(p['ws']), None, st, (0, 0), one, 1)
            tape.append((p, a, apad, s1, m1, r1, r1pad, c1, s2, m2, r2, r2pad))
            a = c2 + sc
        grad, grads = g.astype(dtype), []
        for p, xin, xinpad, s1, m1, r1, r1pad, c1, s2, m2, r2, r2pad in reversed(tape):
            st = (p['stride'],) * 2
            need = (True, True, False)
            d, dw2, _ = oracle.convolution_backward(grad, r2, r2pad, cast(p['conv2']), one, one, one, 1, need=need)
            d, dg2, db2 = oracle.batch_norm_backward(d * m2, c1, cast(p['g2']), s2)
            d, dw1, _ = oracle.convolution_backward(d, r1, r1pad, cast(p['conv1']), st, one, one, 1, need=need)
            d, dg1, db1 = oracle.batch_norm_backward(d * m1, xin, cast(p['g1']), s1)
            dws = None
            if p['ws'] is None:
                d = d + grad
            else:
                ds, dws, _ = oracle.convolution_backward(grad, xin, xinpad, cast(p['ws']), st, (0, 0), one, 1, need=need)
                d = d + ds
            grads.append({'conv1': dw1, 'conv2': dw2, 'short': dws, 'g1': dg1, 'b1': db1, 'g2': dg2, 'b2': db2})
            grad = d
        xpad = np.pad(x.astype(dtype), ((0, 0), (0, 0), (1, 1), (1, 1)))
        dx, dw0, _ = oracle.convolution_backward(grad, x.astype(dtype), xpad, cast(w0), one, one, one, 1)
        return a, dx, dw0, grads[::-1]

    out32, dx32, dw032, grads32 = oracle_stack(np.float32, check_masks=False)
    out64, dx64, dw064, grads64 = oracle_stack(np.float64, check_masks=True)

    worst = {}

    def check(got, ref32, ref64, name):
        scale = float(np.abs(ref64).max())
        err_gpu = float(np.abs(got - ref64).max()) / scale
        err_cpu = float(np.abs(ref32 - ref64).max()) / scale
        worst[name.split('[')[0]] = max(worst.get(name.split('[')[0], 0.0), err_gpu)
        assert err_gpu <= max(3 * err_cpu, 2e-5), f'{name}: device err {err_gpu:.3g} vs oracle err {err_cpu:.3g}'

    check(out.cpu().detach().numpy(), out32, out64, 'out')
    check(xt.grad, dx32, dx64, 'x.grad')
    check(stem.weight.grad.get(), dw032, dw064, 'stem.weight.grad')
    for i, (b, g32, g64) in enumerate(zip(blocks, grads32, grads64)):
        check(b['conv1'].weight.grad.get(), g32['conv1'], g64['conv1'], f'conv1.weight.grad[{i}]')
        check(b['conv2'].weight.grad.get(), g32['conv2'], g64['conv2'], f'conv2.weight.grad[{i}]')
        if b['short'] is not None:
            check(b['short'].weight.grad.get(), g32['short'], g64['short'], f'shortcut.weight.grad[{i}]')
        check(b['bn1'].weight.grad.get(), g32['g1'], g64['g1'], f'bn1.weight.grad[{i}]')
        check(b['bn1'].bias.grad.get(), g32['b1'], g64['b1'], f'bn1.bias.grad[{i}]')
        check(b['bn2'].weight.grad.get(), g32['g2'], g64['g2'], f'bn2.weight.grad[{i}]')
        check(b['bn2'].bias.grad.get(), g32['b2'], g64['b2'], f'bn2.bias.grad[{i}]')
    print('PreAct-ResNet-18 stack, batch 8: worst max|gpu - f64| / max|f64| per tensor kind:',
          {k: f'{v:.2e}' for k, v in worst.items()})
