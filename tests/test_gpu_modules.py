"""GPU parity at the module level: nn.Conv2d / nn.ConvTranspose2d / nn.BatchNorm2d with
``.cuda()`` semantics and autograd, against the CPU oracle on identical seeded inputs."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


def _close(got, ref, rtol=1e-4, atol=1e-5, name=''):
    np.testing.assert_allclose(got, ref, rtol=rtol, atol=atol * max(1.0, float(np.abs(ref).max())), err_msg=name)


def test_config1_conv2d_module_forward_backward():
    """Conv2d(16, 32, 3, stride 1, pad 1, bias) on x = randn(32,16,32,32), upstream grad randn, seed 0."""
    import pytortto_amd as tt
    tt.manual_seed(0)
    conv = tt.nn.Conv2d(16, 32, 3, stride=1, padding=1, bias=True)
    x = tt.randn(32, 16, 32, 32, requires_grad=True)
    g = tt.randn(32, 32, 32, 32)
    w, b = conv.weight.data.copy(), conv.bias.data.copy()
    y_ref, xpad = oracle.convolution_forward(np.asarray(x.data), np.asarray(w), np.asarray(b), (1, 1), (1, 1), (1, 1), 1)
    dx_ref, dw_ref, db_ref = oracle.convolution_backward(np.asarray(g.data), np.asarray(x.data), xpad, np.asarray(w),
                                                         (1, 1), (1, 1), (1, 1), 1)
    conv.cuda()
    xd = x.cuda()
    assert xd.grad_fn.__class__.__name__ == 'ToCopyBackward' and str(xd.device) == 'hip:0'
    y = conv(xd)
    assert y.grad_fn.__class__.__name__ == 'ConvolutionBackward' and y.shape == (32, 32, 32, 32)
    with pytest.raises(TypeError, match="can't convert hip:0 device type tensor to numpy"):
        y.detach().numpy()
    y.backward(g.cuda())
    _close(y.cpu().detach().numpy(), y_ref, name='y')
    assert type(x.grad) is np.ndarray            # came back through ToCopyBackward
    _close(x.grad, dx_ref, name='x.grad')
    _close(conv.weight.grad.get(), dw_ref, name='weight.grad')
    _close(conv.bias.grad.get(), db_ref, name='bias.grad')
    sd = conv.state_dict()
    assert type(sd['weight']) is np.ndarray
    np.testing.assert_array_equal(sd['weight'], w)


def test_batchnorm2d_module_train_steps_and_eval():
    import pytortto_amd as tt
    tt.manual_seed(1)
    bn = tt.nn.BatchNorm2d(6, momentum=None)      # cumulative moving average
    xs = [2 + 3 * np.random.randn(8, 6, 16, 16).astype(np.float32) for _ in range(3)]
    rm, rv = np.zeros(6, np.float32), np.ones(6, np.float32)
    gamma, beta = np.ones(6, np.float32), np.zeros(6, np.float32)
    bn.cuda()
    for step, x in enumerate(xs):
        y_ref, _, rm, rv = oracle.batch_norm_forward(x, gamma, beta, rm, rv, True, 1.0 / (step + 1), 1e-5)
        y = bn(tt.tensor(x).cuda())
        _close(y.cpu().detach().numpy(), y_ref, rtol=1e-5, atol=2e-6)
    assert bn.num_batches_tracked.item() == 3.0
    sd = bn.state_dict()
    _close(sd['running_mean'], rm, rtol=1e-5, atol=1e-6)
    _close(sd['running_var'], rv, rtol=1e-5, atol=1e-6)
    bn.eval()
    y_ref, _, _, _ = oracle.batch_norm_forward(xs[0], gamma, beta, rm, rv, False, None, 1e-5)
    _close(bn(tt.tensor(xs[0]).cuda()).cpu().detach().numpy(), y_ref, rtol=1e-5, atol=2e-6)
    assert bn.num_batches_tracked.item() == 3.0


def test_conv_transpose2d_module_with_output_size():
    import pytortto_amd as tt
    tt.manual_seed(2)
    m = tt.nn.ConvTranspose2d(8, 6, 3, stride=2, padding=1, groups=2)
    x = tt.randn(3, 8, 5, 5, requires_grad=True)
    w, b = np.asarray(m.weight.data).copy(), np.asarray(m.bias.data).copy()
    y_ref = oracle.transposed_convolution_forward(np.asarray(x.data), w, b, (2, 2), (1, 1), (1, 1), (1, 1), 2)
    g = np.random.randn(*y_ref.shape).astype(np.float32)
    dx_ref, dw_ref, db_ref = oracle.transposed_convolution_backward(g, np.asarray(x.data), w, (2, 2), (1, 1), (1, 1), 2)
    m.cuda()
    y = m(x.cuda(), output_size=(10, 10))
    assert y.shape == (3, 6, 10, 10) and y.grad_fn.__class__.__name__ == 'TransposedConvolutionBackward'
    y.backward(tt.tensor(g).cuda())
    _close(y.cpu().detach().numpy(), y_ref)
    _close(x.grad, dx_ref)
    _close(m.weight.grad.get(), dw_ref)
    _close(m.bias.grad.get(), db_ref)


def test_preact_block_on_device_matches_oracle_composition():
    """BN-ReLU-conv3x3(s2)-BN-ReLU-conv3x3 plus a 1x1 stride-2 shortcut on the raw block input:
    the whole block runs on the device (residual add and gradient accumulation included)."""
    import pytortto_amd as tt
    from pytortto_amd import nn
    tt.manual_seed(4)
    bn1, conv1 = nn.BatchNorm2d(8), nn.Conv2d(8, 16, 3, stride=2, padding=1, bias=False)
    bn2, conv2 = nn.BatchNorm2d(16), nn.Conv2d(16, 16, 3, stride=1, padding=1, bias=False)
    short = nn.Conv2d(8, 16, 1, stride=2, bias=False)
    x = (1 + 2 * np.random.randn(6, 8, 12, 12)).astype(np.float32)
    g = np.random.randn(6, 16, 6, 6).astype(np.float32)
    w1, w2, ws = (np.asarray(m.weight.data).copy() for m in (conv1, conv2, short))
    one8, zero8, one16, zero16 = np.ones(8, np.float32), np.zeros(8, np.float32), np.ones(16, np.float32), np.zeros(16, np.float32)

    # oracle composition
    a1, s1, _, _ = oracle.batch_norm_forward(x, one8, zero8, None, None, True, 0.1, 1e-5)
    r1 = np.maximum(a1, 0)
    c1, r1pad = oracle.convolution_forward(r1, w1, None, (2, 2), (1, 1), (1, 1), 1)
    a2, s2, _, _ = oracle.batch_norm_forward(c1, one16, zero16, None, None, True, 0.1, 1e-5)
    r2 = np.maximum(a2, 0)
    c2, r2pad = oracle.convolution_forward(r2, w2, None, (1, 1), (1, 1), (1, 1), 1)
    sc, xpad = oracle.convolution_forward(x, ws, None, (2, 2), (0, 0), (1, 1), 1)
    out_ref = c2 + sc
    d_r2, dw2_ref, _ = oracle.convolution_backward(g, r2, r2pad, w2, (1, 1), (1, 1), (1, 1), 1, need=(True, True, False))
    d_c1, dg2_ref, db2_ref = oracle.batch_norm_backward(d_r2 * (r2 > 0), c1, one16, s2)
    d_r1, dw1_ref, _ = oracle.convolution_backward(d_c1, r1, r1pad, w1, (2, 2), (1, 1), (1, 1), 1, need=(True, True, False))
    dx_main, dg1_ref, db1_ref = oracle.batch_norm_backward(d_r1 * (r1 > 0), x, one8, s1)
    dx_short, dws_ref, _ = oracle.convolution_backward(g, x, xpad, ws, (2, 2), (0, 0), (1, 1), 1, need=(True, True, False))
    dx_ref = dx_main + dx_short

    for m in (bn1, conv1, bn2, conv2, short):
        m.cuda()
    relu = nn.ReLU()
    xt = tt.tensor(x, requires_grad=True)
    xd = xt.cuda()
    out = conv2(relu(bn2(conv1(relu(bn1(xd)))))) + short(xd)
    out.backward(tt.tensor(g).cuda())
    _close(out.cpu().detach().numpy(), out_ref, name='out')
    _close(xt.grad, dx_ref, atol=2e-5, name='dx')
    _close(conv1.weight.grad.get(), dw1_ref, atol=2e-5, name='dw1')
    _close(conv2.weight.grad.get(), dw2_ref, atol=2e-5, name='dw2')
    _close(short.weight.grad.get(), dws_ref, atol=2e-5, name='dws')
    _close(bn1.weight.grad.get(), dg1_ref, atol=2e-5, name='dgamma1')
    _close(bn2.bias.grad.get(), db2_ref, atol=2e-5, name='dbeta2')


def test_dcgan_generator_stack_matches_oracle_composition():
    """ConvTranspose2d 100->512 (k4 s1 p0), then k4 s2 p1: 512->256->128->64->3, BatchNorm2d + ReLU
    in between, no bias: the baseline's conv-transpose configuration at batch 8, through
    nn.Sequential on the device, against the same stack composed from oracle calls."""
    import pytortto_amd as tt
    from pytortto_amd import nn
    tt.manual_seed(0)
    chans = [100, 512, 256, 128, 64, 3]
    geo = [((1, 1), (0, 0))] + [((2, 2), (1, 1))] * 4
    layers = []
    for i in range(5):
        layers.append(nn.ConvTranspose2d(chans[i], chans[i + 1], 4, stride=geo[i][0], padding=geo[i][1], bias=False))
        if i < 4:
            layers += [nn.BatchNorm2d(chans[i + 1]), nn.ReLU()]
    net = nn.Sequential(*layers)
    ws = [np.asarray(m.weight.data).copy() for m in layers if isinstance(m, nn.ConvTranspose2d)]

    def relu_margin(z):
        """Smallest |pre-activation| any ReLU of the stack sees (float32 oracle forward)."""
        a, margin = z, np.inf
        for i in range(4):
            a = oracle.transposed_convolution_forward(a, ws[i], None, geo[i][0], geo[i][1], (0, 0), (1, 1), 1)
            c = chans[i + 1]
            a, _, _, _ = oracle.batch_norm_forward(a, np.ones(c, np.float32), np.zeros(c, np.float32), None, None,
                                                   True, 0.1, 1e-5)
            margin = min(margin, float(np.abs(a).min()))
            a = np.maximum(a, 0)
        return margin

    # ReLU is discontinuous in its gradient: a pre-activation within rounding distance of zero may
    # get a different mask from two correct float32 evaluations, and the gradients then differ by
    # a whole element.  Draw inputs until every pre-activation keeps a safe distance from zero.
    for _ in range(50):
        z = np.random.randn(8, 100, 1, 1).astype(np.float32)
        if relu_margin(z) > 1e-6:   # device and oracle pre-activations differ by ~1e-7
            break
    else:
        pytest.fail('no input with a safe ReLU margin found')
    g = np.random.randn(8, 3, 64, 64).astype(np.float32)

    # The margin above is measured on the oracle's pre-activations; the device's differ from them
    # by a few 1e-6, so one of its masks can still differ in an element or two.  Either mask is a
    # correct float32 result there: the oracle's backward pass is given the device's masks (taken
    # from a second, bit-identical forward pass layer by layer).
    net.cuda()
    device_masks, a = [], tt.tensor(z).cuda()
    for m in layers:
        a = m(a)
        if isinstance(m, nn.ReLU):
            device_masks.append(a.cpu().detach().numpy() > 0)
    del a

    def oracle_stack(dtype):
        """Forward and backward of the stack composed from oracle calls in `dtype`."""
        a, tape, masks = z.astype(dtype), [], list(device_masks)
        wd = [w.astype(dtype) for w in ws]
        for i in range(5):
            st, pd = geo[i]
            y = oracle.transposed_convolution_forward(a, wd[i], None, st, pd, (0, 0), (1, 1), 1)
            tape.append(('convt', a, i))
            a = y
            if i < 4:
                c = chans[i + 1]
                y, saved, _, _ = oracle.batch_norm_forward(a, np.ones(c, dtype), np.zeros(c, dtype), None, None,
                                                           True, 0.1, 1e-5)
                tape.append(('bn', a, saved, c))
                assert np.mean((y > 0) != masks[i]) < 1e-4, 'ReLU masks of device and oracle disagree beyond rounding'
                a = np.maximum(y, 0)
                tape.append(('relu', a))
        grad, dws, dgs = g.astype(dtype), {}, {}
        for rec in reversed(tape):
            if rec[0] == 'relu':
                grad = grad * masks.pop()
            elif rec[0] == 'bn':
                grad, dgs[rec[3]], _ = oracle.batch_norm_backward(grad, rec[1], np.ones(rec[3], dtype), rec[2])
            else:
                st, pd = geo[rec[2]]
                grad, dws[rec[2]], _ = oracle.transposed_convolution_backward(grad, rec[1], wd[rec[2]], st, pd, (1, 1), 1)
        return a, grad, dws, dgs

    out_ref, dz_ref, dws, dgs = oracle_stack(np.float32)
    out64, dz64, dws64, dgs64 = oracle_stack(np.float64)

    def check(got, ref32, ref64, name):
        # Rounding differences compound through five layers and four BatchNorm backward passes
        # (cancellation), so two correct float32 evaluations differ by more than one layer's
        # tolerance: the device result must be as close to the float64 stack as the oracle's.
        scale = float(np.abs(ref64).max())
        err_gpu = float(np.abs(got - ref64).max()) / scale
        err_cpu = float(np.abs(ref32 - ref64).max()) / scale
        assert err_gpu <= max(3 * err_cpu, 2e-5), f'{name}: device err {err_gpu:.3g} vs oracle err {err_cpu:.3g}'

    net.cuda()
    zt = tt.tensor(z, requires_grad=True)
    out = net(zt.cuda())
    assert out.shape == (8, 3, 64, 64)
    out.backward(tt.tensor(g).cuda())
    _close(out.cpu().detach().numpy(), out_ref, atol=2e-5, name='out')
    check(out.cpu().detach().numpy(), out_ref, out64, 'out')
    check(zt.grad, dz_ref, dz64, 'dz')
    convs = [m for m in layers if isinstance(m, nn.ConvTranspose2d)]
    for i, m in enumerate(convs):
        check(m.weight.grad.get(), dws[i], dws64[i], f'dw{i}')
    bns = [m for m in layers if isinstance(m, nn.BatchNorm2d)]
    for m in bns:
        check(m.weight.grad.get(), dgs[m.num_features], dgs64[m.num_features], f'dgamma{m.num_features}')


def test_unbatched_input_and_mixed_device_error():
    import pytortto_amd as tt
    tt.manual_seed(5)
    conv = tt.nn.Conv2d(3, 4, 3, padding=1)
    x = tt.randn(3, 6, 6)
    w, b = np.asarray(conv.weight.data).copy(), np.asarray(conv.bias.data).copy()
    y_ref, _ = oracle.convolution_forward(np.asarray(x.data)[None], w, b, (1, 1), (1, 1), (1, 1), 1)
    with pytest.raises(RuntimeError, match='Input type \\(hiparray\\) and weight type \\(nparray\\) should be the same'):
        conv(x.cuda())
    conv.cuda()
    y = conv(x.cuda())
    assert y.shape == (4, 6, 6)
    _close(y.cpu().detach().numpy(), y_ref[0])


def test_device_memory_is_pooled_and_released():
    import ctypes
    import pytortto_amd as tt
    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    used, pooled, ws = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    a = hiparray(np.ones((256, 256), np.float32))
    _hip.call('tt_mem_stats', ctypes.byref(used), ctypes.byref(pooled), ctypes.byref(ws))
    before = used.value
    ptr = a.ptr
    del a
    _hip.call('tt_mem_stats', ctypes.byref(used), ctypes.byref(pooled), ctypes.byref(ws))
    assert used.value == before - 256 * 256 * 4
    b = hiparray(np.zeros((256, 256), np.float32))
    assert b.ptr == ptr                       # same size class: the pooled block is reused
    _hip.call('tt_empty_cache')


def test_workspace_queries_bound_what_the_calls_request():
    """tt_workspace_size_* report what a call asks the library for: after tt_empty_cache() the
    workspace grows to at least that (the library adds a quarter of head room), never before."""
    import ctypes
    from pytortto_amd import _hip, ops
    from pytortto_amd.xparray import hiparray

    def workspace_now():
        used, pooled, ws = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
        _hip.call('tt_mem_stats', ctypes.byref(used), ctypes.byref(pooled), ctypes.byref(ws))
        return ws.value

    def query(name, *args):
        out = ctypes.c_size_t()
        _hip.call(name, ctypes.byref(out), *args)
        return out.value

    n, c, h, k, r, st, pd = 8, 96, 28, 160, 3, 2, 1
    q = (h + 2 * pd - r) // st + 1
    geo = (n, c, h, h, k, r, r, st, st, pd, pd, 1, 1, 1)
    rng = np.random.default_rng(0)
    x = hiparray(rng.standard_normal((n, c, h, h), dtype=np.float32))
    w = hiparray(rng.standard_normal((k, c, r, r), dtype=np.float32))
    g = hiparray(rng.standard_normal((n, k, q, q), dtype=np.float32))
    sizes = {'fwd': query('tt_workspace_size_conv2d_fwd_f32', *geo),
             'dgrad': query('tt_workspace_size_conv2d_dgrad_f32', *geo, q, q),
             'wgrad': query('tt_workspace_size_conv2d_wgrad_f32', *geo, q, q),
             'bn': query('tt_workspace_size_bn_f32', n, c, h * h)}
    assert all(v > 0 for v in sizes.values()), sizes
    # channels small enough for the single-kernel BatchNorm passes leave no partial sums behind
    assert query('tt_workspace_size_bn_f32', n, k, q * q) == 0
    runs = {'fwd': lambda: ops.conv2d_fwd(x, w, None, (st, st), (pd, pd), (1, 1), 1),
            'dgrad': lambda: ops.conv2d_dgrad(g, w, None, (h, h), (st, st), (pd, pd), (1, 1), 1),
            'wgrad': lambda: ops.conv2d_wgrad(x, g, (k, c, r, r), (st, st), (pd, pd), (1, 1), 1),
            'bn': lambda: ops.bn_fwd_train(x, None, None, None, None, 0.1, 1e-5)}
    for name, run in runs.items():
        _hip.synchronize()
        _hip.call('tt_empty_cache')
        assert workspace_now() == 0
        run()
        got = workspace_now()
        assert sizes[name] <= got <= 2 * sizes[name] + (1 << 20), (name, sizes[name], got)
    _hip.synchronize()
    _hip.call('tt_empty_cache')
    ops.bn_fwd_train(g, None, None, None, None, 0.1, 1e-5)
    assert workspace_now() == 0
    with pytest.raises(RuntimeError, match='not divisible by groups'):
        query('tt_workspace_size_conv2d_fwd_f32', n, c, h, h, k, r, r, st, st, pd, pd, 1, 1, 7)


def _device_leaf(values):
    import pytortto_amd as tt
    from pytortto_amd.xparray import hiparray
    return tt.Tensor(hiparray(np.ascontiguousarray(values, dtype=np.float32)), requires_grad=True)


def test_add_backward_gives_each_operand_its_own_gradient_array():
    """``Add`` hands every operand a gradient array of its own, as the reference's
    ``reverse_broadcast`` does (helper.py:32-42: ``sum((), keepdims=True)`` copies).  LeakyReLU's
    backward scales the array it is given in place (grad_nn.py:92-94), so with a shared array one
    branch would receive the other's already-scaled gradient."""
    import pytortto_amd as tt
    from pytortto_amd.nn import functional as F
    rng = np.random.default_rng(5)
    a, b = rng.standard_normal((3, 4, 5, 6)), rng.standard_normal((3, 4, 5, 6))
    g = rng.standard_normal((3, 4, 5, 6)).astype(np.float32)
    slope = 0.25

    at, bt = _device_leaf(a), _device_leaf(b)
    out = F.leaky_relu(at, slope) + F.leaky_relu(bt, slope)
    out.backward(tt.tensor(g).cuda())
    ga_ref = g * np.where(a.astype(np.float32) >= 0, np.float32(1), np.float32(slope))
    gb_ref = g * np.where(b.astype(np.float32) >= 0, np.float32(1), np.float32(slope))
    assert np.array_equal(at.grad.get(), ga_ref)
    assert np.array_equal(bt.grad.get(), gb_ref)

    # a residual add whose skip operand is consumed after the LeakyReLU branch scaled its gradient
    xt = _device_leaf(a)
    h = F.leaky_relu(xt, slope)
    out = F.leaky_relu(h, 0.5) + h
    out.backward(tt.tensor(g).cuda())
    h_ref = np.maximum(a.astype(np.float32) * np.float32(slope), a.astype(np.float32))
    gh = g * np.where(h_ref >= 0, np.float32(1), np.float32(0.5)) + g
    gx_ref = gh * np.where(a.astype(np.float32) >= 0, np.float32(1), np.float32(slope))
    np.testing.assert_allclose(xt.grad.get(), gx_ref, rtol=1e-6, atol=0)

    # two leaves of one shape: their .grad are distinct buffers, so accumulating into one
    # (a second backward pass) leaves the other alone
    at, bt = _device_leaf(a), _device_leaf(b)
    (at + bt).backward(tt.tensor(g).cuda())
    assert at.grad.ptr != bt.grad.ptr
    (at + at).backward(tt.tensor(g).cuda())
    assert np.array_equal(bt.grad.get(), g)
    assert np.array_equal(at.grad.get(), g + (g + g))


def test_batch_norm_without_buffers_accepts_one_value_per_channel_outside_training():
    """Only training refuses one value per channel (grad_nn.py:921-922); `F.batch_norm` with
    training=False and no running buffers takes the batch statistics, here the value itself and
    zero (:935-937), so y = beta.  (Through the module this shape is refused in eval mode too: it
    passes training=True when it has no buffers, nn/modules/batchnorm.py:75-78.)"""
    import pytortto_amd as tt
    from pytortto_amd import nn
    gamma = np.arange(1, 6, dtype=np.float32)
    beta = np.linspace(-1, 1, 5).astype(np.float32)
    x = np.random.randn(1, 5, 1, 1).astype(np.float32)
    bn = nn.BatchNorm2d(5, track_running_stats=False)
    bn.cuda()
    for mode in (bn.train, bn.eval):
        mode()
        with pytest.raises(ValueError, match='Expected more than 1 value per channel'):
            bn(tt.tensor(x).cuda())
    y = nn.functional.batch_norm(tt.tensor(x).cuda(), None, None, tt.tensor(gamma).cuda(), tt.tensor(beta).cuda(),
                                 False, 0.1, 1e-5).cpu().detach().numpy()
    y_ref, _, _, _ = oracle.batch_norm_forward(x, gamma, beta, None, None, False, 0.1, 1e-5)
    np.testing.assert_allclose(y, y_ref, rtol=1e-6, atol=1e-7)
