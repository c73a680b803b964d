"""GPU parity: SGD / Adam / AdamW steps through the C ABI vs the CPU oracle, bit for bit (the
kernels keep the reference's float32 roundings and its float64 denominator), and a short
training loop of a small network."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('kw', [
    dict(momentum=0, dampening=0, weight_decay=0, nesterov=False),
    dict(momentum=0.9, dampening=0, weight_decay=0, nesterov=False),
    dict(momentum=0.9, dampening=0.1, weight_decay=5e-4, nesterov=False),
    dict(momentum=0.8, dampening=0, weight_decay=1e-3, nesterov=True),
])
def test_sgd_steps_match_the_oracle_bit_for_bit(kw):
    import pytortto_amd as tt
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(0)
    shape = (37, 29)                                   # 1073 elements: not a multiple of the block size
    p0 = rng.standard_normal(shape).astype(np.float32)
    lin = tt.nn.Linear(29, 37, bias=False)
    lin.weight.data[...] = p0
    lin.cuda()
    opt = tt.optim.SGD(lin.parameters(), lr=0.05, **kw)
    ref, bufs = p0.copy(), [None]
    for _ in range(6):
        g = rng.standard_normal(shape).astype(np.float32)
        lin.weight.grad = hiparray(g)
        opt.step()
        oracle.optim.sgd([ref], [g.copy()], bufs, kw['weight_decay'], kw['momentum'], 0.05, kw['dampening'],
                         kw['nesterov'])
        np.testing.assert_array_equal(lin.weight.data.get(), ref)
    if kw['momentum']:
        np.testing.assert_array_equal(opt.state[lin.weight]['momentum_buffer'].get(), bufs[0])
    opt.zero_grad()
    assert lin.weight.grad is None


@pytest.mark.parametrize('cls', ['Adam', 'AdamW'])
@pytest.mark.parametrize('amsgrad', [False, True])
@pytest.mark.parametrize('weight_decay', [0, 1e-2])
def test_adam_steps_match_the_oracle_bit_for_bit(cls, amsgrad, weight_decay):
    import pytortto_amd as tt
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(1)
    shape = (16, 3, 3, 3)
    p0 = rng.standard_normal(shape).astype(np.float32)
    conv = tt.nn.Conv2d(3, 16, 3, bias=False)
    conv.weight.data[...] = p0
    conv.cuda()
    opt = getattr(tt.optim, cls)(conv.parameters(), lr=1e-2, betas=(0.9, 0.99), eps=1e-8, weight_decay=weight_decay,
                                 amsgrad=amsgrad)
    ref = p0.copy()
    m, v, vmax = np.zeros_like(ref), np.zeros_like(ref), np.zeros_like(ref)
    for step in range(1, 8):
        g = rng.standard_normal(shape).astype(np.float32)
        conv.weight.grad = hiparray(g)
        opt.step()
        oracle.optim.adam([ref], [g], [m], [v], [vmax], [step], amsgrad, 0.9, 0.99, 1e-2, weight_decay, 1e-8,
                          cls == 'AdamW')
        np.testing.assert_array_equal(conv.weight.data.get(), ref)
    st = opt.state[conv.weight]
    assert st['step'] == 7
    np.testing.assert_array_equal(st['exp_avg'].get(), m)
    np.testing.assert_array_equal(st['exp_avg_sq'].get(), v)
    # state_dict holds host arrays and loads back onto the device
    sd = opt.state_dict()
    assert type(sd['state'][0]['exp_avg']) is np.ndarray
    opt2 = getattr(tt.optim, cls)(conv.parameters(), lr=1e-2)
    opt2.load_state_dict(sd)
    assert opt2.state[conv.weight]['exp_avg'].__class__ is hiparray and opt2.param_groups[0]['betas'] == (0.9, 0.99)


def test_training_loop_on_device_reduces_the_loss():
    """conv + BN + ReLU + pool + head, SGD with momentum: forty steps on one batch, the loss falls and
    every parameter stays on the device."""
    import pytortto_amd as tt
    from pytortto_amd import nn
    F = nn.functional
    tt.manual_seed(3)
    conv, bn, fc = nn.Conv2d(3, 8, 3, padding=1, bias=False), nn.BatchNorm2d(8), nn.Linear(8, 4)
    pool = nn.MaxPool2d(2)
    params = []
    for mod in (conv, bn, fc):
        mod.cuda()
        params += list(mod.parameters())
    opt = tt.optim.SGD(params, lr=0.1, momentum=0.9)
    x = tt.randn(16, 3, 8, 8).cuda()
    target = tt.tensor(np.random.randint(0, 4, 16)).cuda()
    losses = []
    for _ in range(40):
        opt.zero_grad()
        h = pool(F.relu(bn(conv(x))))
        logp = F.log_softmax(fc(tt.flatten(tt.mean(h, (-1, -2), True), 1)), -1)
        loss = F.nll_loss(logp, target)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert min(losses[-5:]) < 0.8 * losses[0], losses
    assert all(p.data.__class__.__name__ == 'hiparray' for p in params)


def test_optimizer_refuses_host_parameters():
    import pytortto_amd as tt
    lin = tt.nn.Linear(4, 2)
    lin.weight.grad = np.zeros((2, 4), np.float32)
    lin.bias.grad = np.zeros(2, np.float32)
    with pytest.raises(RuntimeError, match='device parameters only'):
        tt.optim.SGD(lin.parameters(), lr=0.1).step()


def test_checkpoint_of_device_model_and_optimizer(tmp_path):
    """state_dict() of device modules and of the optimiser holds host arrays; tt.save / tt.load
    carry them, and a fresh device model resumes with identical parameters, BatchNorm buffers
    and momentum."""
    import pytortto_amd as tt
    from pytortto_amd import nn
    tt.manual_seed(4)

    def make():
        net = nn.Sequential(nn.Conv2d(3, 4, 3, padding=1, bias=False), nn.BatchNorm2d(4), nn.ReLU())
        net.cuda()
        return net, tt.optim.SGD(net.parameters(), lr=0.1, momentum=0.9)

    net, opt = make()
    x = tt.randn(8, 3, 6, 6).cuda()
    g = tt.randn(8, 4, 6, 6).cuda()
    for _ in range(2):
        opt.zero_grad()
        net(x).backward(g)
        opt.step()
    path = str(tmp_path / 'ckpt.npy')
    tt.save({'model': net.state_dict(), 'optim': opt.state_dict()}, path)
    ck = tt.load(path)
    assert all(type(v) is np.ndarray for v in ck['model'].values())
    assert ck['model']['1.num_batches_tracked'] == 2 and not np.allclose(ck['model']['1.running_mean'], 0)
    net2, opt2 = make()
    net2.load_state_dict(ck['model'])
    opt2.load_state_dict(ck['optim'])
    for (k, a), (_, b) in zip(net.state_dict().items(), net2.state_dict().items()):
        np.testing.assert_array_equal(a, b, err_msg=k)
    # one more identical step on both: same result, so the momentum buffers came along
    for n_, o_ in ((net, opt), (net2, opt2)):
        o_.zero_grad()
        n_(x).backward(g)
        o_.step()
    for (k, a), (_, b) in zip(net.state_dict().items(), net2.state_dict().items()):
        np.testing.assert_array_equal(a, b, err_msg=k)


def test_many_parameters_in_one_group_take_several_launches():
    """30 parameters of different sizes (more than one multi-tensor launch holds); one of them
    only receives a gradient every other step, so its Adam step count lags behind."""
    import pytortto_amd as tt
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(5)
    shapes = [(1 + 7 * i, 3 + (i % 5)) for i in range(30)]
    host = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    for kind in ('sgd', 'adam'):
        params = [tt.nn.Parameter(tt.tensor(h.copy()).cuda().detach()) for h in host]
        ref = [h.copy() for h in host]
        if kind == 'sgd':
            opt = tt.optim.SGD(params, lr=0.1, momentum=0.9, weight_decay=1e-3)
            bufs = [None] * 30
        else:
            opt = tt.optim.Adam(params, lr=1e-2, betas=(0.9, 0.99))
            m = [np.zeros_like(h) for h in host]
            v = [np.zeros_like(h) for h in host]
            steps = [0] * 30
        for it in range(4):
            grads = [rng.standard_normal(s).astype(np.float32) for s in shapes]
            live = [i for i in range(30) if not (i == 7 and it % 2)]
            for i, p in enumerate(params):
                p.grad = hiparray(grads[i]) if i in live else None
            opt.step()
            for i in live:
                if kind == 'sgd':
                    b = [bufs[i]]
                    oracle.optim.sgd([ref[i]], [grads[i].copy()], b, 1e-3, 0.9, 0.1, 0, False)
                    bufs[i] = b[0]
                else:
                    steps[i] += 1
                    oracle.optim.adam([ref[i]], [grads[i]], [m[i]], [v[i]], [None], [steps[i]], False, 0.9, 0.99, 1e-2,
                                      0, 1e-8)
            for i in range(30):
                np.testing.assert_array_equal(params[i].data.get(), ref[i], err_msg=f'{kind} step {it} parameter {i}')
