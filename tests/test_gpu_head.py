"""GPU parity for the classifier head (spatial mean, Linear through Transpose + Mm + Add,
LogSoftmax, NLLLoss) through the C ABI vs the CPU oracle.

Tolerances (fp32): the matrix products are convolution kernels and use the convolution bar,
allclose(rtol=1e-4, atol=1e-5) (reductions scaled by the tensor's magnitude); means, log-softmax
and the loss use rtol=1e-5 with atol=1e-6."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


def _dev(a):
    from pytortto_amd.xparray import hiparray
    return hiparray(a)


@pytest.mark.parametrize('shape,k', [((4, 6, 7, 7), 2), ((3, 5, 4), 1), ((2, 3, 9, 14), 2), ((5, 70), 1), ((64, 2048, 7, 7), 2)])
def test_mean_over_trailing_dimensions(shape, k):
    from pytortto_amd import ops
    rng = np.random.default_rng(0)
    x = (1.5 + rng.standard_normal(shape)).astype(np.float32)
    dim = tuple(range(-k, 0))
    for keep in (True, False):
        y = ops.mean_trailing(_dev(x), k, keep).get()
        ref = oracle.mean_forward(x, dim, keep)
        assert y.shape == ref.shape
        np.testing.assert_allclose(y, ref, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(y, x.astype(np.float64).mean(dim, keepdims=keep), rtol=2e-6, atol=1e-7)
    g = rng.standard_normal(ref.shape).astype(np.float32)
    dx = ops.mean_trailing_bwd(_dev(g), shape, k).get()
    np.testing.assert_array_equal(dx, oracle.mean_backward(g, shape, dim, False))


@pytest.mark.parametrize('m,k,n', [(64, 2048, 10), (7, 33, 5), (128, 512, 1000), (1, 16, 3), (50, 100, 64)])
def test_matrix_products_run_on_the_convolution_kernels(m, k, n):
    from pytortto_amd import ops
    rng = np.random.default_rng(1)
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)
    g = rng.standard_normal((m, n)).astype(np.float32)
    ad, bd, gd = _dev(a), _dev(b), _dev(g)
    a64, b64, g64 = (t.astype(np.float64) for t in (a, b, g))

    def check(got, ref32, ref64, name):
        scale = float(np.abs(ref64).max()) or 1.0
        assert np.abs(got - ref64).max() / scale <= max(3 * np.abs(ref32 - ref64).max() / scale, 5e-6), name
        np.testing.assert_allclose(got, ref32, rtol=1e-4, atol=1e-5 * max(1.0, scale), err_msg=name)

    check(ops.mm(ad, bd).get(), oracle.mm_forward(a, b), a64 @ b64, 'a @ b')
    ga, gb = oracle.mm_backward(g, a, b)
    check(ops.mm_grad_a(gd, bd).get(), ga, g64 @ b64.T, 'g @ b.T')
    check(ops.mm_grad_b(ad, gd).get(), gb, a64.T @ g64, 'a.T @ g')
    np.testing.assert_array_equal(ops.transpose2d(ad).get(), a.T)


@pytest.mark.parametrize('r,c', [(64, 10), (5, 1000), (3, 1), (130, 77)])
def test_log_softmax_rows(r, c):
    from pytortto_amd import ops
    rng = np.random.default_rng(2)
    x = (4 * rng.standard_normal((r, c))).astype(np.float32)
    x[0] += 90
    y = ops.log_softmax_fwd(_dev(x))
    ref = oracle.log_softmax_forward(x, -1)
    np.testing.assert_allclose(y.get(), ref, rtol=1e-5, atol=2e-6)
    g = rng.standard_normal((r, c)).astype(np.float32)
    dx = ops.log_softmax_bwd(_dev(g), y).get()
    np.testing.assert_allclose(dx, oracle.log_softmax_backward(g, ref, -1), rtol=1e-5, atol=2e-6)
    if c > 1:
        xn = x.copy()
        xn[1, 0] = np.nan
        yn = ops.log_softmax_fwd(_dev(xn)).get()
        assert np.isnan(yn[1]).all() and not np.isnan(yn[0]).any()       # as NumPy's max / sum propagate it


@pytest.mark.parametrize('reduction', ['mean', 'sum', 'none'])
@pytest.mark.parametrize('weighted', [False, True])
@pytest.mark.parametrize('ignore_index', [-100, 2])
def test_nll_loss(reduction, weighted, ignore_index):
    from pytortto_amd import ops
    rng = np.random.default_rng(3)
    n, c = 300, 10
    logp = oracle.log_softmax_forward(rng.standard_normal((n, c)).astype(np.float32))
    target = rng.integers(0, c, n)
    weight = rng.uniform(0.5, 2.0, c).astype(np.float32) if weighted else None
    loss, count = oracle.nll_loss_forward(logp, target, weight, ignore_index, reduction)
    wd = None if weight is None else _dev(weight)
    td = _dev(target.astype(np.int64))
    out, cnt = ops.nll_loss_fwd(_dev(logp), td, wd, ignore_index, reduction)
    np.testing.assert_allclose(out.get(), loss, rtol=1e-5, atol=1e-6)
    if reduction == 'mean':
        assert cnt.get()[0] == count
    g = rng.standard_normal(np.shape(loss)).astype(np.float32) if reduction == 'none' else np.float32(1.5)
    grad = ops.nll_loss_bwd(_dev(np.asarray(g, np.float32)), logp.shape, td, wd, cnt, ignore_index, reduction).get()
    np.testing.assert_allclose(grad, oracle.nll_loss_backward(g, logp.shape, target, weight, ignore_index, reduction,
                                                              count), rtol=1e-6, atol=1e-8)


@pytest.mark.parametrize('weighted', [False, True])
def test_nll_loss_negative_and_out_of_range_targets(weighted):
    """Classes -C..-1 count from the end, as the reference's NumPy indexing does (grad_nn.py:300,
    :306-309).  Classes outside [-C, C) raise IndexError there; on the device the loss turns NaN."""
    from pytortto_amd import ops
    rng = np.random.default_rng(8)
    n, c = 40, 7
    logp = oracle.log_softmax_forward(rng.standard_normal((n, c)).astype(np.float32))
    target = rng.integers(-c, c, n)
    assert (target < 0).any()
    weight = rng.uniform(0.5, 2.0, c).astype(np.float32) if weighted else None
    wd = None if weight is None else _dev(weight)
    for reduction in ('mean', 'sum', 'none'):
        loss, count = oracle.nll_loss_forward(logp, target, weight, 2, reduction)
        td = _dev(target.astype(np.int64))
        out, cnt = ops.nll_loss_fwd(_dev(logp), td, wd, 2, reduction)
        np.testing.assert_allclose(out.get(), loss, rtol=1e-5, atol=1e-6)
        g = rng.standard_normal(np.shape(loss)).astype(np.float32) if reduction == 'none' else np.float32(0.7)
        grad = ops.nll_loss_bwd(_dev(np.asarray(g, np.float32)), logp.shape, td, wd, cnt, 2, reduction).get()
        np.testing.assert_allclose(grad, oracle.nll_loss_backward(g, logp.shape, target, weight, 2, reduction, count),
                                   rtol=1e-6, atol=1e-8)
    for bad in (c, -c - 1, 1000):
        with pytest.raises(IndexError):
            oracle.nll_loss_forward(logp, np.where(np.arange(n) == 5, bad, target % c), weight, -100, 'mean')
        td = _dev(np.where(np.arange(n) == 5, bad, target % c).astype(np.int64))
        out, _ = ops.nll_loss_fwd(_dev(logp), td, wd, -100, 'mean')
        assert np.isnan(out.get()).all()
        rows, _ = ops.nll_loss_fwd(_dev(logp), td, wd, -100, 'none')
        rows = rows.get()
        assert np.isnan(rows[5]) and not np.isnan(np.delete(rows, 5)).any()


def test_linear_log_softmax_nll_modules_on_device():
    """The head of the reference's ResNet examples: mean over (H, W), flatten, Linear, LogSoftmax,
    NLLLoss -- same graph (MeanBackward, ViewBackward, TransposeBackward, MmBackward, AddBackward)."""
    import pytortto_amd as tt
    from pytortto_amd import nn
    tt.manual_seed(0)
    fc = nn.Linear(32, 10)
    w, b = np.asarray(fc.weight.data).copy(), np.asarray(fc.bias.data).copy()
    assert np.abs(w).max() <= 1 / np.sqrt(32) and np.abs(b).max() <= 1 / np.sqrt(32)
    x = tt.randn(16, 32, 5, 5, requires_grad=True)
    target = np.random.randint(0, 10, 16)
    fc.cuda()
    feat = tt.flatten(tt.mean(x.cuda(), (-1, -2), True), 1)
    assert feat.shape == (16, 32) and feat.grad_fn.__class__.__name__ == 'ViewBackward'
    logits = fc(feat)
    assert logits.grad_fn.__class__.__name__ == 'AddBackward'
    logp = nn.LogSoftmax(dim=-1)(logits)
    loss = nn.NLLLoss()(logp, tt.tensor(target).cuda())
    assert loss.shape == ()
    loss.backward()
    xh = np.asarray(x.data)
    f_ref = oracle.mean_forward(xh, (-1, -2), True).reshape(16, 32)
    l_ref = oracle.linear_forward(f_ref, w, b)
    p_ref = oracle.log_softmax_forward(l_ref)
    loss_ref, count = oracle.nll_loss_forward(p_ref, target)
    np.testing.assert_allclose(loss.item(), loss_ref, rtol=1e-5)
    dp = oracle.nll_loss_backward(np.float32(1.0), p_ref.shape, target, count=count)
    dl = oracle.log_softmax_backward(dp, p_ref)
    df, dw, db = oracle.linear_backward(dl, f_ref, w)
    dx = oracle.mean_backward(df.reshape(16, 32, 1, 1), xh.shape, (-1, -2), True)
    np.testing.assert_allclose(fc.weight.grad.get(), dw, rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(fc.bias.grad.get(), db, rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(x.grad, dx, rtol=1e-4, atol=1e-7)


def test_small_resnet_training_step_stays_on_device():
    """Stem (conv 7x7 s2 + BN + ReLU + MaxPool 3x3 s2), one bottleneck-style block with a strided
    shortcut, mean / flatten / Linear / LogSoftmax / NLLLoss: every op between .cuda() and the
    scalar loss runs in the library, and the gradients match the oracle's composition."""
    import pytortto_amd as tt
    from pytortto_amd import nn
    F = nn.functional
    tt.manual_seed(1)
    conv1, bn1 = nn.Conv2d(3, 8, 7, stride=2, padding=3, bias=False), nn.BatchNorm2d(8)
    conv2, bn2 = nn.Conv2d(8, 16, 3, stride=2, padding=1, bias=False), nn.BatchNorm2d(16)
    short = nn.Conv2d(8, 16, 1, stride=2, bias=False)
    fc = nn.Linear(16, 5)
    pool = nn.MaxPool2d(3, stride=2, padding=1)
    mods = [conv1, bn1, conv2, bn2, short, fc]
    host = [{k: np.asarray(v.data).copy() for k, v in m.named_parameters()} for m in mods]
    x = tt.randn(6, 3, 32, 32, requires_grad=True)
    target = np.random.randint(0, 5, 6)
    for m in mods:
        m.cuda()
    h = pool(F.relu(bn1(conv1(x.cuda()))))
    h = F.relu(bn2(conv2(h)) + short(h))
    logp = F.log_softmax(fc(tt.flatten(tt.mean(h, (-1, -2), True), 1)), -1)
    loss = F.nll_loss(logp, tt.tensor(target).cuda())
    loss.backward()

    # the same network from oracle pieces, in float32
    xh = np.asarray(x.data)
    one = np.ones
    c1, xp1 = oracle.convolution_forward(xh, host[0]['weight'], None, (2, 2), (3, 3), (1, 1), 1)
    b1 = oracle.batch_norm_forward(c1, host[1]['weight'], host[1]['bias'], np.zeros(8, np.float32), one(8, np.float32),
                                   True, 0.1, 1e-5)
    r1 = oracle.relu_forward(b1[0])
    p1, pos = oracle.max_pool2d(r1, (3, 3), (2, 2), (1, 1))
    c2, xp2 = oracle.convolution_forward(p1, host[2]['weight'], None, (2, 2), (1, 1), (1, 1), 1)
    b2 = oracle.batch_norm_forward(c2, host[3]['weight'], host[3]['bias'], np.zeros(16, np.float32),
                                   one(16, np.float32), True, 0.1, 1e-5)
    s2, xps = oracle.convolution_forward(p1, host[4]['weight'], None, (2, 2), (0, 0), (1, 1), 1)
    r2 = oracle.relu_forward(b2[0] + s2)
    f = oracle.mean_forward(r2, (-1, -2), True).reshape(6, 16)
    lp = oracle.log_softmax_forward(oracle.linear_forward(f, host[5]['weight'], host[5]['bias']))
    loss_ref, count = oracle.nll_loss_forward(lp, target)
    np.testing.assert_allclose(loss.item(), loss_ref, rtol=1e-5)
    dlp = oracle.nll_loss_backward(np.float32(1.0), lp.shape, target, count=count)
    df, dwf, dbf = oracle.linear_backward(oracle.log_softmax_backward(dlp, lp), f, host[5]['weight'])
    dr2 = oracle.relu_backward(oracle.mean_backward(df.reshape(6, 16, 1, 1), r2.shape, (-1, -2), True), r2)
    dc2, dg2, dbeta2 = oracle.batch_norm_backward(dr2, c2, host[3]['weight'], b2[1])
    dp1a, dw2, _ = oracle.convolution_backward(dc2, p1, xp2, host[2]['weight'], (2, 2), (1, 1), (1, 1), 1)
    dp1b, dws, _ = oracle.convolution_backward(dr2, p1, xps, host[4]['weight'], (2, 2), (0, 0), (1, 1), 1)
    dr1 = oracle.max_pool2d_backward(r1.shape, dp1a + dp1b, pos, (3, 3), (2, 2), (1, 1))
    dc1, dg1, dbeta1 = oracle.batch_norm_backward(oracle.relu_backward(dr1, r1), c1, host[1]['weight'], b1[1])
    dx, dw1, _ = oracle.convolution_backward(dc1, xh, xp1, host[0]['weight'], (2, 2), (3, 3), (1, 1), 1)

    def close(got, ref, name):
        scale = float(np.abs(ref).max())
        np.testing.assert_allclose(got, ref, rtol=1e-3, atol=2e-5 * scale, err_msg=name)

    close(fc.weight.grad.get(), dwf, 'fc.weight')
    close(fc.bias.grad.get(), dbf, 'fc.bias')
    close(conv2.weight.grad.get(), dw2, 'conv2.weight')
    close(short.weight.grad.get(), dws, 'shortcut.weight')
    close(bn2.weight.grad.get(), dg2, 'bn2.weight')
    close(bn1.bias.grad.get(), dbeta1, 'bn1.bias')
    close(conv1.weight.grad.get(), dw1, 'conv1.weight')
    close(x.grad, dx, 'x')
