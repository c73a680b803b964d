"""GPU: BatchNorm with the ReLU behind it fused into its kernels.

C ABI: ``tt_bn_relu_fwd_train_f32`` must give bit for bit what ``tt_bn_fwd_train_f32`` followed by
``tt_relu_fwd_f32`` gives, and ``tt_bn_relu_bwd_f32`` what ``tt_relu_bwd_f32`` followed by
``tt_bn_bwd_f32`` gives (same kernels, same summation order, the elementwise step folded in) -- on
shapes that reach every kernel variant, with NaN and non-finite gradients at masked elements.  The
unfused pair is itself held to the oracle by the BatchNorm and elementwise tests.

Host side: the autograd nodes stay two (``BatchNormBackward``, ``ReluBackward``); the BatchNorm
launch is parked and absorbed by a ReLU that comes next.  Checked here: the graph, the results
against the oracle composition, an in-place ReLU, a second consumer of the BatchNorm output (its
values are then recomputed on demand), and that anything other than a ReLU finds the parked launch
done.
"""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

# two-sweep kernels: plane mode, flat float4, flat scalar, stream reduce with several splits;
# single-kernel path for small channels (256 threads x 16 values, 1024 x 16 with few channels, 256 x 64 with many)
SHAPES = [(4, 3, 5, 5), (16, 5, 4, 4), (8, 64, 14, 14), (6, 16, 16, 16), (5, 7, 24, 20), (64, 64, 28, 28),
          (128, 4, 32, 32), (96, 12, 28, 28), (4, 128, 7, 7), (8, 256, 14, 14), (16, 130, 9, 7),
          (32, 256, 14, 14), (24, 576, 14, 14)]


def _bits_equal(a, b, name):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    na, nb = np.isnan(a), np.isnan(b)
    assert np.array_equal(na, nb), f'{name}: NaN pattern differs'
    assert np.array_equal(a.view(np.uint32)[~na], b.view(np.uint32)[~nb]), f'{name}: bits differ'


@pytest.mark.parametrize('shape', SHAPES, ids=lambda s: 'x'.join(map(str, s)))
@pytest.mark.parametrize('affine', [True, False])
def test_fused_entry_points_match_the_unfused_pair_bit_for_bit(shape, affine):
    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(sum(shape))
    n, c = shape[:2]
    hw = int(np.prod(shape[2:]))
    x = (0.5 + 2 * rng.standard_normal(shape)).astype(np.float32)
    if x.size > 100:
        x.flat[7] = np.nan if c > 3 else x.flat[7]      # a NaN poisons its channel in both paths alike
    gamma = rng.uniform(0.5, 1.5, c).astype(np.float32) if affine else None
    beta = (0.3 * rng.standard_normal(c)).astype(np.float32) if affine else None
    dy = rng.standard_normal(shape).astype(np.float32)
    dy.flat[:4] = [np.inf, -np.inf, np.nan, -1.0]
    xd, dyd = hiparray(x), hiparray(dy)
    gd = None if gamma is None else hiparray(gamma)
    bd = None if beta is None else hiparray(beta)
    ptr = lambda a: None if a is None else a.ptr

    def forward(entry):
        y = hiparray.empty(shape)
        st = [hiparray.empty((c,)) for _ in range(5)]
        rm, rv, nbt = hiparray(np.zeros(c, np.float32)), hiparray(np.ones(c, np.float32)), hiparray(np.zeros(1, np.float32))
        _hip.call(entry, xd.ptr, ptr(gd), ptr(bd), y.ptr, st[0].ptr, st[1].ptr, st[2].ptr, rm.ptr, rv.ptr,
                  st[3].ptr, st[4].ptr, nbt.ptr, 0.1, 1e-5, n, c, hw)
        assert nbt.get()[0] == 1.0
        return y, st

    y_plain, st_plain = forward('tt_bn_fwd_train_f32')
    y_ref = hiparray.empty(shape)
    _hip.call('tt_relu_fwd_f32', y_plain.ptr, y_ref.ptr, x.size)
    y_fused, st_fused = forward('tt_bn_relu_fwd_train_f32')
    _bits_equal(y_fused.get(), y_ref.get(), 'y')
    for a, b, name in zip(st_fused, st_plain, ('mean', 'var_eps', 'sd', 'running_mean', 'running_var')):
        _bits_equal(a.get(), b.get(), name)

    def backward(fused):
        dx, dg, db = hiparray.empty(shape), hiparray.empty((c,)), hiparray.empty((c,))
        tail = (ptr(gd), st_plain[0].ptr, st_plain[1].ptr, st_plain[2].ptr, dx.ptr, dg.ptr, db.ptr, n, c, hw)
        if fused:
            _hip.call('tt_bn_relu_bwd_f32', xd.ptr, dyd.ptr, y_ref.ptr, *tail)
        else:
            g = hiparray.empty(shape)
            _hip.call('tt_relu_bwd_f32', dyd.ptr, y_ref.ptr, g.ptr, x.size)
            _hip.call('tt_bn_bwd_f32', xd.ptr, g.ptr, *tail)
        return dx.get(), dg.get(), db.get()

    for a, b, name in zip(backward(True), backward(False), ('dx', 'dgamma', 'dbeta')):
        _bits_equal(a, b, name)


def _away_from_zero(x, gamma, beta):
    """Nudges the inputs whose normalised value lies within 1e-4 of zero: a ReLU mask there may
    differ between two correct float32 evaluations, and the gradients then differ by an element."""
    for _ in range(10):
        y, _, _, _ = oracle.batch_norm_forward(x, gamma, beta, None, None, True, 0.1, 1e-5)
        close = np.abs(y) < 1e-4
        if not close.any():
            return x
        x = x + np.float32(0.01) * close
    raise AssertionError('could not move the pre-activations away from zero')


def _oracle_bn_relu(x, gamma, beta, g):
    y, saved, _, _ = oracle.batch_norm_forward(x, gamma, beta, None, None, True, 0.1, 1e-5)
    r = np.maximum(y, 0)
    dx, dg, db = oracle.batch_norm_backward(g * (r > 0), x, gamma, saved)
    return y, r, dx, dg, db


@pytest.mark.parametrize('inplace', [False, True])
def test_relu_after_batchnorm_through_the_modules(inplace):
    import pytortto_amd as tt
    from pytortto_amd import _hip, nn, ops
    rng = np.random.default_rng(2)
    x = (1 + 2 * rng.standard_normal((6, 16, 12, 12))).astype(np.float32)
    g = rng.standard_normal(x.shape).astype(np.float32)
    gamma, beta = rng.uniform(0.5, 1.5, 16).astype(np.float32), (0.2 * rng.standard_normal(16)).astype(np.float32)
    x = _away_from_zero(x, gamma, beta)
    bn = nn.BatchNorm2d(16)
    bn.weight.data[...] = gamma
    bn.bias.data[...] = beta
    bn.cuda()
    xt = tt.tensor(x, requires_grad=True)
    out_bn = bn(xt.cuda())
    assert _hip.pending().__class__ is ops.DeferredBatchNorm          # parked, nothing launched yet
    out = nn.functional.relu(out_bn, inplace=inplace)
    assert _hip.pending() is None
    assert out.grad_fn.__class__.__name__ == 'ReluBackward'
    assert out.grad_fn.next_functions[0][0].__class__.__name__ == 'BatchNormBackward'
    assert bn.num_batches_tracked.item() == 1.0
    out.backward(tt.tensor(g).cuda())
    _, r_ref, dx_ref, dg_ref, db_ref = _oracle_bn_relu(x, gamma, beta, g)
    tol = dict(rtol=1e-4, atol=2e-5)
    np.testing.assert_allclose(out.cpu().detach().numpy(), r_ref, **tol)
    np.testing.assert_allclose(xt.grad, dx_ref, **tol)
    np.testing.assert_allclose(bn.weight.grad.get(), dg_ref, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(bn.bias.grad.get(), db_ref, rtol=1e-4, atol=1e-4)


def test_batchnorm_output_with_a_second_consumer_is_recomputed_on_demand():
    """relu(bn(x)) + bn(x): the ReLU absorbs the launch, the normalised values are produced when the
    Add asks for them; gradients of both branches accumulate (no fused backward then)."""
    import pytortto_amd as tt
    from pytortto_amd import nn
    rng = np.random.default_rng(3)
    x = (1 + 2 * rng.standard_normal((4, 8, 10, 10))).astype(np.float32)
    g = rng.standard_normal(x.shape).astype(np.float32)
    gamma, beta = np.ones(8, np.float32), np.zeros(8, np.float32)
    x = _away_from_zero(x, gamma, beta)
    bn = nn.BatchNorm2d(8)
    bn.cuda()
    xt = tt.tensor(x, requires_grad=True)
    y = bn(xt.cuda())
    out = nn.functional.relu(y) + y
    out.backward(tt.tensor(g).cuda())
    y_ref, saved, rm_ref, rv_ref = oracle.batch_norm_forward(x, gamma, beta, np.zeros(8, np.float32),
                                                              np.ones(8, np.float32), True, 0.1, 1e-5)
    r_ref = np.maximum(y_ref, 0)
    dx_ref, _, _ = oracle.batch_norm_backward(g * (r_ref > 0) + g, x, gamma, saved)
    np.testing.assert_allclose(out.cpu().detach().numpy(), r_ref + y_ref, rtol=1e-4, atol=2e-5)
    np.testing.assert_allclose(xt.grad, dx_ref, rtol=1e-4, atol=2e-5)
    np.testing.assert_allclose(bn.running_mean.data.get(), rm_ref, rtol=1e-5, atol=1e-7)   # updated once
    np.testing.assert_allclose(bn.running_var.data.get(), rv_ref, rtol=1e-5)
    assert bn.num_batches_tracked.item() == 1.0


def test_anything_but_a_relu_finds_the_parked_batchnorm_done():
    import pytortto_amd as tt
    from pytortto_amd import _hip, nn, ops
    rng = np.random.default_rng(4)
    x = rng.standard_normal((4, 8, 6, 6)).astype(np.float32)
    bn = nn.BatchNorm2d(8)
    bn.cuda()
    y_ref, _, rm_ref, _ = oracle.batch_norm_forward(x, np.ones(8, np.float32), np.zeros(8, np.float32),
                                                    np.zeros(8, np.float32), np.ones(8, np.float32), True, 0.1, 1e-5)
    y = bn(tt.tensor(x).cuda())
    assert _hip.pending().__class__ is ops.DeferredBatchNorm
    np.testing.assert_allclose(bn.running_mean.data.get(), rm_ref, rtol=1e-5, atol=1e-7)    # reading a buffer flushes
    assert _hip.pending() is None
    np.testing.assert_allclose(y.cpu().detach().numpy(), y_ref, rtol=1e-5, atol=1e-5)
    # LeakyReLU does not absorb it either
    z = nn.functional.leaky_relu(bn(tt.tensor(x).cuda()), 0.1)
    np.testing.assert_allclose(z.cpu().detach().numpy(), np.maximum(y_ref * np.float32(0.1), y_ref), rtol=1e-5, atol=1e-5)
    # eval mode launches at once
    bn.eval()
    bn(tt.tensor(x).cuda())
    assert _hip.pending() is None


@pytest.mark.parametrize('n', [1, 3, 4, 1023, 4099, (1 << 20) + 3])
def test_add_relu_entry_point_matches_add_then_relu_bit_for_bit(n):
    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(n)
    a, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    if n >= 4:
        a[:4] = [np.nan, np.inf, -np.inf, -0.0]
        b[:4] = [1.0, -np.inf, 1.0, 0.0]
    ad, bd, s, want, got = hiparray(a), hiparray(b), hiparray.empty((n,)), hiparray.empty((n,)), hiparray.empty((n,))
    _hip.call('tt_add_f32', ad.ptr, bd.ptr, s.ptr, n)
    _hip.call('tt_relu_fwd_f32', s.ptr, want.ptr, n)
    _hip.call('tt_add_relu_f32', ad.ptr, bd.ptr, got.ptr, n)
    _bits_equal(got.get(), want.get(), 'add_relu')
    with np.errstate(invalid='ignore'):
        _bits_equal(got.get(), np.maximum(a + b, 0), 'add_relu vs NumPy')


@pytest.mark.parametrize('inplace', [False, True])
def test_relu_after_a_residual_add_through_the_autograd_nodes(inplace):
    """relu(a + b): the Add is parked and the ReLU absorbs it; the graph keeps AddBackward and
    ReluBackward, both operands receive dy * (y > 0) in arrays of their own."""
    import pytortto_amd as tt
    from pytortto_amd import _hip, nn, ops
    rng = np.random.default_rng(6)
    a, b = rng.standard_normal((3, 4, 5, 7)).astype(np.float32), rng.standard_normal((3, 4, 5, 7)).astype(np.float32)
    g = rng.standard_normal(a.shape).astype(np.float32)
    at, bt = _leaf(a), _leaf(b)
    s = at + bt
    assert _hip.pending().__class__ is ops.DeferredAdd
    out = nn.functional.relu(s, inplace=inplace)
    assert _hip.pending() is None
    assert out.grad_fn.__class__.__name__ == 'ReluBackward'
    assert out.grad_fn.next_functions[0][0].__class__.__name__ == 'AddBackward'
    out.backward(tt.tensor(g).cuda())
    want = np.maximum(a + b, 0)
    np.testing.assert_array_equal(out.cpu().detach().numpy(), want)
    np.testing.assert_array_equal(at.grad.get(), g * (want > 0))
    np.testing.assert_array_equal(bt.grad.get(), g * (want > 0))
    assert at.grad.ptr != bt.grad.ptr
    # a second consumer of the sum finds it computed on demand; anything but a ReLU finds it done
    at, bt = _leaf(a), _leaf(b)
    s = at + bt
    out = nn.functional.relu(s) + s
    np.testing.assert_array_equal(out.cpu().detach().numpy(), want + (a + b))
    s2 = at + bt
    np.testing.assert_array_equal(s2.data.get(), a + b)


def _leaf(values):
    import pytortto_amd as tt
    from pytortto_amd.xparray import hiparray
    return tt.Tensor(hiparray(np.ascontiguousarray(values, dtype=np.float32)), requires_grad=True)


def test_absorbed_batchnorm_output_read_after_an_optimiser_step_is_the_value_of_the_forward():
    """y = bn(x); z = relu(y); SGD.step() changes gamma and beta in place; y read afterwards must be what
    the reference stored when the forward ran (grad_nn.py:952-959), not a recomputation from the new
    parameters."""
    import pytortto_amd as tt
    from pytortto_amd import nn, optim
    rng = np.random.default_rng(11)
    x = (1 + 2 * rng.standard_normal((4, 8, 6, 6))).astype(np.float32)
    gamma, beta = rng.uniform(0.5, 1.5, 8).astype(np.float32), (0.3 * rng.standard_normal(8)).astype(np.float32)
    bn = nn.BatchNorm2d(8)
    bn.weight.data[...] = gamma
    bn.bias.data[...] = beta
    bn.cuda()
    y = bn(tt.tensor(x).cuda())
    z = nn.functional.relu(y)
    z.backward(tt.tensor(np.ones_like(x)).cuda())
    optim.SGD(bn.parameters(), lr=0.5).step()
    assert not np.allclose(bn.weight.data.get(), gamma)               # the step did move the parameters
    y_ref, _, _, _ = oracle.batch_norm_forward(x, gamma, beta, None, None, True, 0.1, 1e-5)
    np.testing.assert_allclose(y.data.get(), y_ref, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(z.data.get(), np.maximum(y_ref, 0), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize('write', ['iadd_scalar', 'iadd_array', 'fill', 'copy_', 'relu_'])
def test_absorbed_outputs_are_produced_before_an_operand_is_written_in_place(write):
    """s = a + b; r = relu(s); a is written in place; s read afterwards equals the a + b of the time the
    Add ran (autograd/grad_fcn.py:177-203 materialises it then).  The same for bn(x) with x written."""
    import pytortto_amd as tt
    from pytortto_amd import nn
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(12)
    a, b = rng.standard_normal((2, 4, 6, 6)).astype(np.float32), rng.standard_normal((2, 4, 6, 6)).astype(np.float32)

    def overwrite(t):
        if write == 'iadd_scalar':
            t.data += 1
        elif write == 'iadd_array':
            t.data += hiparray(np.full(a.shape, 2, np.float32))
        elif write == 'fill':
            t.data.fill(7.0)
        elif write == 'copy_':
            with tt.no_grad():
                t.copy_(tt.tensor(np.zeros_like(a)))
        else:
            nn.functional.relu(t, inplace=True)

    at, bt = tt.Tensor(hiparray(a)), tt.Tensor(hiparray(b))
    s = at + bt
    r = nn.functional.relu(s)
    overwrite(at)
    assert not np.array_equal(at.data.get(), a)
    np.testing.assert_array_equal(s.data.get(), a + b)
    np.testing.assert_array_equal(r.data.get(), np.maximum(a + b, 0))

    x = (1 + 2 * a).astype(np.float32)
    bn = nn.BatchNorm2d(4)
    bn.cuda()
    xt = tt.Tensor(hiparray(x))
    y = bn(xt)
    r = nn.functional.relu(y)
    overwrite(xt)
    y_ref, _, _, _ = oracle.batch_norm_forward(x, np.ones(4, np.float32), np.zeros(4, np.float32), None, None, True,
                                               0.1, 1e-5)
    np.testing.assert_allclose(y.data.get(), y_ref, rtol=1e-5, atol=1e-5)


def test_a_parked_operation_is_seen_by_a_second_thread():
    """Thread B reads the output of an operation thread A parked: it must find it run (one slot shared
    by all threads, behind a lock), and two threads parking and fusing at once must not mix their ops."""
    import threading
    import pytortto_amd as tt
    from pytortto_amd import _hip, nn, ops
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(13)
    a, b = rng.standard_normal((64, 33)).astype(np.float32), rng.standard_normal((64, 33)).astype(np.float32)
    s = tt.Tensor(hiparray(a)) + tt.Tensor(hiparray(b))
    assert _hip.pending().__class__ is ops.DeferredAdd
    got = {}
    t = threading.Thread(target=lambda: got.setdefault('s', s.data.get()))
    t.start()
    t.join()
    np.testing.assert_array_equal(got['s'], a + b)

    errors = []

    def worker(seed):
        try:
            r = np.random.default_rng(seed)
            for _ in range(50):
                u, v = r.standard_normal((8, 16)).astype(np.float32), r.standard_normal((8, 16)).astype(np.float32)
                out = nn.functional.relu(tt.Tensor(hiparray(u)) + tt.Tensor(hiparray(v)))
                np.testing.assert_array_equal(out.data.get(), np.maximum(u + v, 0))
        except Exception as exc:           # reported by the main thread
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
