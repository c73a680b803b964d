"""GPU parity: BatchNorm2d training forward/backward through the C ABI vs the CPU oracle."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

# outputs and running statistics: rtol 1e-5.  Two correct float32 evaluations of
# (x-mean)/sd*gamma+beta differ by ~1 ulp of the larger term, so where the two terms cancel to a y
# near zero the element-wise relative error has no bound; such elements -- and only such -- fall
# back on an absolute floor of 2e-6 of the tensor's magnitude.  _close() checks that the floor is
# used nowhere else: every element outside the pure rtol must be smaller than 5 % of the tensor's
# magnitude, and in tensors of 4096 elements or more they must be fewer than 2 % of it (measured:
# 0.1 - 1.0 % of y, where gamma * xhat and beta cancel to within a few percent; 2 - 4e-6 of dx).
RTOL = 1e-5


def _close(got, ref, rtol=RTOL, atol_scale=2e-6, name=''):
    """Returns the share of elements that needed the absolute floor."""
    got, ref = np.asarray(got), np.asarray(ref)
    scale = float(np.abs(ref).max()) or 1.0
    np.testing.assert_allclose(got, ref, rtol=rtol, atol=atol_scale * scale, err_msg=name)
    outside = np.abs(got - ref) > rtol * np.abs(ref)
    share = float(outside.mean()) if outside.size else 0.0
    if outside.any():
        assert float(np.abs(ref[outside]).max()) <= 0.05 * scale, f'{name}: the floor was needed away from zero'
        if ref.size >= 4096:
            assert share <= 2e-2, f'{name}: {share:.2%} of the elements needed the floor'
    return share


def _inputs(shape, seed=0):
    np.random.seed(seed)
    c = shape[1]
    x = (2 + 3 * np.random.randn(*shape)).astype(np.float32)
    gamma, beta = oracle.bn_affine_c4(c)
    dy = np.random.randn(*shape).astype(np.float32)
    return x, gamma, beta, dy


SHAPES = [
    (4, 3, 5, 5),        # flat scalar kernel, tiny
    (2, 8, 1, 3),
    (16, 5, 4, 4),       # flat float4 kernel
    (8, 64, 14, 14),     # flat float4 (HW/4 = 49)
    (8, 32, 7, 7),       # flat scalar, HW = 49
    (6, 16, 16, 16),     # plane kernel, HW/4 = 64
    (5, 7, 24, 20),      # plane kernel, ragged plane count per block
    (64, 64, 28, 28),    # plane kernel with several splits per channel
    (128, 4, 32, 32),    # few channels: maximum number of splits
    # the BatchNorm shapes of the PreAct-ResNet-18 stack at its own batch size
    (128, 64, 32, 32), (128, 128, 16, 16), (128, 256, 8, 8), (128, 512, 4, 4),
]


@pytest.mark.parametrize('shape', SHAPES)
def test_bn_train_fwd_bwd_matches_oracle(shape):
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    x, gamma, beta, dy = _inputs(shape)
    c = shape[1]
    rm0 = np.zeros(c, np.float32)
    rv0 = np.ones(c, np.float32)
    y_ref, saved, rm_ref, rv_ref = oracle.batch_norm_forward(x, gamma, beta, rm0, rv0, True, 0.1, 1e-5)
    dx_ref, dg_ref, db_ref = oracle.batch_norm_backward(dy, x, gamma, saved)

    xd, gd, bd, dyd = hiparray(x), hiparray(gamma), hiparray(beta), hiparray(dy)
    y, mean, var_eps, sd, rm, rv = ops.bn_fwd_train(xd, gd, bd, hiparray(rm0), hiparray(rv0), 0.1, 1e-5)
    dx, dg, db = ops.bn_bwd(xd, dyd, gd, mean, var_eps, sd)

    _close(y.get(), y_ref, name='y')
    _close(mean.get(), saved['mean'].ravel(), name='mean')
    _close(var_eps.get(), saved['var'].ravel(), name='var+eps')
    _close(sd.get(), saved['sd'].ravel(), name='sd')
    _close(rm.get(), rm_ref, name='running_mean')
    _close(rv.get(), rv_ref, name='running_var')
    # gradients: long float32 reductions with cancellation on the CPU side -> compare against
    # float64 truth as well and require the GPU to be at least as close as the oracle
    x64, dy64 = x.astype(np.float64), dy.astype(np.float64)
    y64, saved64, _, _ = oracle.batch_norm_forward(x64, gamma.astype(np.float64), beta.astype(np.float64),
                                                   None, None, True, 0.1, 1e-5)
    dx64, dg64, db64 = oracle.batch_norm_backward(dy64, x64, gamma.astype(np.float64), saved64)
    for got, ref32, ref64, name in ((dx.get(), dx_ref, dx64, 'dx'), (dg.get(), dg_ref, dg64, 'dgamma'),
                                    (db.get(), db_ref, db64, 'dbeta')):
        scale = float(np.abs(ref64).max()) or 1.0
        err_gpu = float(np.abs(got - ref64).max()) / scale
        err_cpu = float(np.abs(ref32 - ref64).max()) / scale
        assert err_gpu <= max(2 * err_cpu, 2e-6), (name, err_gpu, err_cpu)
        _close(got, ref32, rtol=1e-4, atol_scale=1e-5, name=name)


def test_bn_without_affine_and_without_running_stats():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    x, _, _, dy = _inputs((6, 16, 16, 16), seed=3)
    y_ref, saved, rm_ref, rv_ref = oracle.batch_norm_forward(x, None, None, None, None, True, 0.1, 1e-5)
    dx_ref, _, _ = oracle.batch_norm_backward(dy, x, None, saved, need=(True, False, False))
    xd = hiparray(x)
    y, mean, var_eps, sd, rm, rv = ops.bn_fwd_train(xd, None, None, None, None, 0.1, 1e-5)
    assert rm is None and rv is None
    dx, dg, db = ops.bn_bwd(xd, hiparray(dy), None, mean, var_eps, sd, need=(True, False, False))
    assert dg is None and db is None
    _close(y.get(), y_ref)
    _close(dx.get(), dx_ref, rtol=1e-4, atol_scale=1e-5)


def test_bn_running_stats_recurrence_three_steps():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    c = 16
    rm, rv = np.zeros(c, np.float32), np.ones(c, np.float32)
    rmd, rvd = hiparray(rm), hiparray(rv)
    for step in range(3):
        x, gamma, beta, _ = _inputs((6, c, 16, 16), seed=10 + step)
        _, _, rm, rv = oracle.batch_norm_forward(x, gamma, beta, rm, rv, True, 0.3, 1e-5)
        _, _, _, _, rmd, rvd = ops.bn_fwd_train(hiparray(x), hiparray(gamma), hiparray(beta), rmd, rvd, 0.3, 1e-5)
    _close(rmd.get(), rm)
    _close(rvd.get(), rv)


def test_bn_eval_mode_matches_oracle():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    x, gamma, beta, dy = _inputs((6, 16, 16, 16), seed=5)
    rm = np.linspace(1, 3, 16).astype(np.float32)
    rv = np.linspace(4, 12, 16).astype(np.float32)
    y_ref, saved, _, _ = oracle.batch_norm_forward(x, gamma, beta, rm, rv, False, 0.1, 1e-5)
    dx_ref, dg_ref, db_ref = oracle.batch_norm_backward(dy, x, gamma, saved)
    xd, gd = hiparray(x), hiparray(gamma)
    y, mean, var_eps, sd = ops.bn_fwd_eval(xd, gd, hiparray(beta), hiparray(rm), hiparray(rv), 1e-5)
    dx, dg, db = ops.bn_bwd(xd, hiparray(dy), gd, mean, var_eps, sd)
    _close(y.get(), y_ref)
    _close(dx.get(), dx_ref, rtol=1e-4, atol_scale=1e-5)
    _close(dg.get(), dg_ref, rtol=1e-4, atol_scale=1e-5)
    _close(db.get(), db_ref, rtol=1e-4, atol_scale=1e-5)


def test_bn_large_mean_small_sigma_is_stable():
    """|mean| >> sigma: a raw E[x^2]-E[x]^2 in float32 would lose every digit of the variance."""
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    np.random.seed(7)
    x = (1000 + 0.5 * np.random.randn(8, 16, 16, 16)).astype(np.float32)
    var64 = x.astype(np.float64).var((0, 2, 3))
    _, mean, var_eps, _, _, _ = ops.bn_fwd_train(hiparray(x), None, None, None, None, 0.1, 0.0)
    np.testing.assert_allclose(var_eps.get(), var64, rtol=1e-4)
    np.testing.assert_allclose(mean.get(), x.astype(np.float64).mean((0, 2, 3)), rtol=1e-6)


def test_bn_single_value_per_channel_is_an_error():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    with pytest.raises(RuntimeError, match='Expected more than 1 value per channel'):
        ops.bn_fwd_train(hiparray(np.zeros((1, 3, 1, 1), np.float32)), None, None, None, None, 0.1, 1e-5)


def test_channel_sum_matches_numpy():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    np.random.seed(2)
    for shape in [(4, 6, 5, 5), (32, 32, 32, 32), (3, 5, 8, 4)]:
        t = np.random.randn(*shape).astype(np.float32)
        ref = t.astype(np.float64).sum((0, 2, 3))
        got = ops.channel_sum(hiparray(t)).get()
        np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-5 * np.abs(ref).max())


@pytest.mark.parametrize('shape', [(64, 256, 56, 56), (128, 64, 112, 112)])
def test_bn_benchmark_shapes_full_size(shape):
    """The two shapes the BatchNorm metric is quoted on, x ~ N(2, 3): the float32 oracle for y, dx
    and the statistics; float64 reductions for the per-channel sums; and what the algebra fixes:
    mean(y) = beta, var(y) = gamma^2 var / (var + eps), sum(dx) = 0, sum(dx * xhat) = 0."""
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(11)
    n, c, h, w = shape
    x = (2 + 3 * rng.standard_normal(shape, dtype=np.float32)).astype(np.float32)
    dy = rng.standard_normal(shape, dtype=np.float32)
    gamma = rng.uniform(0.5, 1.5, c).astype(np.float32)
    beta = (0.1 * rng.standard_normal(c)).astype(np.float32)
    rm0, rv0 = np.zeros(c, np.float32), np.ones(c, np.float32)
    xd, dyd, gd = hiparray(x), hiparray(dy), hiparray(gamma)
    y, mean, var_eps, sd, rm, rv = ops.bn_fwd_train(xd, gd, hiparray(beta), hiparray(rm0), hiparray(rv0), 0.1, 1e-5)
    dx, dg, db = ops.bn_bwd(xd, dyd, gd, mean, var_eps, sd)
    y, dx = y.get(), dx.get()

    axis, m = (0, 2, 3), n * h * w
    mu64 = x.mean(axis, dtype=np.float64)
    var64 = ((x.astype(np.float64) - mu64[None, :, None, None]) ** 2).mean(axis)
    np.testing.assert_allclose(mean.get(), mu64, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(var_eps.get(), var64 + 1e-5, rtol=2e-6)
    np.testing.assert_allclose(rm.get(), 0.1 * mu64, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(rv.get(), 0.9 + 0.1 * var64 * (m / (m - 1)), rtol=1e-5)

    y_ref, saved, rm_ref, rv_ref = oracle.batch_norm_forward(x, gamma, beta, rm0, rv0, True, 0.1, 1e-5)
    share_y = _close(y, y_ref, name='y')
    _close(rm.get(), rm_ref, name='running_mean')
    _close(rv.get(), rv_ref, name='running_var')
    np.testing.assert_allclose(y.mean(axis, dtype=np.float64), beta, atol=2e-6)
    np.testing.assert_allclose(y.var(axis, dtype=np.float64), gamma.astype(np.float64) ** 2 * var64 / (var64 + 1e-5),
                               rtol=1e-5)

    dx_ref, dg_ref, db_ref = oracle.batch_norm_backward(dy, x, gamma, saved)
    xhat = (x.astype(np.float64) - mu64[None, :, None, None]) / np.sqrt(var64 + 1e-5)[None, :, None, None]
    db64 = dy.sum(axis, dtype=np.float64)
    dg64 = (dy * xhat).sum(axis)
    np.testing.assert_allclose(db.get(), db64, rtol=1e-5, atol=1e-5 * np.abs(db64).max())
    np.testing.assert_allclose(dg.get(), dg64, rtol=1e-5, atol=1e-5 * np.abs(dg64).max())
    share_dx = _close(dx, dx_ref, rtol=1e-4, atol_scale=1e-5, name='dx')
    print(f'BatchNorm {shape}: share of elements outside the pure relative tolerance: y {share_y:.2e} (rtol 1e-5), '
          f'dx {share_dx:.2e} (rtol 1e-4)')
    scale = float(np.abs(dx).sum(axis, dtype=np.float64).max())
    assert np.abs(dx.sum(axis, dtype=np.float64)).max() <= 1e-5 * scale
    assert np.abs((dx * xhat).sum(axis)).max() <= 1e-4 * scale          # exact only up to O(eps / var)


def _random_bn_shapes(count, seed):
    rng = np.random.default_rng(seed)
    shapes = []
    while len(shapes) < count:
        n, c = int(rng.integers(1, 40)), int(rng.integers(1, 70))
        h, w = int(rng.integers(1, 30)), int(rng.integers(1, 30))
        if n * h * w < 2:
            continue
        shapes.append((n, c, h, w))
    return shapes


@pytest.mark.parametrize('shape', _random_bn_shapes(40, 31), ids=lambda s: '%dx%dx%dx%d' % s)
def test_bn_random_shapes(shape):
    test_bn_train_fwd_bwd_matches_oracle(shape)


# at least 128 channels of at most 16384 values each: the single-kernel passes (one block per channel
# keeps the channel in registers); the last two sit just inside and just outside that limit
SMALL_CHANNEL_SHAPES = [
    (64, 256, 7, 7),      # 3136 values: 256 threads x 16 values
    (32, 128, 14, 14),    # 6272 values, few channels: 1024 threads x 16 values, partly filled
    (64, 256, 14, 14),    # 12544 values, 256 channels (ResNet-50's 14x14 stage): 1024 threads x 16
    (16, 640, 20, 20),    # 6400 values, more channels than two blocks per CU: 256 threads x 64 values
    (64, 1024, 14, 14),   # the same at ResNet-50's size
    (2, 128, 1, 1),       # two values per channel
    (3, 200, 5, 7),       # odd plane, threads without a value
    (128, 512, 4, 4),     # DCGAN / PreAct-ResNet-18 deepest layers
    (16, 130, 31, 33),    # 16368 values
    (64, 128, 16, 16),    # 16384 values: exactly the capacity
    (65, 128, 16, 16),    # 16640 values: back on the two-sweep kernels
]


@pytest.mark.parametrize('shape', SMALL_CHANNEL_SHAPES, ids=lambda s: '%dx%dx%dx%d' % s)
def test_bn_small_channels_single_kernel(shape):
    test_bn_train_fwd_bwd_matches_oracle(shape)


def test_bn_small_channels_optional_arguments_and_stability():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    shape = (16, 160, 9, 9)
    x, gamma, beta, dy = _inputs(shape, seed=8)
    # no affine parameters, no running statistics, only dx wanted
    y_ref, saved, _, _ = oracle.batch_norm_forward(x, None, None, None, None, True, 0.1, 1e-5)
    dx_ref, _, _ = oracle.batch_norm_backward(dy, x, None, saved, need=(True, False, False))
    xd, dyd = hiparray(x), hiparray(dy)
    y, mean, var_eps, sd, rm, rv = ops.bn_fwd_train(xd, None, None, None, None, 0.1, 1e-5)
    assert rm is None and rv is None
    dx, dg, db = ops.bn_bwd(xd, dyd, None, mean, var_eps, sd, need=(True, False, False))
    assert dg is None and db is None
    _close(y.get(), y_ref)
    _close(dx.get(), dx_ref, rtol=1e-4, atol_scale=1e-5)
    # only the parameter gradients wanted
    gd = hiparray(gamma)
    y_ref, saved, _, _ = oracle.batch_norm_forward(x, gamma, beta, None, None, True, 0.1, 1e-5)
    _, dg_ref, db_ref = oracle.batch_norm_backward(dy, x, gamma, saved)
    _, mean, var_eps, sd, _, _ = ops.bn_fwd_train(xd, gd, hiparray(beta), None, None, 0.1, 1e-5)
    dx, dg, db = ops.bn_bwd(xd, dyd, gd, mean, var_eps, sd, need=(False, True, True))
    assert dx is None
    _close(dg.get(), dg_ref, rtol=1e-4, atol_scale=1e-5)
    _close(db.get(), db_ref, rtol=1e-4, atol_scale=1e-5)
    # |mean| >> sigma
    np.random.seed(9)
    xs = (1000 + 0.5 * np.random.randn(8, 128, 12, 12)).astype(np.float32)
    _, mean, var_eps, _, _, _ = ops.bn_fwd_train(hiparray(xs), None, None, None, None, 0.1, 0.0)
    np.testing.assert_allclose(var_eps.get(), xs.astype(np.float64).var((0, 2, 3)), rtol=1e-4)
    np.testing.assert_allclose(mean.get(), xs.astype(np.float64).mean((0, 2, 3)), rtol=1e-6)
    # running statistics over three steps
    c = 144
    rm, rv = np.zeros(c, np.float32), np.ones(c, np.float32)
    rmd, rvd = hiparray(rm), hiparray(rv)
    for step in range(3):
        x, gamma, beta, _ = _inputs((6, c, 10, 10), seed=20 + step)
        _, _, rm, rv = oracle.batch_norm_forward(x, gamma, beta, rm, rv, True, 0.3, 1e-5)
        _, _, _, _, rmd, rvd = ops.bn_fwd_train(hiparray(x), hiparray(gamma), hiparray(beta), rmd, rvd, 0.3, 1e-5)
    _close(rmd.get(), rm)
    _close(rvd.get(), rv)
