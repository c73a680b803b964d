"""Host-only: the index tables behind the convolution forward, input gradient and weight gradient,
checked through the C ABI without a device (``tt_conv2d_check_tables_*``).

The kernels address the gathered operand through per-geometry tables (reduction index -> offset
and tap).  The library builds them on the host and replays every entry for the extreme pixels of
its tap under the kernel's own bounds rule: the element reached must be the one the reference pairs
with that reduction index (``grad_nn.py:603-611`` forward, ``:659-682`` input gradient) and lie inside
the tensor; 32-bit buffer offsets must stay in range.  The weight gradient's table has one entry
per output pixel (``grad_nn.py:646-656``: image, dy offset, x window offset, padding bits), each
checked tap by tap.  Here that check runs over the benchmark's
layer shapes at their full batch sizes, the geometries of the GPU parity tests (tile shapes,
large images, dense few-channel input gradients with every cell size) and seeded random ones.
"""
import ctypes

import pytest

from tests.cases import CONV_CASES, CONVT_CASES, random_conv_cases, random_convt_cases, random_large_kernel_cases


def _lib():
    from pytortto_amd import _hip
    return _hip.load_library()


def _ok(rc):
    assert rc == 0, _lib().tt_last_error().decode()


def _out(size, k, s, p, d):
    return (size + 2 * p - d * (k - 1) - 1) // s + 1


def _check_conv(case):
    n, c, h, w, k, r, s, st, pd, dl, g = case
    p, q = _out(h, r, st[0], pd[0], dl[0]), _out(w, s, st[1], pd[1], dl[1])
    geo = (r, s, st[0], st[1], pd[0], pd[1], dl[0], dl[1], g)
    _ok(_lib().tt_conv2d_check_tables_fwd_f32(n, c, h, w, k, *geo))
    _ok(_lib().tt_conv2d_check_tables_dgrad_f32(n, c, h, w, k, *geo, p, q))
    _ok(_lib().tt_conv2d_check_tables_wgrad_f32(n, c, h, w, k, *geo, p, q))


def _check_convt(case):
    """ConvTranspose2d forward is the input gradient of the convolution with the same geometry."""
    n, ci, h, w, co, r, s, st, pd, op, dl, g = case
    ho = (h - 1) * st[0] - 2 * pd[0] + dl[0] * (r - 1) + op[0] + 1
    wo = (w - 1) * st[1] - 2 * pd[1] + dl[1] * (s - 1) + op[1] + 1
    geo = (r, s, st[0], st[1], pd[0], pd[1], dl[0], dl[1], g)
    _ok(_lib().tt_conv2d_check_tables_dgrad_f32(n, co, ho, wo, ci, *geo, h, w))
    _ok(_lib().tt_conv2d_check_tables_fwd_f32(n, co, ho, wo, ci, *geo))     # its input gradient
    _ok(_lib().tt_conv2d_check_tables_wgrad_f32(n, co, ho, wo, ci, *geo, h, w))   # x := gy, dy := the layer's input


def test_table_check_refuses_damaged_tables():
    """Single entries moved by one element, one row or one image, in both addressing modes,
    forward and input gradient: each damaged table is refused, each undamaged one accepted."""
    _ok(_lib().tt_conv2d_check_tables_selftest())


def test_pixel_table_check_refuses_damaged_tables():
    """Weight gradient: a wrong image index, dy offset, x offset or tap bit (let through in the
    padding, or blocked inside the image) in one entry, 32- and 64-bit masks: each is refused."""
    _ok(_lib().tt_conv2d_check_tables_selftest_wgrad())


def test_weight_gradient_refuses_a_dy_that_does_not_belong_to_the_geometry():
    """P, Q beyond what (H, R, stride, padding, dilation) allow: the roles of x and dy mixed up."""
    lib = _lib()
    geo = (3, 3, 2, 2, 1, 1, 1, 1, 1)
    _ok(lib.tt_conv2d_check_tables_wgrad_f32(2, 4, 9, 9, 6, *geo, 5, 5))
    _ok(lib.tt_conv2d_check_tables_wgrad_f32(2, 4, 9, 9, 6, *geo, 4, 5))          # cropped: fewer windows is fine
    assert lib.tt_conv2d_check_tables_wgrad_f32(2, 4, 9, 9, 6, *geo, 6, 5) != 0
    assert b'does not belong to this geometry' in lib.tt_last_error()
    assert lib.tt_conv2d_check_tables_wgrad_f32(2, 4, 9, 9, 6, *geo, 5, 9) != 0
    assert lib.tt_conv2d_check_tables_wgrad_f32(2, 4, 2, 2, 6, 5, 5, 1, 1, 0, 0, 1, 1, 1, 1, 1) != 0
    assert b'larger than padded input' in lib.tt_last_error()


def test_tables_of_the_benchmark_configurations():
    import bench
    for c, h, k, r, s, p, _ in bench.RESNET50_CONVS:                     # ResNet-50, batch 64
        _check_conv((64, c, h, h, k, r, r, (s, s), (p, p), (1, 1), 1))
    _check_conv((32, 16, 32, 32, 32, 3, 3, (1, 1), (1, 1), (1, 1), 1))   # the single-layer configuration
    cin = 3                                                             # PreAct-ResNet-18 stack, batch 128
    _check_conv((128, 3, 32, 32, 64, 3, 3, (1, 1), (1, 1), (1, 1), 1))
    size, cin = 32, 64
    for cout, stride in ((64, 1), (128, 2), (256, 2), (512, 2)):
        _check_conv((128, cin, size, size, cout, 3, 3, (stride, stride), (1, 1), (1, 1), 1))
        if stride != 1:
            _check_conv((128, cin, size, size, cout, 1, 1, (stride, stride), (0, 0), (1, 1), 1))
        size //= stride
        _check_conv((128, cout, size, size, cout, 3, 3, (1, 1), (1, 1), (1, 1), 1))
        cin = cout
    chans = [100, 512, 256, 128, 64, 3]                                  # DCGAN generator, batch 128
    size = 1
    for i in range(5):
        st, pd = ((1, 1), (0, 0)) if i == 0 else ((2, 2), (1, 1))
        _check_convt((128, chans[i], size, size, chans[i + 1], 4, 4, st, pd, (0, 0), (1, 1), 1))
        size = 4 if i == 0 else size * 2


def test_tables_of_the_parity_test_geometries():
    from tests.test_gpu_conv import LARGE_IMAGE_CASES, TILE_CASES
    for case in CONV_CASES + TILE_CASES + LARGE_IMAGE_CASES:
        _check_conv(case)
    for case in CONVT_CASES:
        _check_convt(case)


def test_dense_input_gradient_tables_with_every_cell_size():
    """Few-channel strided layers: with the tile-count threshold lifted the planner takes the
    larger cells (two or four stride periods side by side) also on small inputs."""
    from tests.test_gpu_conv import TILE_CASES
    lib = _lib()
    few = [c for c in TILE_CASES if c[1] <= 5 and c[7] != (1, 1)]
    assert len(few) >= 8
    _ok(lib.tt_set_conv_dense_cell_min_tiles(0))
    try:
        for case in few:
            _check_conv(case)
        _check_conv((64, 3, 224, 224, 64, 7, 7, (2, 2), (3, 3), (1, 1), 1))
        _check_convt((128, 64, 32, 32, 3, 4, 4, (2, 2), (1, 1), (0, 0), (1, 1), 1))
    finally:
        _ok(lib.tt_set_conv_dense_cell_min_tiles(-1))      # back to the default


@pytest.mark.parametrize('seed', [5, 6, 7])
def test_tables_of_random_geometries(seed):
    for case in random_conv_cases(150, seed):
        _check_conv(case)
    for case in random_convt_cases(100, seed):
        _check_convt(case)
    for case in random_large_kernel_cases(100, seed):   # 64-bit tap masks, and the fall-back beyond 63 taps
        _check_conv(case)


def test_table_check_reports_unsupported_geometries_instead_of_tables():
    lib = _lib()
    assert lib.tt_conv2d_check_tables_fwd_f32(1, 4, 8, 8, 6, 3, 3, 1, 1, 1, 1, 1, 1, 3) != 0      # channels vs groups
    assert b'groups' in lib.tt_last_error()
    assert lib.tt_conv2d_check_tables_fwd_f32(1, 4, 2, 2, 4, 5, 5, 1, 1, 0, 0, 1, 1, 1) != 0      # kernel larger than input
    assert b'larger than padded input' in lib.tt_last_error()
