"""Shared convolution parameter grids for the oracle and GPU parity tests."""

# (N, C, H, W, K, R, S, stride, padding, dilation, groups)
CONV_CASES = [
    (2, 4, 8, 8, 6, 3, 3, (1, 1), (1, 1), (1, 1), 1),
    (2, 4, 8, 8, 6, 3, 3, (2, 2), (1, 1), (1, 1), 1),     # (H+2p-d(R-1)-1) % s != 0: uncovered rows
    (2, 4, 9, 7, 6, 3, 2, (2, 1), (0, 1), (1, 2), 2),
    (1, 6, 10, 11, 4, 2, 3, (3, 2), (2, 0), (2, 1), 2),
    (3, 3, 7, 7, 5, 1, 1, (1, 1), (0, 0), (1, 1), 1),     # 1x1: plain matrix product
    (2, 4, 8, 8, 8, 1, 1, (2, 2), (0, 0), (1, 1), 1),     # 1x1 stride 2 (shortcut): 3/4 of dx is zero
    (2, 3, 12, 12, 4, 7, 7, (2, 2), (3, 3), (1, 1), 1),   # stem-like
    (2, 8, 6, 5, 8, 3, 3, (1, 1), (2, 2), (2, 2), 4),
    (1, 2, 5, 5, 2, 5, 5, (1, 1), (0, 0), (1, 1), 1),     # kernel == input
    (2, 4, 8, 8, 4, 4, 4, (2, 2), (1, 1), (1, 1), 1),     # DCGAN-style geometry, as a conv
    (2, 6, 9, 9, 3, 3, 3, (3, 3), (1, 1), (1, 1), 3),     # stride 3 with dead input rows
    (2, 4, 11, 10, 6, 3, 3, (2, 3), (1, 2), (2, 1), 1),   # gcd(stride, dilation) > 1 in H
]

# (N, C_in, H, W, C_out, R, S, stride, padding, output_padding, dilation, groups)
CONVT_CASES = [
    (2, 5, 1, 1, 6, 4, 4, (1, 1), (0, 0), (0, 0), (1, 1), 1),   # DCGAN first layer geometry
    (2, 6, 4, 4, 4, 4, 4, (2, 2), (1, 1), (0, 0), (1, 1), 1),   # DCGAN upsampling geometry
    (2, 4, 5, 6, 6, 3, 3, (2, 2), (1, 1), (1, 1), (1, 1), 2),
    (1, 4, 5, 4, 2, 3, 2, (3, 2), (1, 0), (2, 1), (2, 1), 2),
    (2, 3, 6, 6, 5, 1, 1, (1, 1), (0, 0), (0, 0), (1, 1), 1),
    (2, 4, 4, 5, 4, 3, 3, (2, 2), (0, 0), (1, 0), (2, 2), 1),   # gcd(stride, dilation) = 2
    (1, 2, 3, 3, 2, 2, 2, (3, 3), (0, 0), (2, 2), (1, 1), 1),   # stride > kernel: holes in the output
]

# (N, C, H, W, kernel, stride, padding, dilation, ceil_mode)
POOL_CASES = [
    (2, 3, 8, 8, (2, 2), (2, 2), (0, 0), (1, 1), False),      # non-overlapping
    (2, 3, 9, 7, (3, 3), (2, 2), (1, 1), (1, 1), False),      # ResNet stem geometry: overlapping windows
    (1, 4, 12, 12, (3, 3), (2, 2), (1, 1), (1, 1), True),     # ceil_mode adds a partial window
    (2, 2, 10, 11, (3, 2), (1, 2), (1, 0), (1, 1), False),    # stride 1 in H: heavy overlap
    (2, 2, 11, 10, (2, 3), (2, 1), (1, 1), (2, 2), False),    # dilation
    (1, 3, 7, 7, (3, 3), (3, 3), (0, 0), (1, 1), True),       # ceil_mode, window hanging over the edge
    (1, 2, 6, 6, (2, 2), (2, 2), (1, 1), (1, 1), True),       # ceil_mode whose last window is dropped
    (3, 1, 5, 9, (5, 3), (1, 3), (2, 1), (1, 1), False),      # tall kernel
    (2, 2, 8, 8, (2, 2), (3, 3), (0, 0), (1, 1), False),      # stride > kernel: uncovered pixels
]


def random_pool_cases(count, seed):
    """Seeded random pooling geometries (kernel, stride, padding <= kernel / 2, dilation, ceil_mode)."""
    import numpy as np
    import oracle
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        ks = (int(rng.integers(1, 6)), int(rng.integers(1, 6)))
        st = (int(rng.integers(1, 5)), int(rng.integers(1, 5)))
        pd = (int(rng.integers(0, ks[0] // 2 + 1)), int(rng.integers(0, ks[1] // 2 + 1)))
        dl = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        cm = bool(rng.integers(0, 2))
        h, w = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        if min(oracle.pool_output_size(h, ks[0], st[0], pd[0], dl[0], cm),
               oracle.pool_output_size(w, ks[1], st[1], pd[1], dl[1], cm)) < 1:
            continue
        cases.append((int(rng.integers(1, 4)), int(rng.integers(1, 6)), h, w, ks, st, pd, dl, cm))
    return cases


def random_conv_cases(count, seed):
    """Seeded random geometries: every combination of stride, padding, dilation and groups the
    validation admits, with sizes that are not multiples of any tile."""
    import numpy as np
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        g = int(rng.choice([1, 1, 1, 2, 3, 4]))
        c, k = g * int(rng.integers(1, 24)), g * int(rng.integers(1, 24))
        r, s = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        st = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        dl = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        pd = (int(rng.integers(0, 4)), int(rng.integers(0, 4)))
        h, w = int(rng.integers(1, 23)), int(rng.integers(1, 23))
        n = int(rng.integers(1, 6))
        if h + 2 * pd[0] < dl[0] * (r - 1) + 1 or w + 2 * pd[1] < dl[1] * (s - 1) + 1:
            continue
        cases.append((n, c, h, w, k, r, s, st, pd, dl, g))
    return cases


def random_large_kernel_cases(count, seed):
    """Seeded random geometries with kernels of 26 to 81 taps: beyond a 32-bit tap mask (31 taps) the
    device kernels keep 64-bit masks, beyond 63 taps they compare bounds per element."""
    import numpy as np
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        g = int(rng.choice([1, 1, 2]))
        c, k = g * int(rng.integers(1, 12)), g * int(rng.integers(1, 20))
        r, s = int(rng.integers(3, 10)), int(rng.integers(3, 10))
        if r * s < 26:
            continue
        st = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        dl = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        pd = (int(rng.integers(0, 6)), int(rng.integers(0, 6)))
        h, w = int(rng.integers(6, 30)), int(rng.integers(6, 30))
        n = int(rng.integers(1, 5))
        if h + 2 * pd[0] < dl[0] * (r - 1) + 1 or w + 2 * pd[1] < dl[1] * (s - 1) + 1:
            continue
        cases.append((n, c, h, w, k, r, s, st, pd, dl, g))
    return cases


def random_convt_cases(count, seed):
    """Seeded random transposed-convolution geometries with output_padding < stride: what the
    reference's own `output_size` path can produce (nn/modules/conv.py:137-153); beyond that its
    backward returns an input gradient larger than the input."""
    import numpy as np
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        g = int(rng.choice([1, 1, 2, 3]))
        ci, co = g * int(rng.integers(1, 16)), g * int(rng.integers(1, 16))
        r, s = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        st = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        dl = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        pd = (int(rng.integers(0, 3)), int(rng.integers(0, 3)))
        op = (int(rng.integers(0, st[0])), int(rng.integers(0, st[1])))
        h, w = int(rng.integers(1, 12)), int(rng.integers(1, 12))
        ho = (h - 1) * st[0] - 2 * pd[0] + dl[0] * (r - 1) + op[0] + 1
        wo = (w - 1) * st[1] - 2 * pd[1] + dl[1] * (s - 1) + op[1] + 1
        if ho < 1 or wo < 1:
            continue
        cases.append((int(rng.integers(1, 5)), ci, h, w, co, r, s, st, pd, op, dl, g))
    return cases
