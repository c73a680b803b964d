"""The host-side model of bfloat16 rounding used to pin the optional bf16 convolution variant."""
import numpy as np
import torch

from tests.brute import bf16_round


def test_ties_go_to_even_and_low_bits_are_cleared():
    # 1 + 2^-8 lies halfway between 1 and 1 + 2^-7: to even (1); 1 + 3*2^-8 goes to 1 + 2^-6
    a = np.array([1.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, -3.1415927, 0.0], np.float32)
    r = bf16_round(a)
    assert r[0] == 1.0 and r[1] == 1.0 and r[2] == np.float32(1.0 + 2.0 ** -6) and r[3] == np.float32(1.0 + 2.0 ** -7)
    assert r[4] == np.float32(-3.140625) and r[5] == 0.0
    assert np.all((r.view(np.uint32) & 0xffff) == 0)


def test_matches_torch_bfloat16_cast():
    rng = np.random.default_rng(0)
    a = (rng.standard_normal((64, 257)) * np.exp(rng.uniform(-20, 20, (64, 257)))).astype(np.float32)
    ref = torch.from_numpy(a).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(bf16_round(a), ref)


def _three_terms(a):
    """What the kernels of the 'bf16x3' convolution arithmetic make of a float32 value."""
    t0 = bf16_round(a)
    r1 = (a - t0).astype(np.float32)
    t1 = bf16_round(r1)
    r2 = (r1 - t1).astype(np.float32)
    return t0, t1, bf16_round(r2), r1, r2


def test_three_bf16_terms_add_up_to_the_float32_value_exactly():
    rng = np.random.default_rng(1)
    a = (rng.standard_normal((64, 513)) * np.exp(rng.uniform(-60, 60, (64, 513)))).astype(np.float32)
    a[0, :8] = [0.0, -0.0, 1.0, -1.0, 1.0 + 2.0 ** -23, 1.0 - 2.0 ** -24, 3.3e38, 2.0 ** -100]
    t0, t1, t2, r1, r2 = _three_terms(a)
    # every difference the kernel takes is exact in float32 ...
    np.testing.assert_array_equal(r1.astype(np.float64), a.astype(np.float64) - t0.astype(np.float64))
    np.testing.assert_array_equal(r2.astype(np.float64), r1.astype(np.float64) - t1.astype(np.float64))
    # ... and the third term takes all that is left
    np.testing.assert_array_equal(t2, r2)
    np.testing.assert_array_equal(t0.astype(np.float64) + t1.astype(np.float64) + t2.astype(np.float64), a.astype(np.float64))
    mag = np.abs(a.astype(np.float64))
    assert np.all(np.abs(t1) <= 2.0 ** -8 * mag) and np.all(np.abs(t2) <= 2.0 ** -17 * mag)


def test_the_three_products_left_out_stay_below_2_to_minus_24_of_the_product():
    """Six of the nine products of terms are accumulated: (t0,t0) (t0,t1) (t1,t0) (t1,t1) (t0,t2) (t2,t0).
    bf16 x bf16 is exact in float32, so what the kernel loses per product is the rest alone."""
    rng = np.random.default_rng(2)
    a = (rng.standard_normal(200000) * np.exp(rng.uniform(-10, 10, 200000))).astype(np.float32)
    b = (rng.standard_normal(200000) * np.exp(rng.uniform(-10, 10, 200000))).astype(np.float32)
    ta = [t.astype(np.float64) for t in _three_terms(a)[:3]]
    tb = [t.astype(np.float64) for t in _three_terms(b)[:3]]
    kept = sum(ta[i] * tb[j] for i, j in ((0, 0), (0, 1), (1, 0), (1, 1), (0, 2), (2, 0)))
    exact = a.astype(np.float64) * b.astype(np.float64)
    lost = np.abs(kept - exact) / np.abs(exact)
    assert lost.max() <= 2.0 ** -24          # half an ulp of the float32 product: what rounding it once costs
    assert np.sqrt(np.mean(lost ** 2)) <= 2.0 ** -27
    for i in range(3):
        for j in range(3):   # every product of two terms fits float32's 24 bits
            p = ta[i] * tb[j]
            np.testing.assert_array_equal(p.astype(np.float32).astype(np.float64), p)
