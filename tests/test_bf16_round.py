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
