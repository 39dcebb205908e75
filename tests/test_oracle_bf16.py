"""Pins oracle/bf16.py against torch's bfloat16 (a library routine) and
hand-computed round-to-nearest-even cases."""
import numpy as np
import torch

from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits, round_to_bf16


def _torch_bits(a):
    t = torch.from_numpy(np.asarray(a, dtype=np.float32)).to(torch.bfloat16)
    return t.view(torch.int16).numpy().view(np.uint16)


def test_rne_matches_torch_on_random_and_special_values():
    rng = np.random.default_rng(0)
    a = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 10,
        rng.standard_normal(1000).astype(np.float32) * 1e-30,
        np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, 3.0234375, 1e38, 3.3e38, 3.4e38], dtype=np.float32),
        rng.integers(0, 2**32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32),
    ])
    a = a[~np.isnan(a)]
    assert np.array_equal(f32_to_bf16_bits(a), _torch_bits(a))


def test_hand_computed_ties():
    # 3 * 1.0078125 = 3.0234375 = 0x40418000 sits exactly between 0x4041 and 0x4042:
    # ties go to the even mantissa 0x4042.
    assert f32_to_bf16_bits(np.float32(3.0234375)) == 0x4042
    # 1 + 2^-8 lies between 0x3F80 and 0x3F81 -> even 0x3F80; 1 + 3*2^-8 -> 0x3F82.
    assert f32_to_bf16_bits(np.float32(1.0 + 2.0**-8)) == 0x3F80
    assert f32_to_bf16_bits(np.float32(1.0 + 3 * 2.0**-8)) == 0x3F82
    # just above the tie rounds up
    assert f32_to_bf16_bits(np.float32(1.0 + 2.0**-8 + 2.0**-20)) == 0x3F81


def test_nan_stays_nan_and_round_trip_is_exact():
    bits = f32_to_bf16_bits(np.array([np.nan], dtype=np.float32))
    assert np.isnan(bf16_bits_to_f32(bits))[0]
    all_bits = np.arange(65536, dtype=np.uint16)
    f = bf16_bits_to_f32(all_bits)
    ok = ~np.isnan(f)
    assert np.array_equal(f32_to_bf16_bits(f[ok]), all_bits[ok])
    assert np.array_equal(round_to_bf16(f[ok]), f[ok])
