"""Pins oracle/bf16.py, the comparator behind every 1-ulp check: the rounding against torch's own
float32 -> bfloat16 conversion, the ulp distance against the rank of a value among all finite bf16
values (brute force)."""

import numpy as np
import torch

from oracle import bf16_bits_to_f32, bf16_ulp_distance, f32_to_bf16_bits, round_to_bf16


def _torch_bits(x: np.ndarray) -> np.ndarray:
    return torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def test_rounding_matches_torch_on_random_tie_and_special_values():
    rng = np.random.default_rng(5)
    rand = rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 200000).astype(np.float32)
    anybits = rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    anybits = anybits[~np.isnan(anybits)]
    # exact ties (low half 0x8000) on even and odd upper halves, and their neighbours: round-to-nearest-even
    hi = rng.integers(0, 0x7F7F, 20000, dtype=np.uint32) << np.uint32(16)
    ties = np.concatenate([hi | np.uint32(0x8000), hi | np.uint32(0x7FFF), hi | np.uint32(0x8001)]).view(np.float32)
    ties = np.concatenate([ties, -ties])
    special = np.array([0.0, -0.0, np.inf, -np.inf, 1e-45, -1e-45, 1e-40, 5.877e-39, 1.1754944e-38,
                        3.3895314e38, 3.4028235e38, -3.4028235e38, 1.0, -1.0, 65504.0], dtype=np.float32)
    for x in (rand, anybits, ties, special):
        np.testing.assert_array_equal(f32_to_bf16_bits(x), _torch_bits(x))
    # NaN stays NaN (payloads may differ between implementations)
    assert np.isnan(bf16_bits_to_f32(f32_to_bf16_bits(np.array([np.nan], dtype=np.float32)))).all()
    # the largest float32 values round up to infinity, as IEEE round-to-nearest does
    assert np.isinf(round_to_bf16(np.array([3.4028235e38], dtype=np.float32))).all()


def test_bits_to_f32_is_the_inverse_on_every_pattern():
    allbits = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    f = bf16_bits_to_f32(allbits)
    want = torch.from_numpy(allbits.view(np.int16).copy()).view(torch.bfloat16).float().numpy()
    np.testing.assert_array_equal(f.view(np.uint32), want.view(np.uint32))
    finite = np.isfinite(f)
    np.testing.assert_array_equal(f32_to_bf16_bits(f[finite]), allbits[finite])


def test_ulp_distance_is_the_rank_difference_over_all_finite_values():
    allbits = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    vals = bf16_bits_to_f32(allbits)
    finite = allbits[np.isfinite(vals) & (allbits != 0x8000)]     # one zero: -0 and +0 are the same value
    order = np.argsort(bf16_bits_to_f32(finite).astype(np.float64), kind="stable")
    rank = np.empty(len(finite), dtype=np.int64)
    rank[order] = np.arange(len(finite))
    lookup = np.full(0x10000, -1, dtype=np.int64)
    lookup[finite] = rank
    lookup[0x8000] = lookup[0x0000]
    rng = np.random.default_rng(6)
    a = rng.choice(finite, 100000)
    b = rng.choice(finite, 100000)
    np.testing.assert_array_equal(bf16_ulp_distance(a, b), np.abs(lookup[a] - lookup[b]))
    # neighbours are one apart, across zero and across a binade boundary too
    assert bf16_ulp_distance(np.uint16(0x0001), np.uint16(0x8001)) == 2
    assert bf16_ulp_distance(np.uint16(0x0000), np.uint16(0x8000)) == 0
    assert bf16_ulp_distance(np.uint16(0x3F7F), np.uint16(0x3F80)) == 1
