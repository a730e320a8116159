"""Pins for the decode-step linear oracles (oracle.linear_ref, oracle.swiglu_linear_ref)."""

import numpy as np
import torch
import torch.nn.functional as F

from helpers import randn_bf16, t2bits, t2f32
from oracle import bf16_ulp_distance, f32_to_bf16_bits, linear_ref, swiglu_linear_ref


def test_linear_matches_brute_force_and_torch():
    x = t2f32(randn_bf16((3, 40), 1)).astype(np.float64)
    w = t2f32(randn_bf16((7, 40), 2)).astype(np.float64)
    ref = linear_ref(x, w)
    brute = np.array([[sum(x[m, k] * w[n, k] for k in range(40)) for n in range(7)] for m in range(3)])
    np.testing.assert_allclose(ref, brute, rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(ref, F.linear(torch.from_numpy(x), torch.from_numpy(w)).numpy(), rtol=1e-13)
    # a transposed weight or a swapped operand would fail these
    one_hot = np.zeros((1, 40))
    one_hot[0, 5] = 1.0
    np.testing.assert_array_equal(linear_ref(one_hot, w)[0], w[:, 5])
    assert linear_ref(x[None], w).shape == (1, 3, 7)


def test_swiglu_matches_torch_bf16_operators():
    x = randn_bf16((5, 64), 3)
    wg = randn_bf16((48, 64), 4, scale=0.3)
    wu = randn_bf16((48, 64), 5, scale=0.3)
    ref = swiglu_linear_ref(t2f32(x), t2f32(wg), t2f32(wu))
    # torch on the CPU: bf16 linear (float accumulation, one rounding), bf16 silu, bf16 product
    lib = F.silu(F.linear(x, wg)) * F.linear(x, wu)
    d = bf16_ulp_distance(t2bits(lib), f32_to_bf16_bits(ref.astype(np.float32)))
    assert d.max() <= 1 and (d > 0).mean() < 0.02
    # closed forms: a zero gate gives zero; a large gate passes the up projection through
    x1 = np.ones((1, 32))
    big = np.full((4, 32), 1.0)
    up = t2f32(randn_bf16((4, 32), 6)).astype(np.float64)
    out = swiglu_linear_ref(x1, big, up)
    g = 32.0
    np.testing.assert_allclose(out[0], t2f32(torch.tensor(g / (1 + np.exp(-g))).to(torch.bfloat16)) *
                               t2f32(torch.from_numpy(up.sum(axis=1)).to(torch.bfloat16)), rtol=1e-6)
    np.testing.assert_array_equal(swiglu_linear_ref(x1, np.zeros((4, 32)), up), np.zeros((1, 4)))
