"""Pins oracle.attention_decode_ref / attention_split_partials_ref / lse_combine_ref.

The reference's own tests hold no vectors for this path, so the oracle is pinned against
(1) torch's scaled_dot_product_attention on the CPU -- the routine the reference itself
benchmarks against (benchmark_kernel.py:27-28) and uses for prefill (model.py:116),
(2) a pure-Python brute force on tiny shapes, and (3) properties softmax attention must
have.  Each check is chosen so that a plausible slip (wrong kv head for a query head,
missing scale, transposed operand, averaging instead of LSE-weighting) fails it.
"""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import make_qkv, t2f32
from oracle import attention_decode_ref, attention_split_partials_ref, lse_combine_ref


def _np(q, k, v):
    return t2f32(q), t2f32(k), t2f32(v)


@pytest.mark.parametrize("B,QH,KVH,S,HD", [(1, 32, 8, 256, 64), (2, 8, 2, 65, 128), (3, 4, 4, 7, 64),
                                             (1, 24, 8, 130, 128), (2, 16, 2, 33, 64)])
def test_matches_torch_sdpa_fp32(B, QH, KVH, S, HD):
    q, k, v = make_qkv(B, QH, KVH, S, HD, seed=B * 1000 + S)
    ref = attention_decode_ref(*_np(q, k, v))
    lib = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), enable_gqa=True)
    np.testing.assert_allclose(ref, lib.numpy(), rtol=2e-5, atol=2e-6)


def test_brute_force_tiny():
    B, QH, KVH, S, HD = 2, 4, 2, 5, 64
    q, k, v = _np(*make_qkv(B, QH, KVH, S, HD, seed=7))
    ref = attention_decode_ref(q, k, v)
    R = QH // KVH
    for b in range(B):
        for h in range(QH):
            g = h // R
            scores = [sum(float(q[b, h, 0, d]) * float(k[b, g, j, d]) for d in range(HD)) / math.sqrt(HD)
                      for j in range(S)]
            mx = max(scores)
            w = [math.exp(s - mx) for s in scores]
            z = sum(w)
            for d in range(0, HD, 13):
                want = sum(w[j] * float(v[b, g, j, d]) for j in range(S)) / z
                assert abs(ref[b, h, 0, d] - want) < 1e-12


def test_gqa_equals_mha_on_repeated_kv():
    q, k, v = _np(*make_qkv(2, 8, 2, 40, 64, seed=11))
    a = attention_decode_ref(q, k, v)
    b = attention_decode_ref(q, np.repeat(k, 4, axis=1), np.repeat(v, 4, axis=1))
    np.testing.assert_allclose(a, b, rtol=0, atol=1e-14)
    # a wrong head map (h % KVH instead of h // R) must be visible on the same data
    wrong = attention_decode_ref(q, np.tile(k, (1, 4, 1, 1)), np.tile(v, (1, 4, 1, 1)))
    assert np.abs(a - wrong).max() > 1e-2


def test_equal_value_rows_and_dominant_key():
    q, k, v = _np(*make_qkv(1, 8, 2, 100, 64, seed=3))
    v_const = np.broadcast_to(v[:, :, :1], v.shape)
    out = attention_decode_ref(q, k, v_const)
    np.testing.assert_allclose(out, np.repeat(v_const[:, :, :1], 4, axis=1), atol=1e-12)
    # one key aligned with a query and scaled up gets ~all the weight for that query head
    k2 = k.copy()
    k2[0, 1, 77] = q[0, 5, 0] * 8.0
    out2 = attention_decode_ref(q, k2, v)
    np.testing.assert_allclose(out2[0, 5, 0], v[0, 1, 77], atol=1e-6)


def test_token_permutation_invariance_and_scale():
    q, k, v = _np(*make_qkv(1, 4, 1, 50, 128, seed=5))
    perm = np.random.default_rng(0).permutation(50)
    np.testing.assert_allclose(attention_decode_ref(q, k, v), attention_decode_ref(q, k[:, :, perm], v[:, :, perm]),
                               atol=1e-13)
    # scale enters the scores only: doubling q equals doubling the scale
    np.testing.assert_allclose(attention_decode_ref(2 * q, k, v), attention_decode_ref(q, k, v, scale=2 / math.sqrt(128)),
                               atol=1e-13)
    # default scale is 1/sqrt(HD), not 1/HD or 1
    assert np.abs(attention_decode_ref(q, k, v) - attention_decode_ref(q, k, v, scale=1.0)).max() > 1e-2


@pytest.mark.parametrize("bounds", [[0, 200], [0, 64, 128, 192, 200], [0, 1, 199, 200], [0, 37, 200]])
def test_split_then_combine_reproduces_unsplit(bounds):
    q, k, v = _np(*make_qkv(2, 8, 2, 200, 64, seed=9))
    k[0, 0, 150] = q[0, 1, 0] * 4.0   # a dominant key in a late split: an unweighted mean of splits fails
    full = attention_decode_ref(q, k, v)
    o, m, l = attention_split_partials_ref(q, k, v, bounds)
    np.testing.assert_allclose(lse_combine_ref(o, m, l), full, atol=1e-13)
    if len(bounds) > 2:
        mean_of_splits = (o / l[..., None]).mean(axis=0)[:, :, None, :]
        assert np.abs(mean_of_splits - full).max() > 1e-2


# ------------------------------------------------------------------ causal prefill oracle
from oracle import attention_prefill_ref  # noqa: E402


def _prefill_inputs(B, QH, KVH, T, S, HD, seed):
    from helpers import randn_bf16
    q = randn_bf16((B, T, QH, HD), seed).transpose(1, 2)
    k = randn_bf16((B, S, KVH, HD), seed + 1).transpose(1, 2)
    v = randn_bf16((B, S, KVH, HD), seed + 2).transpose(1, 2)
    return q, k, v


@pytest.mark.parametrize("B,QH,KVH,T,HD", [(1, 8, 2, 17, 64), (2, 4, 4, 5, 128), (1, 12, 4, 33, 64)])
def test_prefill_matches_torch_causal_sdpa(B, QH, KVH, T, HD):
    q, k, v = _prefill_inputs(B, QH, KVH, T, T, HD, seed=T)
    ref = attention_prefill_ref(t2f32(q), t2f32(k), t2f32(v))
    lib = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True, enable_gqa=True)
    np.testing.assert_allclose(ref, lib.numpy(), rtol=2e-5, atol=2e-6)


def test_prefill_rows_are_decode_calls_on_prefixes():
    """Row i of a prefill over S cached tokens is single-token attention over the first S-T+i+1
    tokens; the first row of a prompt from position 0 sees only token 0."""
    B, QH, KVH, T, S, HD = 2, 8, 2, 6, 10, 64
    q, k, v = (t2f32(t) for t in _prefill_inputs(B, QH, KVH, T, S, HD, seed=3))
    ref = attention_prefill_ref(q, k, v)
    for i in range(T):
        n = S - T + i + 1
        row = attention_decode_ref(q[:, :, i:i + 1], k[:, :, :n], v[:, :, :n])
        np.testing.assert_allclose(ref[:, :, i:i + 1], row, atol=1e-13)
    q2, k2, v2 = (t2f32(t) for t in _prefill_inputs(1, 4, 2, 5, 5, 64, seed=4))
    first = attention_prefill_ref(q2, k2, v2)[:, :, 0]
    np.testing.assert_allclose(first, np.repeat(v2[:, :, 0], 2, axis=1), atol=1e-13)
    # an explicit mask with the same alignment gives the same thing through torch
    mask = torch.ones(T, S, dtype=torch.bool).tril(diagonal=S - T)
    lib = F.scaled_dot_product_attention(torch.from_numpy(q).double(), torch.from_numpy(k).double(),
                                         torch.from_numpy(v).double(),
                                         attn_mask=mask, enable_gqa=True)
    np.testing.assert_allclose(ref, lib.numpy(), rtol=1e-9, atol=1e-12)
