"""Pins oracle.rms_norm_ref, rot_embed_ref and the frequency-table restatement against
closed forms and library twins already in the image (F.rms_norm, view_as_complex * polar,
transformers' llama3 rope parameters).  No vectors for these exist in the reference."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import randn_bf16, t2f32
from oracle import (llama3_scaled_inv_freq_ref, precompute_freqs_cis_ref, rms_norm_ref, rot_embed_ref)


# ------------------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("rows,C", [(5, 2048), (3, 4096), (7, 136)])
def test_rms_norm_matches_torch(rows, C):
    x = randn_bf16((rows, C), 1)
    w = randn_bf16((C,), 2, scale=0.02, mean=1.0)
    ref = rms_norm_ref(t2f32(x), t2f32(w), 1e-5)
    lib = F.rms_norm(x.double(), (C,), w.double(), eps=1e-5).numpy()
    np.testing.assert_allclose(ref, lib, rtol=1e-12, atol=0)


def test_rms_norm_closed_forms():
    C, eps = 64, 1e-5
    w = np.linspace(0.5, 1.5, C)
    x = np.full((1, C), 3.0)
    np.testing.assert_allclose(rms_norm_ref(x, w, eps)[0], w * 3.0 / math.sqrt(9.0 + eps), rtol=1e-14)
    onehot = np.zeros((1, C)); onehot[0, 10] = -2.0
    want = np.zeros(C); want[10] = -2.0 / math.sqrt(4.0 / C + eps) * w[10]
    np.testing.assert_allclose(rms_norm_ref(onehot, w, eps)[0], want, rtol=1e-14)
    assert np.all(rms_norm_ref(np.zeros((2, C)), w, eps) == 0.0)               # eps keeps 0/0 away
    r = np.random.default_rng(0).normal(size=(4, C))
    np.testing.assert_allclose(rms_norm_ref(8 * r, w, 0.0), rms_norm_ref(r, w, 0.0), rtol=1e-13)  # scale-free
    np.testing.assert_allclose(rms_norm_ref(r, w, eps)[2], rms_norm_ref(r[2:3], w, eps)[0], rtol=0)  # rows independent
    # the mean is over C (not a sum, not C-1): a unit row has rms 1
    np.testing.assert_allclose(rms_norm_ref(np.ones((1, C)), np.ones(C), 0.0), 1.0, rtol=1e-15)


# --------------------------------------------------------------------------------- RoPE
def _table(T, HD, seed=0):
    ang = np.random.default_rng(seed).uniform(-3, 3, size=(T, HD // 2))
    tab = np.empty((T, HD), dtype=np.float32)
    tab[:, 0::2] = np.cos(ang)
    tab[:, 1::2] = np.sin(ang)
    return tab, ang


@pytest.mark.parametrize("HD", [64, 128])
def test_rot_embed_matches_complex_multiply(HD):
    B, T, NH = 2, 5, 3
    x = randn_bf16((B, T, NH, HD), 4)
    tab, _ = _table(T, HD)
    ref = rot_embed_ref(t2f32(x), tab)
    xc = torch.view_as_complex(x.double().reshape(B, T, NH, HD // 2, 2))
    fc = torch.view_as_complex(torch.from_numpy(tab).double().reshape(T, HD // 2, 2))
    lib = torch.view_as_real(xc * fc[None, :, None, :]).flatten(3).numpy()
    np.testing.assert_allclose(ref, lib, rtol=1e-14, atol=1e-15)


def test_rot_embed_properties():
    B, T, NH, HD = 1, 4, 2, 64
    x = t2f32(randn_bf16((B, T, NH, HD), 8)).astype(np.float64)
    tab, ang = _table(T, HD, seed=1)
    tab64 = np.empty((T, HD)); tab64[:, 0::2] = np.cos(ang); tab64[:, 1::2] = np.sin(ang)
    y = rot_embed_ref(x, tab64)
    # identity at angle 0 (position 0 of a real table: cos 1, sin 0)
    ident = np.zeros((T, HD)); ident[:, 0::2] = 1.0
    np.testing.assert_array_equal(rot_embed_ref(x, ident), x)
    # pair norms are preserved, and rotations compose: R(a) then R(b) = R(a+b)
    np.testing.assert_allclose(y[..., 0::2] ** 2 + y[..., 1::2] ** 2, x[..., 0::2] ** 2 + x[..., 1::2] ** 2, rtol=1e-12)
    tab2 = np.empty((T, HD)); tab2[:, 0::2] = np.cos(2 * ang); tab2[:, 1::2] = np.sin(2 * ang)
    np.testing.assert_allclose(rot_embed_ref(y, tab64), rot_embed_ref(x, tab2), atol=1e-12)
    # sign convention: a quarter turn sends (1, 0) to (0, 1)
    q = np.zeros((1, 1, 1, 2)); q[..., 0] = 1.0
    np.testing.assert_allclose(rot_embed_ref(q, np.array([[0.0, 1.0]])), [[[[0.0, 1.0]]]], atol=1e-15)
    # row t of the table serves token t (not head, not batch)
    y_t2 = rot_embed_ref(x[:, 2:3], tab64[2:3])
    np.testing.assert_array_equal(y[:, 2:3], y_t2)


# --------------------------------------------------------------------- frequency table
def test_inv_freq_bands():
    inv = llama3_scaled_inv_freq_ref(128, theta=500000.0, use_scaled=False)
    np.testing.assert_allclose(inv, 500000.0 ** (-np.arange(0, 128, 2) / 128.0), rtol=1e-15)
    sc = llama3_scaled_inv_freq_ref(128, theta=500000.0, use_scaled=True, scale_factor=32.0)
    wavelen = 2 * math.pi / inv
    hi, lo = 8192 / 4.0, 8192 / 1.0
    np.testing.assert_array_equal(sc[wavelen < hi], inv[wavelen < hi])
    np.testing.assert_allclose(sc[wavelen > lo], inv[wavelen > lo] / 32.0, rtol=1e-15)
    mid = (wavelen >= hi) & (wavelen <= lo)
    assert mid.any() and (wavelen < hi).any() and (wavelen > lo).any()
    assert np.all(sc[mid] < inv[mid]) and np.all(sc[mid] > inv[mid] / 32.0)
    assert np.all(np.diff(sc) < 0)  # still monotone


@pytest.mark.parametrize("HD,factor", [(64, 32.0), (128, 8.0), (64, 8.0), (128, 32.0)])
def test_inv_freq_matches_transformers_llama3(HD, factor):
    from transformers import LlamaConfig
    from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS

    cfg = LlamaConfig(hidden_size=HD * 4, num_attention_heads=4, num_key_value_heads=4, num_hidden_layers=1,
                      intermediate_size=64, vocab_size=32, max_position_embeddings=131072,
                      rope_parameters={"rope_type": "llama3", "rope_theta": 500000.0, "factor": factor,
                                       "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                       "original_max_position_embeddings": 8192})
    inv_tf, att = ROPE_INIT_FUNCTIONS["llama3"](cfg, "cpu")
    assert att == 1.0
    mine = llama3_scaled_inv_freq_ref(HD, theta=500000.0, use_scaled=True, scale_factor=factor)
    np.testing.assert_allclose(mine, inv_tf.double().numpy(), rtol=1e-6)  # float32 chain in the library


def test_table_layout_and_values():
    HD, end = 64, 40
    tab = precompute_freqs_cis_ref(HD, end, theta=500000.0, use_scaled=True, scale_factor=32.0)
    assert tab.shape == (end, HD) and tab.dtype == np.float32
    np.testing.assert_array_equal(tab[0, 0::2], 1.0)
    np.testing.assert_array_equal(tab[0, 1::2], 0.0)
    inv = llama3_scaled_inv_freq_ref(HD, 500000.0, True, 32.0)
    np.testing.assert_allclose(tab[7, 0::2], np.cos(7 * inv), atol=2e-6)
    np.testing.assert_allclose(tab[7, 1::2], np.sin(7 * inv), atol=2e-6)
    np.testing.assert_allclose(tab[:, 0::2] ** 2 + tab[:, 1::2] ** 2, 1.0, atol=3e-7)
    # same layout as view_as_real(polar(1, angle)).flatten(1) (model.py:59-60)
    ang = torch.outer(torch.arange(end, dtype=torch.float32), torch.from_numpy(inv.astype(np.float32)))
    lib = torch.view_as_real(torch.polar(torch.ones_like(ang), ang)).flatten(1).numpy()
    np.testing.assert_allclose(tab, lib, atol=3e-7)


def test_product_table_builder_matches_oracle():
    """The shipped builder (custom_kernels.rope_table) against the oracle restatement."""
    from custom_kernels import precompute_freqs_cis

    for HD, factor in [(64, 32.0), (128, 8.0)]:
        got = precompute_freqs_cis(HD, 300, 500000.0, True, scale_factor=factor).numpy()
        inv32 = llama3_scaled_inv_freq_ref(HD, 500000.0, True, factor).astype(np.float32)
        # frequencies agree to float32 rounding of pow(); given the same frequencies the
        # table agrees to float32 rounding of cos/sin
        np.testing.assert_allclose(np.arctan2(got[1, 1::2], got[1, 0::2]), inv32, rtol=2e-6)
        want = precompute_freqs_cis_ref(HD, 300, theta=500000.0, use_scaled=True, scale_factor=factor)
        np.testing.assert_allclose(got, want, atol=3e-4)  # 300 positions x 1 ulp of frequency
        unscaled = precompute_freqs_cis(HD, 16, 10000.0, False).numpy()
        np.testing.assert_allclose(unscaled, precompute_freqs_cis_ref(HD, 16, 10000.0, False), atol=2e-6)
