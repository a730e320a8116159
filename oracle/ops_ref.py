"""float64 numpy restatement of the three operators and the frequency table.

TEST INFRASTRUCTURE ONLY -- see oracle/__init__.py.  Inputs are numpy arrays that
hold bf16-representable values (any float dtype, any strides); all arithmetic is
float64 and nothing is rounded on the way out, so callers round once to bf16
(oracle.round_to_bf16) when they need the expected output tensor.
"""

import math

import numpy as np


# --------------------------------------------------------------------------- attention
def attention_decode_ref(q, k, v, scale=None) -> np.ndarray:
    """Single-token GQA attention.

    q (B, QH, 1, HD); k, v (B, KVH, S, HD); returns (B, QH, 1, HD) float64.
    Query head h attends through kv head h // (QH // KVH)
    (custom_kernels.cu:55,163: query ``head*R + i`` pairs with kv ``head``);
    scale defaults to 1/sqrt(HD) (custom_kernels.cu:253); no mask: the caller bounds
    S by slicing its cache (model.py:107-108).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    B, QH, one, HD = q.shape
    assert one == 1
    Bk, KVH, S, HDk = k.shape
    assert Bk == B and HDk == HD and v.shape == k.shape and QH % KVH == 0 and S >= 1
    R = QH // KVH
    if scale is None:
        scale = 1.0 / math.sqrt(HD)
    qg = q.reshape(B, KVH, R, HD)
    s = np.einsum("bgrd,bgsd->bgrs", qg, k) * scale
    s -= s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    o = np.einsum("bgrs,bgsd->bgrd", p, v)
    return o.reshape(B, QH, 1, HD)


def attention_prefill_ref(q, k, v, scale=None) -> np.ndarray:
    """Causal GQA attention for T query tokens against S >= T cached tokens.

    q (B, QH, T, HD); k, v (B, KVH, S, HD); returns (B, QH, T, HD) float64.  Query i sits at
    absolute position S - T + i and attends to tokens 0 .. S - T + i; for S == T this is the
    is_causal mask of the scaled_dot_product_attention call the reference makes for T > 1
    (model.py:114-116).  Head mapping and scale as in attention_decode_ref.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    B, QH, T, HD = q.shape
    _, KVH, S, _ = k.shape
    assert S >= T and QH % KVH == 0
    R = QH // KVH
    if scale is None:
        scale = 1.0 / math.sqrt(HD)
    qg = q.reshape(B, KVH, R, T, HD)
    s = np.einsum("bgrtd,bgsd->bgrts", qg, k) * scale
    allowed = np.arange(S)[None, :] <= (S - T + np.arange(T))[:, None]
    s = np.where(allowed, s, -np.inf)
    s -= s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("bgrts,bgsd->bgrtd", p, v).reshape(B, QH, T, HD)


def attention_split_partials_ref(q, k, v, bounds, scale=None):
    """Per-split unnormalised partials over token ranges ``bounds`` = [0, ..., S].

    Returns (o, m, l): o (n, B, QH, HD) = sum_j exp(s_j - m) v_j over the split,
    m (n, B, QH) the split's score maximum, l (n, B, QH) = sum_j exp(s_j - m).
    This is what a split-KV kernel hands to its combine step
    (intended behaviour of custom_kernels.cu:119-174).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    B, QH, _, HD = q.shape
    KVH = k.shape[1]
    R = QH // KVH
    if scale is None:
        scale = 1.0 / math.sqrt(HD)
    qg = q.reshape(B, KVH, R, HD)
    os_, ms, ls = [], [], []
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        s = np.einsum("bgrd,bgsd->bgrs", qg, k[:, :, lo:hi]) * scale
        m = s.max(axis=-1)
        p = np.exp(s - m[..., None])
        os_.append(np.einsum("bgrs,bgsd->bgrd", p, v[:, :, lo:hi]).reshape(B, QH, HD))
        ms.append(m.reshape(B, QH))
        ls.append(p.sum(axis=-1).reshape(B, QH))
    return np.stack(os_), np.stack(ms), np.stack(ls)


def lse_combine_ref(o, m, l) -> np.ndarray:
    """Log-sum-exp merge of split partials -> (B, QH, 1, HD).

    out = sum_i o_i e^{m_i - M} / sum_i l_i e^{m_i - M}, M = max_i m_i: what
    custom_kernels.cu:198-222 intends (and, indexing the statistics by blockIdx.z,
    does not do).
    """
    o = np.asarray(o, dtype=np.float64)
    m = np.asarray(m, dtype=np.float64)
    l = np.asarray(l, dtype=np.float64)
    M = m.max(axis=0, keepdims=True)
    w = np.exp(m - M)
    num = (o * w[..., None]).sum(axis=0)
    den = (l * w).sum(axis=0)
    out = num / den[..., None]
    return out[:, :, None, :]


# ----------------------------------------------------------------------------- RMSNorm
def rms_norm_ref(x, w, eps) -> np.ndarray:
    """y = x * (mean(x^2) + eps)^-1/2 * w over the last axis (custom_kernels.cu:343-366)."""
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    ms = np.mean(x * x, axis=-1, keepdims=True)
    return x / np.sqrt(ms + float(eps)) * w


# ------------------------------------------------------------------------------ linear
def linear_ref(x, w) -> np.ndarray:
    """y = x . w^T in float64: x (..., K), w (N, K) -> (..., N).  What nn.Linear without bias
    computes (model.py:95,121,134,225)."""
    return np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T


def swiglu_linear_ref(x, w_gate, w_up) -> np.ndarray:
    """bf16(silu(g)) * u with g = bf16(x . w_gate^T), u = bf16(x . w_up^T): the front half of the
    MLP (model.py:134, F.silu(c_fc2(x)) * c_fc(x)) with the roundings of its three bf16 torch
    operators; the final product is left unrounded for the caller."""
    from .bf16 import round_to_bf16
    g = round_to_bf16(linear_ref(x, w_gate)).astype(np.float64)
    u = round_to_bf16(linear_ref(x, w_up)).astype(np.float64)
    s = round_to_bf16(g / (1.0 + np.exp(-g))).astype(np.float64)
    return s * u


# -------------------------------------------------------------------------------- RoPE
def rot_embed_ref(x, freq) -> np.ndarray:
    """Rotate adjacent pairs: x (B, T, NH, HD), freq (T, HD) = [cos0, sin0, cos1, sin1, ...].

    (y0, y1) = (x0 c - x1 s, x0 s + x1 c) with (c, s) = freq[t, 2i:2i+2]
    (custom_kernels.cu:400-414); the same row of freq serves every batch row and head.
    """
    x = np.asarray(x, dtype=np.float64)
    f = np.asarray(freq, dtype=np.float64)
    B, T, NH, HD = x.shape
    assert f.shape == (T, HD) and HD % 2 == 0
    c = f[:, 0::2][None, :, None, :]
    s = f[:, 1::2][None, :, None, :]
    x0 = x[..., 0::2]
    x1 = x[..., 1::2]
    y = np.empty_like(x)
    y[..., 0::2] = x0 * c - x1 * s
    y[..., 1::2] = x0 * s + x1 * c
    return y


# --------------------------------------------------------------------- frequency table
def llama3_scaled_inv_freq_ref(dim, theta=500000.0, use_scaled=True, scale_factor=8.0,
                               low_freq_factor=1.0, high_freq_factor=4.0,
                               old_context_len=8192) -> np.ndarray:
    """Inverse frequencies theta^(-2i/dim), optionally with Llama-3 wavelength banding.

    model.py:27-49: wavelengths shorter than old_ctx/high are kept, longer than
    old_ctx/low are divided by scale_factor, the band between is blended linearly in
    old_ctx/wavelen.  model.py:29 fixes scale_factor to 8; it is a parameter here.
    Computed in float64 and returned as float64.
    """
    i = np.arange(0, dim, 2, dtype=np.float64)[: dim // 2]
    inv = 1.0 / (float(theta) ** (i / dim))
    if not use_scaled:
        return inv
    low_wavelen = old_context_len / low_freq_factor
    high_wavelen = old_context_len / high_freq_factor
    out = np.empty_like(inv)
    for n, f in enumerate(inv):
        wavelen = 2.0 * math.pi / f
        if wavelen < high_wavelen:
            out[n] = f
        elif wavelen > low_wavelen:
            out[n] = f / scale_factor
        else:
            smooth = (old_context_len / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
            out[n] = (1.0 - smooth) * f / scale_factor + smooth * f
    return out


def precompute_freqs_cis_ref(dim, end, theta=10000.0, use_scaled=False, scale_factor=8.0,
                             low_freq_factor=1.0, high_freq_factor=4.0, old_context_len=8192,
                             inv_freq=None) -> np.ndarray:
    """(end, dim) float32 table of interleaved cos/sin (model.py:51-60).

    The reference forms ``angle = outer(t, inv_freq)`` in float32 and then takes
    cos/sin in float32; here inv_freq is rounded to float32, the product is rounded to
    float32 (so the angle is the one a float32 implementation sees) and cos/sin are
    taken in float64 and rounded once.  Pass ``inv_freq`` (float32) to pin the table
    layout independently of the pow() implementation.
    """
    if inv_freq is None:
        inv_freq = llama3_scaled_inv_freq_ref(dim, theta, use_scaled, scale_factor, low_freq_factor,
                                              high_freq_factor, old_context_len)
    inv32 = np.asarray(inv_freq, dtype=np.float32)
    t = np.arange(end, dtype=np.float32)
    angle = np.outer(t, inv32).astype(np.float32).astype(np.float64)
    table = np.empty((end, dim), dtype=np.float32)
    table[:, 0::2] = np.cos(angle)
    table[:, 1::2] = np.sin(angle)
    return table
