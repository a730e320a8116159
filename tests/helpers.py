"""Shared test helpers: seeded bf16 inputs and torch <-> numpy bf16 plumbing."""

import numpy as np
import torch

from oracle import bf16_bits_to_f32, bf16_ulp_distance, f32_to_bf16_bits, round_to_bf16  # noqa: F401

ATTN_ATOL = 2e-2     # north-star tolerance for attention in bf16
ATTN_RTOL = 1.6e-2
# Regression bound, far inside the contract, for N(0,1) inputs: what float32 accumulation, one final
# bf16 rounding (half an ulp <= 2^-8 relative) and bf16 probabilities in the second product can cost.
# The last term is 2^-9 * sum_j p_j |v_j|: about 1.6e-3 once a row averages over many tokens (measured
# maximum over the long shapes: 1.2e-3), up to 2^-9 * max|v| when a couple of tokens carry the row.
# A kernel that loses a rescale or a term on some path at small magnitude stays inside the contract
# tolerance; it does not stay inside this.
ATTN_REG_ATOL = 2e-3
ATTN_REG_RTOL = 2.0 ** -7
ATTN_REG_FEW_TOKENS = 2.0 ** -9 * 6.0   # added when a row may attend to fewer than 64 tokens


def t2bits(t: torch.Tensor) -> np.ndarray:
    """bf16 torch tensor (any device/strides) -> uint16 numpy bit patterns."""
    assert t.dtype == torch.bfloat16
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def t2f32(t: torch.Tensor) -> np.ndarray:
    """torch tensor -> float32 numpy values (bf16 goes through its bits: exact)."""
    if t.dtype == torch.bfloat16:
        return bf16_bits_to_f32(t2bits(t))
    return t.detach().cpu().float().numpy()


def randn_bf16(shape, seed, scale=1.0, mean=0.0) -> torch.Tensor:
    """N(mean, scale) drawn on the CPU in float32 from a seed, rounded to bf16."""
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * scale + mean).to(torch.bfloat16)


def make_qkv(B, QH, KVH, S, HD, seed=42, cache_len=None, device=None):
    """q (B,QH,1,HD) and k,v (B,KVH,S,HD) as the model hands them over: token-major storage
    (B, L, KVH, HD) sliced to S tokens and transposed (model.py:107-111,
    benchmark_kernel.py:165-173).  Values are drawn on the CPU; with ``device`` the storage
    is moved first and the views are taken there, so strides are the same on both sides."""
    L = S if cache_len is None else cache_len
    q = randn_bf16((B, 1, QH, HD), seed)
    k = randn_bf16((B, L, KVH, HD), seed + 1)
    v = randn_bf16((B, L, KVH, HD), seed + 2)
    if device is not None:
        q, k, v = q.to(device), k.to(device), v.to(device)
    return q.transpose(1, 2), k[:, :S].transpose(1, 2), v[:, :S].transpose(1, 2)


def to_device_like(t: torch.Tensor, device) -> torch.Tensor:
    """Move a (possibly strided, non-dense) view to ``device`` keeping its exact strides."""
    base = t._base if t._base is not None else t
    moved = base.to(device)
    return moved.as_strided(t.shape, t.stride(), t.storage_offset())


def assert_attn_close(out_bits_or_tensor, ref_f64, what="", min_kv_len=None, regression=True):
    """The contract tolerance, and inside it the regression bound; `min_kv_len` is the smallest
    number of tokens an output row attends to (None = unknown or few)."""
    out = t2f32(out_bits_or_tensor).astype(np.float64) if isinstance(out_bits_or_tensor, torch.Tensor) \
        else bf16_bits_to_f32(out_bits_or_tensor).astype(np.float64)
    ref = np.asarray(ref_f64, dtype=np.float64)
    err = np.abs(out - ref)
    tol = ATTN_ATOL + ATTN_RTOL * np.abs(ref)
    bad = err > tol
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} outside atol {ATTN_ATOL}/rtol {ATTN_RTOL}; max err {err.max():.4g}"
    if regression:
        atol = ATTN_REG_ATOL + (0.0 if (min_kv_len is not None and min_kv_len >= 64) else ATTN_REG_FEW_TOKENS)
        worse = err > atol + ATTN_REG_RTOL * np.abs(ref)
        assert not worse.any(), (f"{what}: inside the contract tolerance but {worse.sum()} of {worse.size} elements are "
                                 f"outside the regression bound atol {atol:.3g}/rtol {ATTN_REG_RTOL:.3g}; "
                                 f"max err {err.max():.4g}")
    return float(err.max())


def assert_within_ulps(out: torch.Tensor, ref_f64, max_ulps=1, what=""):
    got = t2bits(out)
    want = f32_to_bf16_bits(np.asarray(ref_f64, dtype=np.float32))
    d = bf16_ulp_distance(got, want)
    assert d.max() <= max_ulps, f"{what}: max distance {d.max()} bf16 ulp ({(d > max_ulps).sum()} elements over)"
    return int(d.max()), float((d > 0).mean())
