"""GPU parity on shapes drawn from a seeded generator: decode attention (plan chosen by the
library, or a forced split count; few and many sequences), causal prefill, RMSNorm, rotary embedding and the decode
linears, each against the float64 oracle.  The draws are deterministic (same cases every run);
every case prints its parameters before it launches anything."""

import numpy as np
import pytest
import torch

from helpers import assert_attn_close, assert_within_ulps, make_qkv, randn_bf16, t2f32
from oracle import (attention_decode_ref, attention_prefill_ref, linear_ref, precompute_freqs_cis_ref, rms_norm_ref,
                    rot_embed_ref)

pytestmark = pytest.mark.gpu

RATIOS = (1, 2, 3, 4, 8)


def _draw_attention_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(n):
        HD = int(rng.choice((64, 128)))
        R = int(rng.choice(RATIOS))
        KVH = int(rng.integers(1, 9))
        B = int(rng.integers(1, 6))
        # lengths cluster around tile and split boundaries as well as being spread out
        S = int(rng.choice((int(rng.integers(1, 70)), int(rng.integers(70, 700)), int(rng.integers(700, 5000)))))
        extra = int(rng.choice((0, 0, 1, 9, 100)))          # cache longer than the attended length
        splits = int(rng.choice((0, 0, 0, 1, 2, 3, 7, 33, 512)))
        cases.append((i, B, R * KVH, KVH, S, HD, S + extra, splits))
    return cases


@pytest.mark.parametrize("case", _draw_attention_cases(48, 2024), ids=lambda c: f"a{c[0]}")
def test_decode_attention_random_shapes(gpu, case):
    from custom_kernels import custom_kernels_extension as cke

    i, B, QH, KVH, S, HD, L, splits = case
    print(f"decode case {i}: B={B} QH={QH} KVH={KVH} S={S} HD={HD} L={L} splits={splits}", flush=True)
    q, k, v = make_qkv(B, QH, KVH, S, HD, seed=1000 + i, cache_len=L)
    qg, kg, vg = make_qkv(B, QH, KVH, S, HD, seed=1000 + i, cache_len=L, device=gpu)
    out = cke.flash_attention_decode(qg, kg, vg, splits)
    torch.cuda.synchronize()
    assert_attn_close(out, attention_decode_ref(t2f32(q), t2f32(k), t2f32(v)), what=f"decode case {i}", min_kv_len=S)


def _draw_large_batch_cases(n, seed):
    """Dozens to hundreds of sequences with every kv-head count the kernel groups differently (1, 2, 3, 4, 8,
    16 heads per batch row): the split plan's branches for many (batch, head group) pairs, the combine
    with a wavefront per pair, and the cooperative form with many workgroups."""
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(n):
        HD = int(rng.choice((64, 128)))
        R = int(rng.choice(RATIOS))
        KVH = int(rng.choice((1, 2, 3, 4, 8, 16)))
        B = int(rng.integers(30, 270))
        S = int(rng.choice((int(rng.integers(1, 130)), int(rng.integers(130, 1100)))))
        S = max(1, min(S, int(2e8 // (B * R * KVH * HD))))     # keeps the float64 oracle in seconds
        extra = int(rng.choice((0, 5, 64)))
        splits = int(rng.choice((0, 0, 0, 2, 3)))
        cases.append((100 + i, B, R * KVH, KVH, S, HD, S + extra, splits))
    return cases


@pytest.mark.parametrize("case", _draw_large_batch_cases(16, 2025), ids=lambda c: f"b{c[0]}")
def test_decode_attention_large_batches(gpu, case):
    test_decode_attention_random_shapes(gpu, case)


def _draw_prefill_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(n):
        HD = int(rng.choice((64, 128)))
        R = int(rng.choice(RATIOS))
        KVH = int(rng.integers(1, 5))
        B = int(rng.integers(1, 4))
        T = int(rng.choice((int(rng.integers(2, 40)), int(rng.integers(40, 300)), int(rng.integers(300, 700)))))
        past = int(rng.choice((0, 0, 1, 50, 130)))          # tokens already in the cache
        form = str(rng.choice(("auto", "wave", "tiled")))
        cases.append((i, B, R * KVH, KVH, T, T + past, HD, form))
    return cases


@pytest.mark.parametrize("case", _draw_prefill_cases(24, 77), ids=lambda c: f"p{c[0]}")
def test_prefill_attention_random_shapes(gpu, case):
    from custom_kernels import custom_kernels_extension as cke

    i, B, QH, KVH, T, S, HD, form = case
    print(f"prefill case {i}: B={B} QH={QH} KVH={KVH} T={T} S={S} HD={HD} form={form}", flush=True)
    q = randn_bf16((B, T, QH, HD), 2000 + i)
    k = randn_bf16((B, S, KVH, HD), 3000 + i)
    v = randn_bf16((B, S, KVH, HD), 4000 + i)
    with cke.attention_flags(prefill=form):
        out = cke.flash_attention_prefill(*(t.to(gpu).transpose(1, 2) for t in (q, k, v)))
        torch.cuda.synchronize()
    ref = attention_prefill_ref(*(t2f32(t.transpose(1, 2)) for t in (q, k, v)))
    assert_attn_close(out, ref, what=f"prefill case {i}")


def _draw_prefill_cases_all_forms(n, seed):
    """Like the cases above, with the no-maximum loop among the forms, longer prompts now and then, and for a
    third of the cases queries scaled so that a few keys carry a row (scores over tens of powers of two)."""
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(n):
        HD = int(rng.choice((64, 128)))
        R = int(rng.choice(RATIOS))
        KVH = int(rng.integers(1, 5))
        B = int(rng.integers(1, 4))
        T = int(rng.choice((int(rng.integers(2, 70)), int(rng.integers(70, 400)), int(rng.integers(400, 1500)))))
        past = int(rng.choice((0, 0, 3, 64, 200)))
        form = str(rng.choice(("auto", "tiled", "tiled-no-max", "tiled-no-max")))
        gain = float(rng.choice((1.0, 1.0, 3.0)))
        cases.append((i, B, R * KVH, KVH, T, T + past, HD, form, gain))
    return cases


@pytest.mark.parametrize("case", _draw_prefill_cases_all_forms(40, 78), ids=lambda c: f"q{c[0]}")
def test_prefill_attention_random_shapes_all_forms(gpu, case):
    from custom_kernels import custom_kernels_extension as cke

    i, B, QH, KVH, T, S, HD, form, gain = case
    print(f"prefill case q{i}: B={B} QH={QH} KVH={KVH} T={T} S={S} HD={HD} form={form} gain={gain}", flush=True)
    q = (randn_bf16((B, T, QH, HD), 5000 + i).float() * gain).to(torch.bfloat16)
    k = randn_bf16((B, S, KVH, HD), 6000 + i)
    v = randn_bf16((B, S, KVH, HD), 7000 + i)
    with cke.attention_flags(prefill=form):
        out = cke.flash_attention_prefill(*(t.to(gpu).transpose(1, 2) for t in (q, k, v)))
        torch.cuda.synchronize()
    ref = attention_prefill_ref(*(t2f32(t.transpose(1, 2)) for t in (q, k, v)))
    assert_attn_close(out, ref, what=f"prefill case q{i}", regression=gain == 1.0)


def test_rms_norm_random_shapes(gpu):
    from custom_kernels import custom_kernels_extension as cke

    rng = np.random.default_rng(5)
    for i in range(24):
        C = int(rng.choice((int(rng.integers(1, 64)), 8 * int(rng.integers(1, 1100)), int(rng.integers(64, 9000)))))
        rows = int(rng.choice((1, 2, 3, int(rng.integers(4, 70)), int(rng.integers(1000, 1400)))))
        eps = float(rng.choice((1e-5, 1e-6, 1e-3)))
        scale = float(rng.choice((1.0, 1e-3, 30.0)))
        print(f"rms_norm case {i}: rows={rows} C={C} eps={eps} scale={scale}", flush=True)
        x = randn_bf16((1, rows, C), 5000 + i, scale=scale)
        w = randn_bf16((C,), 6000 + i, scale=0.02, mean=1.0)
        y = cke.rms_norm(x.to(gpu), w.to(gpu), eps)
        torch.cuda.synchronize()
        assert_within_ulps(y, rms_norm_ref(t2f32(x), t2f32(w), eps), 1, what=f"rms_norm case {i}")


def test_rot_embed_random_shapes(gpu):
    from custom_kernels import custom_kernels_extension as cke

    rng = np.random.default_rng(6)
    for i in range(16):
        HD = int(rng.choice((64, 128, 32, 16)))
        NH = int(rng.integers(1, 33))
        T = int(rng.choice((1, int(rng.integers(2, 20)), int(rng.integers(20, 300)))))
        B = int(rng.integers(1, 4))
        start = int(rng.integers(0, 8000))
        pad = int(rng.choice((0, 8, 3 * HD)))                # x is a view into wider rows
        print(f"rot_embed case {i}: B={B} T={T} NH={NH} HD={HD} start={start} pad={pad}", flush=True)
        tab = precompute_freqs_cis_ref(HD, start + T, theta=500000.0, use_scaled=True, scale_factor=32.0)[start:]
        wide = randn_bf16((B, T, NH * HD + pad), 7000 + i)
        x = wide[..., :NH * HD].view(B, T, NH, HD)
        xg = wide.to(gpu)[..., :NH * HD].view(B, T, NH, HD)
        y = cke.rot_embed(xg, torch.from_numpy(np.ascontiguousarray(tab)).to(gpu))
        torch.cuda.synchronize()
        assert y.is_contiguous()
        assert_within_ulps(y, rot_embed_ref(t2f32(x), tab), 1, what=f"rot_embed case {i}")


def test_decode_linear_random_shapes(gpu):
    from custom_kernels import custom_kernels_extension as cke

    rng = np.random.default_rng(7)
    for i in range(20):
        M = int(rng.choice((1, 2, 3, 4, 5, 8, 15, 16, 17, 31, 48, 64)))
        N = 4 * int(rng.integers(1, 1200))
        K = 32 * int(rng.integers(1, 200))
        if M > 16:                                           # split-K + finish: N % 8 == 0, K % 128 == 0
            N, K = 8 * ((N + 7) // 8), 128 * ((K + 127) // 128)
        print(f"linear case {i}: M={M} N={N} K={K}", flush=True)
        x = randn_bf16((M, 1, K), 8000 + i)
        w = randn_bf16((N, K), 9000 + i, scale=0.05)
        y = cke.linear_decode(x.to(gpu), w.to(gpu))
        torch.cuda.synchronize()
        ref = linear_ref(t2f32(x), t2f32(w))
        got = t2f32(y).astype(np.float64)
        # one bf16 rounding of a float32-accumulated sum: half an ulp of the result plus the
        # accumulation error, bounded through the magnitudes that were summed
        bound = 2.0 ** -8 * np.abs(ref) + 2.0 ** -18 * (np.abs(t2f32(x).astype(np.float64)) @ np.abs(t2f32(w).astype(np.float64)).T)
        assert (np.abs(got - ref) <= bound + 1e-30).all(), f"linear case {i}: max err {np.abs(got - ref).max()}"
