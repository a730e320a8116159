"""Committed golden vectors (tests/golden/hot_path_golden.npz, written by
tests/golden/make_golden.py): the oracle must keep reproducing them on the CPU, and the
HIP kernels must meet them on the GPU through the C ABI."""

import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import cases  # noqa: E402
from helpers import (assert_attn_close, assert_within_ulps, bf16_bits_to_f32, t2bits, t2f32,  # noqa: E402
                     to_device_like)
from oracle import (attention_decode_ref, attention_prefill_ref, f32_to_bf16_bits, linear_ref,  # noqa: E402
                    precompute_freqs_cis_ref, rms_norm_ref, rot_embed_ref, swiglu_linear_ref)

GOLD = np.load(os.path.join(HERE, "golden", "hot_path_golden.npz"))


# ------------------------------------------------------------------ CPU: oracle vs vectors
@pytest.mark.parametrize("name", list(cases.ATTN_CASES))
def test_oracle_attention_golden(name):
    q, k, v = cases.attn_inputs(name)
    assert cases.bits_crc(q, k, v) == int(GOLD[f"attn/{name}/input_crc"]), "seeded inputs drifted"
    ref = attention_decode_ref(t2f32(q), t2f32(k), t2f32(v))
    np.testing.assert_allclose(ref, GOLD[f"attn/{name}/expected_f32"], rtol=2e-7, atol=1e-8)


@pytest.mark.parametrize("name", list(cases.RMS_CASES))
def test_oracle_rms_golden(name):
    x, w = cases.rms_inputs(name)
    assert cases.bits_crc(x, w) == int(GOLD[f"rms/{name}/input_crc"])
    ref = rms_norm_ref(t2f32(x), t2f32(w), 1e-5)
    np.testing.assert_array_equal(f32_to_bf16_bits(ref.astype(np.float32)), GOLD[f"rms/{name}/expected_bits"])


@pytest.mark.parametrize("name", list(cases.ROPE_CASES))
def test_oracle_rope_golden(name):
    x, start, factor = cases.rope_inputs(name)
    assert cases.bits_crc(x) == int(GOLD[f"rope/{name}/input_crc"])
    ref = rot_embed_ref(t2f32(x), GOLD[f"rope/{name}/freq"])
    np.testing.assert_array_equal(f32_to_bf16_bits(ref.astype(np.float32)), GOLD[f"rope/{name}/expected_bits"])


@pytest.mark.parametrize("name", list(cases.PREFILL_CASES))
def test_oracle_prefill_golden(name):
    q, k, v = cases.prefill_inputs(name)
    assert cases.bits_crc(q, k, v) == int(GOLD[f"prefill/{name}/input_crc"]), "seeded inputs drifted"
    ref = attention_prefill_ref(t2f32(q), t2f32(k), t2f32(v))
    np.testing.assert_allclose(ref, GOLD[f"prefill/{name}/expected_f32"], rtol=2e-7, atol=1e-8)


@pytest.mark.parametrize("name", list(cases.LINEAR_CASES))
def test_oracle_linear_golden(name):
    x, w, w2 = cases.linear_inputs(name)
    assert cases.bits_crc(*([x, w] + ([w2] if w2 is not None else []))) == int(GOLD[f"linear/{name}/input_crc"])
    ref = linear_ref(t2f32(x), t2f32(w)) if w2 is None else swiglu_linear_ref(t2f32(x), t2f32(w), t2f32(w2))
    np.testing.assert_allclose(ref, GOLD[f"linear/{name}/expected_f32"], rtol=2e-7, atol=1e-8)


@pytest.mark.parametrize("name", list(cases.FREQ_CASES))
def test_freq_table_golden(name):
    from custom_kernels import precompute_freqs_cis

    HD, factor, positions = cases.FREQ_CASES[name]
    rows = GOLD[f"freq/{name}/rows"]
    ref = precompute_freqs_cis_ref(HD, max(positions) + 1, theta=500000.0, use_scaled=True, scale_factor=factor)
    np.testing.assert_array_equal(ref[list(positions)], rows)
    # the shipped builder: float32 pow/cos/sin, so positions * 1 ulp of frequency apart at most
    got = precompute_freqs_cis(HD, max(positions) + 1, 500000.0, True, scale_factor=factor).numpy()[list(positions)]
    tol = np.maximum(2e-6, np.array(positions, dtype=np.float64)[:, None] * 1.5e-7)
    assert np.all(np.abs(got - rows) <= tol)


# ---------------------------------------------------------------- GPU: kernels vs vectors
@pytest.mark.gpu
@pytest.mark.parametrize("name", list(cases.ATTN_CASES))
@pytest.mark.parametrize("splits", [0, 1, 3])
def test_gpu_attention_golden(gpu, attn_kernel, name, splits):
    from custom_kernels import custom_kernels_extension as cke

    q, k, v = cases.attn_inputs(name)
    print(f"attention golden {attn_kernel} {name} splits={splits} shapes q{tuple(q.shape)} k{tuple(k.shape)}", flush=True)
    qg, kg, vg = (to_device_like(t, gpu) for t in (q, k, v))
    assert kg.stride() == k.stride()
    out = cke.flash_attention_decode(qg, kg, vg, splits)
    torch.cuda.synchronize()
    assert out.shape == q.shape and out.stride() == q.stride() and out.dtype == torch.bfloat16
    assert_attn_close(out, GOLD[f"attn/{name}/expected_f32"], what=name)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(cases.RMS_CASES))
def test_gpu_rms_golden(gpu, name):
    from custom_kernels import custom_kernels_extension as cke

    x, w = cases.rms_inputs(name)
    print(f"rms golden {name} x{tuple(x.shape)}", flush=True)
    out = cke.rms_norm(x.to(gpu), w.to(gpu), 1e-5)
    torch.cuda.synchronize()
    assert out.shape == x.shape and out.is_contiguous()
    assert_within_ulps(out, bf16_bits_to_f32(GOLD[f"rms/{name}/expected_bits"]), 1, what=name)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(cases.ROPE_CASES))
def test_gpu_rope_golden(gpu, name):
    from custom_kernels import custom_kernels_extension as cke

    x, start, factor = cases.rope_inputs(name)
    print(f"rope golden {name} x{tuple(x.shape)} strides {x.stride()}", flush=True)
    xg = to_device_like(x, gpu)
    assert xg.stride() == x.stride()
    out = cke.rot_embed(xg, torch.from_numpy(GOLD[f"rope/{name}/freq"]).to(gpu))
    torch.cuda.synchronize()
    assert out.is_contiguous() and out.shape == x.shape
    assert_within_ulps(out, bf16_bits_to_f32(GOLD[f"rope/{name}/expected_bits"]), 1, what=name)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(cases.PREFILL_CASES))
def test_gpu_prefill_golden(gpu, name):
    from custom_kernels import custom_kernels_extension as cke

    q, k, v = cases.prefill_inputs(name)
    out = cke.flash_attention_prefill(q.to(gpu), k.to(gpu), v.to(gpu))
    torch.cuda.synchronize()
    assert_attn_close(out, GOLD[f"prefill/{name}/expected_f32"], what=name)


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(cases.LINEAR_CASES))
def test_gpu_linear_golden(gpu, name):
    from custom_kernels import custom_kernels_extension as cke

    x, w, w2 = cases.linear_inputs(name)
    if w2 is None:
        y = cke.linear_decode(x.to(gpu), w.to(gpu))
    else:
        y = cke.linear_swiglu_decode(x.to(gpu), w.to(gpu), w2.to(gpu))
    torch.cuda.synchronize()
    ref = GOLD[f"linear/{name}/expected_f32"].astype(np.float64)
    got = t2f32(y).astype(np.float64)
    # 1 bf16 ulp of the result plus the float32 accumulation slack of a cancelling sum; the SwiGLU
    # form may also flip the rounding of its gate or up factor (one more ulp of that factor)
    tol = (2.0 ** -7 if w2 is not None else 2.0 ** -8) * np.abs(ref) + 2.0 ** -16 * max(1.0, np.abs(ref).max())
    assert np.all(np.abs(got - ref) <= tol), f"{name}: max excess {(np.abs(got - ref) - tol).max():.3e}"
