"""Writes tests/golden/*.npz: expected outputs of the float64 oracle on seeded inputs.

Run from the repo root:  python tests/golden/make_golden.py
The reference's own tests hold no vectors for this path (it has no assertions at all), and
every oracle function is pinned by closed forms and library twins (tests/test_oracle_*.py),
so these fixtures are produced by the oracle, not by running the reference.  They freeze
today's expected bits so that a later change to oracle, generator or kernels shows up.
"""

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "llama3-custom-inference_amd"), os.path.dirname(HERE), HERE):
    if p not in sys.path:
        sys.path.insert(0, p)

import cases  # noqa: E402
from helpers import t2f32  # noqa: E402
from oracle import (attention_decode_ref, attention_prefill_ref, f32_to_bf16_bits, linear_ref,  # noqa: E402
                    precompute_freqs_cis_ref, rms_norm_ref, rot_embed_ref, swiglu_linear_ref)


def main():
    out = {}
    for name in cases.ATTN_CASES:
        q, k, v = cases.attn_inputs(name)
        ref = attention_decode_ref(t2f32(q), t2f32(k), t2f32(v))
        out[f"attn/{name}/expected_f32"] = ref.astype(np.float32)
        out[f"attn/{name}/input_crc"] = np.uint32(cases.bits_crc(q, k, v))
    for name in cases.RMS_CASES:
        x, w = cases.rms_inputs(name)
        ref = rms_norm_ref(t2f32(x), t2f32(w), 1e-5)
        out[f"rms/{name}/expected_bits"] = f32_to_bf16_bits(ref.astype(np.float32))
        out[f"rms/{name}/input_crc"] = np.uint32(cases.bits_crc(x, w))
    for name, (B, T, NH, HD, start, factor, seed) in cases.ROPE_CASES.items():
        x, _, _ = cases.rope_inputs(name)
        tab = precompute_freqs_cis_ref(HD, start + T, theta=500000.0, use_scaled=True, scale_factor=factor)[start:]
        ref = rot_embed_ref(t2f32(x), tab)
        out[f"rope/{name}/freq"] = tab
        out[f"rope/{name}/expected_bits"] = f32_to_bf16_bits(ref.astype(np.float32))
        out[f"rope/{name}/input_crc"] = np.uint32(cases.bits_crc(x))
    for name, (HD, factor, positions) in cases.FREQ_CASES.items():
        tab = precompute_freqs_cis_ref(HD, max(positions) + 1, theta=500000.0, use_scaled=True, scale_factor=factor)
        out[f"freq/{name}/rows"] = tab[list(positions)]
    for name in cases.PREFILL_CASES:
        q, k, v = cases.prefill_inputs(name)
        out[f"prefill/{name}/expected_f32"] = attention_prefill_ref(t2f32(q), t2f32(k), t2f32(v)).astype(np.float32)
        out[f"prefill/{name}/input_crc"] = np.uint32(cases.bits_crc(q, k, v))
    for name in cases.LINEAR_CASES:
        x, w, w2 = cases.linear_inputs(name)
        ref = linear_ref(t2f32(x), t2f32(w)) if w2 is None else swiglu_linear_ref(t2f32(x), t2f32(w), t2f32(w2))
        out[f"linear/{name}/expected_f32"] = ref.astype(np.float32)
        out[f"linear/{name}/input_crc"] = np.uint32(cases.bits_crc(*([x, w] + ([w2] if w2 is not None else []))))
    path = os.path.join(HERE, "hot_path_golden.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
