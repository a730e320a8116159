"""CPU oracle for the custom-kernel hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this directory: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do,
and there only as the checker / the reported CPU baseline, never as the thing
that is measured or shipped.  The product path raises when the HIP library is
missing instead of falling back to anything in here.

What is restated, and from where (paths relative to the reference checkout):

* prefill attention     model.py:114-116 (what the reference asks of torch for T > 1).
* decode attention      custom_kernels/custom_kernels.cu:233-253 (shape, stride
                        and scale conventions), :55 and :163 (GQA head mapping,
                        output layout).  The arithmetic is textbook softmax
                        attention in float64, NOT the reference combine kernel
                        (custom_kernels.cu:184,201,209 read split 0's statistics
                        for every split, which averages the per-split outputs).
* RMSNorm               custom_kernels/custom_kernels.cu:341-366 (formula), with
                        a single final rounding instead of the bf16 multiplies.
* rotary embedding      custom_kernels/custom_kernels.cu:400-414.
* decode-step linear    model.py:95,121,134,225 (nn.Linear without bias; SwiGLU front half).
* frequency table       model.py:27-60.

Pinning status (every function below is pinned; none is "parity unpinned"):
the reference's own tests hold no golden vectors for this path, so each
function is pinned by closed forms, library twins already in the image
(torch SDPA / F.rms_norm / view_as_complex*polar, transformers' llama3 rope
helper) and brute force on tiny inputs -- see tests/test_oracle_*.py.
"""

from .bf16 import (  # noqa: F401
    bf16_bits_to_f32,
    bf16_ulp_distance,
    f32_to_bf16_bits,
    round_to_bf16,
)
from .ops_ref import (  # noqa: F401
    attention_decode_ref,
    attention_prefill_ref,
    attention_split_partials_ref,
    linear_ref,
    swiglu_linear_ref,
    lse_combine_ref,
    precompute_freqs_cis_ref,
    llama3_scaled_inv_freq_ref,
    rms_norm_ref,
    rot_embed_ref,
)
