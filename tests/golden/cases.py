"""Case table shared by make_golden.py and the tests that read the fixtures.

Inputs are not stored: they are re-drawn from the seed with the CPU generator (helpers.py)
and guarded by a CRC of their bits, so a drift in the generator is reported as such rather
than as a kernel failure.
"""

import zlib

import numpy as np

from helpers import make_qkv, randn_bf16, t2bits

ATTN_CASES = {
    # name: (B, QH, KVH, S, HD, cache_len, seed)
    "c1_llama32_1b_s256": (1, 32, 8, 256, 64, None, 42),          # Llama-3.2-1B decode shape, KV length 256
    "hd128_s130_cacheview": (1, 32, 8, 130, 128, 192, 43),        # ragged S, batch stride of a longer cache
    "b2_r4_s200": (2, 8, 2, 200, 64, None, 44),
    "r1_s65": (2, 4, 4, 65, 64, None, 45),
    "r3_hd128_s77": (1, 24, 8, 77, 128, None, 46),                # Llama-3.2-3B ratio
    "r8_hd128_s300": (1, 16, 2, 300, 128, 512, 47),               # Llama-3.3-70B ratio
    "s1": (3, 8, 2, 1, 64, 16, 48),
}

RMS_CASES = {
    # name: (B, T, C, seed)
    "decode_c2048": (3, 1, 2048, 50),
    "rows_c4096": (1, 5, 4096, 51),
    "odd_c136": (2, 3, 136, 52),
    "generic_c100": (1, 4, 100, 53),
}

ROPE_CASES = {
    # name: (B, T, NH, HD, start_pos, factor, seed)
    "q_hd64": (2, 5, 32, 64, 0, 32.0, 60),
    "k_hd128": (1, 4, 8, 128, 1000, 8.0, 61),
    "decode_hd64": (3, 1, 8, 64, 8191, 32.0, 62),
}

FREQ_CASES = {
    # name: (HD, factor, positions)
    "hd64_f32": (64, 32.0, (0, 1, 2, 100, 8191, 16383)),
    "hd128_f8": (128, 8.0, (0, 1, 255, 4096, 16383)),
}


PREFILL_CASES = {
    # name: (B, QH, KVH, T, S, HD, seed)
    "prompt_r4_hd64": (1, 32, 8, 40, 40, 64, 70),
    "chunk_after_cache_hd128": (2, 8, 2, 9, 21, 128, 71),         # 9 new tokens on top of 12 cached ones
    "r1_hd64_t17": (1, 4, 4, 17, 17, 64, 72),
}

LINEAR_CASES = {
    # name: (M, N, K, swiglu, seed)
    "gemv_qkv": (1, 96, 256, False, 80),
    "rows5": (5, 40, 128, False, 81),
    "swiglu_rows3": (3, 64, 192, True, 82),
    "rows40": (40, 24, 384, False, 83),
}


def crc(*arrays) -> int:
    c = 0
    for a in arrays:
        c = zlib.crc32(np.ascontiguousarray(a).tobytes(), c)
    return c


def attn_inputs(name):
    B, QH, KVH, S, HD, L, seed = ATTN_CASES[name]
    return make_qkv(B, QH, KVH, S, HD, seed=seed, cache_len=L)


def rms_inputs(name):
    B, T, C, seed = RMS_CASES[name]
    return randn_bf16((B, T, C), seed), randn_bf16((C,), seed + 1, scale=0.02, mean=1.0)


def rope_inputs(name):
    """x is a strided view into a fused qkv-like buffer (model.py:96-97)."""
    B, T, NH, HD, start, factor, seed = ROPE_CASES[name]
    buf = randn_bf16((B, T, (NH + 16) * HD), seed)
    x = buf[..., : NH * HD].view(B, T, NH, HD)
    return x, start, factor


def bits_crc(*tensors) -> int:
    return crc(*[t2bits(t) for t in tensors])


def prefill_inputs(name):
    B, QH, KVH, T, S, HD, seed = PREFILL_CASES[name]
    q = randn_bf16((B, T, QH, HD), seed).transpose(1, 2)
    k = randn_bf16((B, S, KVH, HD), seed + 100).transpose(1, 2)
    v = randn_bf16((B, S, KVH, HD), seed + 200).transpose(1, 2)
    return q, k, v


def linear_inputs(name):
    M, N, K, swiglu, seed = LINEAR_CASES[name]
    x = randn_bf16((M, K), seed)
    w = randn_bf16((N, K), seed + 100, scale=0.1)
    w2 = randn_bf16((N, K), seed + 200, scale=0.1) if swiglu else None
    return x, w, w2
