"""GPU parity at buffer sizes whose element offsets do not fit 32 bits: a KV cache of 2.7e9
elements per tensor (decode attention, prefill attention and the rotary-embedding cache append
address its last batch rows), and an RMSNorm input of 2.5e9 elements.  Only the region a case
touches is filled and checked against the oracle; the rest of the allocation is never read."""

import numpy as np
import pytest
import torch

from helpers import assert_attn_close, assert_within_ulps, randn_bf16, t2bits, t2f32
from oracle import attention_decode_ref, attention_prefill_ref, precompute_freqs_cis_ref, rms_norm_ref, rot_embed_ref

pytestmark = pytest.mark.gpu

MAXB, L, KVH, HD = 40, 65536, 8, 128   # 40 * 65536 * 8 * 128 = 2.7e9 elements (5.4 GB) per cache tensor
QH = 32


@pytest.fixture(scope="module")
def big_cache(gpu):
    assert MAXB * L * KVH * HD > 2 ** 31
    ck = torch.empty((MAXB, L, KVH, HD), dtype=torch.bfloat16, device=gpu)
    cv = torch.empty((MAXB, L, KVH, HD), dtype=torch.bfloat16, device=gpu)
    yield ck, cv
    del ck, cv
    torch.cuda.empty_cache()


def test_decode_attention_on_the_last_batch_rows_of_a_large_cache(gpu, big_cache):
    from custom_kernels import custom_kernels_extension as cke

    ck, cv = big_cache
    S = 300
    k = randn_bf16((MAXB, S, KVH, HD), 1)
    v = randn_bf16((MAXB, S, KVH, HD), 2)
    q = randn_bf16((MAXB, 1, QH, HD), 3)
    ck[:, :S] = k.to(gpu)
    cv[:, :S] = v.to(gpu)
    print(f"attention over cache views B={MAXB} S={S} batch stride {ck.stride(0)}", flush=True)
    out = cke.flash_attention_decode(q.to(gpu).transpose(1, 2), ck[:, :S].transpose(1, 2), cv[:, :S].transpose(1, 2))
    torch.cuda.synchronize()
    rows = [0, 31, 32, MAXB - 1]   # offsets below and above 2^31 elements
    assert (MAXB - 1) * ck.stride(0) > 2 ** 31 > 31 * ck.stride(0)
    ref = attention_decode_ref(t2f32(q.transpose(1, 2)[rows]), t2f32(k.transpose(1, 2)[rows]),
                               t2f32(v.transpose(1, 2)[rows]))
    assert_attn_close(out[rows], ref, what="large cache decode", min_kv_len=S)


def test_prefill_attention_on_the_last_batch_row_of_a_large_cache(gpu, big_cache):
    from custom_kernels import custom_kernels_extension as cke

    ck, cv = big_cache
    T = 130
    k = randn_bf16((MAXB, T, KVH, HD), 4)
    v = randn_bf16((MAXB, T, KVH, HD), 5)
    q = randn_bf16((MAXB, T, QH, HD), 6)
    ck[:, :T] = k.to(gpu)
    cv[:, :T] = v.to(gpu)
    print(f"prefill over cache views B={MAXB} T={T}", flush=True)
    out = cke.flash_attention_prefill(q.to(gpu).transpose(1, 2), ck[:, :T].transpose(1, 2), cv[:, :T].transpose(1, 2))
    torch.cuda.synchronize()
    rows = [0, MAXB - 1]
    ref = attention_prefill_ref(t2f32(q.transpose(1, 2)[rows]), t2f32(k.transpose(1, 2)[rows]),
                                t2f32(v.transpose(1, 2)[rows]))
    assert_attn_close(out[rows], ref, what="large cache prefill")


def test_rot_embed_append_into_a_large_cache(gpu, big_cache):
    from custom_kernels import custom_kernels_extension as cke

    ck, cv = big_cache
    p = L - 3
    tab = precompute_freqs_cis_ref(HD, 8, theta=500000.0, use_scaled=True, scale_factor=32.0)
    # the table row the kernel reads is row `pos`; give it a table as long as the cache, of which
    # only the last rows matter
    table = torch.zeros((L, HD), dtype=torch.float32, device=gpu)
    table[p] = torch.from_numpy(tab[5]).to(gpu)
    qkv = randn_bf16((MAXB, 1, (QH + 2 * KVH) * HD), 7)
    pos = torch.full((1,), p, dtype=torch.int32, device=gpu)
    ck[:, p - 1:p + 2].zero_()
    cv[:, p - 1:p + 2].zero_()
    print(f"rot_embed_append B={MAXB} pos={p} offset {(MAXB - 1) * ck.stride(0) + p * ck.stride(1)}", flush=True)
    q_out = cke.rot_embed_append(qkv.to(gpu), table, ck, cv, pos, QH)
    torch.cuda.synchronize()
    q, k, v = qkv.split([QH * HD, KVH * HD, KVH * HD], dim=-1)
    q, k, v = (t.view(MAXB, 1, -1, HD) for t in (q, k, v))
    assert_within_ulps(q_out, rot_embed_ref(t2f32(q), tab[5:6]), 1, what="q")
    assert_within_ulps(ck[:, p:p + 1].contiguous(), rot_embed_ref(t2f32(k), tab[5:6]), 1, what="k row")
    np.testing.assert_array_equal(t2bits(cv[:, p]), t2bits(v[:, 0]))
    assert not ck[:, p - 1].any().item() and not ck[:, p + 1].any().item()
    assert not cv[:, p - 1].any().item() and not cv[:, p + 1].any().item()


def test_rms_norm_with_more_than_2_to_31_elements(gpu):
    from custom_kernels import custom_kernels_extension as cke

    rows, C = 600_000, 4096
    assert rows * C > 2 ** 31
    x = torch.empty((1, rows, C), dtype=torch.bfloat16, device=gpu)
    pick = [0, 1, 524287, 524288, rows - 2, rows - 1]   # 524288 * 4096 = 2^31
    xs = randn_bf16((len(pick), C), 8)
    x.zero_()
    x[0, pick] = xs.to(gpu)
    w = randn_bf16((C,), 9, scale=0.02, mean=1.0)
    print(f"rms_norm rows={rows} C={C}", flush=True)
    y = cke.rms_norm(x, w.to(gpu), 1e-5)
    torch.cuda.synchronize()
    assert_within_ulps(y[0, pick].contiguous(), rms_norm_ref(t2f32(xs), t2f32(w), 1e-5), 1, what="large rms_norm")
    # rows of zeros stay zero (eps keeps the scale finite)
    assert not y[0, 2:1000].any().item() and not y[0, rows - 1000:rows - 2].any().item()
    del x, y
    torch.cuda.empty_cache()
