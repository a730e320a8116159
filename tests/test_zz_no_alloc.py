"""l3_attn_decode_static -- decode attention whose partials and arrival counters live in the library's
static device array, so that the call allocates nothing -- against l3_attn_decode with a caller's
prepared workspace (l3_attn_workspace_init, L3_ATTN_FLAG_WS_COUNTERS), through the C ABI.  Same plan
and kernels, so the outputs must agree bit for bit; two calls in a row, the second on a smaller
problem, show that what the first call left in the array does no harm."""

import math

import pytest
import torch

from helpers import assert_attn_close, make_qkv, t2f32

FAKE = 0x7F0000001000


def _strides(t, n):
    from custom_kernels import _l3lib

    return _l3lib.i64_array(tuple(t.stride(i) for i in range(n)))


def _both(lib, dev, B, QH, KVH, S, HD, seed, splits=0):
    """Outputs of the workspace entry point and of the static-scratch one on the same inputs."""
    q, k, v = make_qkv(B, QH, KVH, S, HD, seed=seed, cache_len=S + 37, device=dev)
    scale = 1.0 / math.sqrt(HD)
    stream = torch.cuda.current_stream().cuda_stream
    from custom_kernels import _l3lib

    W = _l3lib.L3_ATTN_FLAG_WS_COUNTERS
    ws_bytes = lib.l3_attn_decode_workspace_bytes(B, QH, KVH, S, HD, splits, W)
    ws = torch.empty(max(ws_bytes, _l3lib.L3_ATTN_COUNTER_BYTES), dtype=torch.uint8, device=dev)
    assert lib.l3_attn_workspace_init(ws.data_ptr(), ws.numel(), stream) == 0
    want = torch.full_like(q, float("nan"))
    got = torch.full_like(q, float("nan"))
    plain = torch.full_like(q, float("nan"))
    shape = (B, QH, KVH, S, HD, _strides(q, 2), _strides(k, 3), _strides(v, 3), _strides(want, 2), scale, splits)
    rc = lib.l3_attn_decode(q.data_ptr(), k.data_ptr(), v.data_ptr(), want.data_ptr(), ws.data_ptr(), ws_bytes,
                            *shape, W, stream)
    assert rc == 0, rc
    rc = lib.l3_attn_decode_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), got.data_ptr(), *shape, 0, stream)
    assert rc == 0, rc
    # the entry point without counters (always split kernel + combine kernel) on a workspace of its own
    pb = lib.l3_attn_decode_workspace_bytes(B, QH, KVH, S, HD, splits, 0)
    pws = torch.empty(max(pb, 256), dtype=torch.uint8, device=dev)
    rc = lib.l3_attn_decode(q.data_ptr(), k.data_ptr(), v.data_ptr(), plain.data_ptr(), pws.data_ptr(), pb, *shape, 0, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return want, got, plain, ws_bytes, (q, k, v)


@pytest.mark.gpu
def test_static_scratch_entry_matches_the_workspace_entry(gpu):
    from custom_kernels import _l3lib
    from oracle import attention_decode_ref

    lib = _l3lib.load()
    # first call: 128 splits of a long sequence fill 2.1 MiB of the array; second call, right after
    # it: a smaller problem (24 rows of partials) that lands on what the first one left there
    for (B, QH, KVH, S, HD, splits, seed) in ((1, 32, 8, 8192, 128, 0, 901), (2, 12, 4, 700, 64, 3, 902)):
        print(f"static scratch: B={B} QH={QH} KVH={KVH} S={S} HD={HD} splits={splits}", flush=True)
        want, got, plain, ws_bytes, (q, k, v) = _both(lib, gpu, B, QH, KVH, S, HD, seed, splits)
        assert 0 < ws_bytes <= _l3lib.L3_ATTN_STATIC_SCRATCH_BYTES
        assert not torch.isnan(got.float()).any()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), "static scratch and workspace paths differ"
        # against the two-launch form: another merge order of the same float32 partials, the last bf16 bit at most
        assert (got.float() - plain.float()).abs().max().item() <= 2.0 ** -8 * max(1e-3, plain.float().abs().max().item())
        assert_attn_close(got, attention_decode_ref(t2f32(q.cpu()), t2f32(k.cpu()), t2f32(v.cpu())),
                          what="static scratch vs oracle", min_kv_len=S)
    # and through the Python operator, into the caller's output
    from custom_kernels import custom_kernels_extension as cke

    q, k, v = make_qkv(1, 32, 8, 4096, 64, seed=903, device=gpu)
    out = torch.empty_like(q)
    assert cke.flash_attention_decode_static(q, k, v, out) is out
    assert torch.equal(out, cke.flash_attention_decode(q, k, v))


def test_static_scratch_entry_rejects_what_does_not_fit():
    """The size check runs before any HIP call (no GPU needed): 64 sequences x 32 heads x 512 splits
    of float32 partials is far beyond the static array."""
    from custom_kernels import _l3lib

    lib = _l3lib.load()
    qs, ks = _l3lib.i64_array((4096, 128)), _l3lib.i64_array((1 << 26, 128, 1024))
    need = lib.l3_attn_decode_workspace_bytes(64, 32, 8, 65536, 128, 512, 0)
    assert need > _l3lib.L3_ATTN_STATIC_SCRATCH_BYTES
    rc = lib.l3_attn_decode_static(FAKE, FAKE, FAKE, FAKE, 64, 32, 8, 65536, 128, qs, ks, ks, qs, 0.1, 512, 0, None)
    assert rc == _l3lib.L3_ERR_SCRATCH
    assert "scratch" in _l3lib.strerror(rc)
    assert lib.l3_attn_decode_static(FAKE, FAKE, FAKE, None, 1, 32, 8, 256, 64, qs, ks, ks, qs, 0.1, 0, 0, None) \
        == _l3lib.L3_ERR_NULL_POINTER
