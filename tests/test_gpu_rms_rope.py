"""GPU parity: fused RMSNorm and rotary embedding (through the C ABI) against the float64
oracle, to within 1 bf16 ulp."""

import numpy as np
import pytest
import torch

from helpers import assert_within_ulps, bf16_ulp_distance, randn_bf16, round_to_bf16, t2bits, t2f32, to_device_like
from oracle import precompute_freqs_cis_ref, rms_norm_ref, rot_embed_ref

pytestmark = pytest.mark.gpu


def bf16_ulp(a, b):
    return bf16_ulp_distance(t2bits(a), t2bits(b))


# ------------------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("C", [2048, 4096])
@pytest.mark.parametrize("shape", [(1, 1), (1, 64), (64, 1), (1, 256), (2, 2048), (1, 1500)])
def test_rms_norm_config_shapes(gpu, C, shape):
    from custom_kernels import custom_kernels_extension as cke

    B, T = shape
    print(f"rms_norm B={B} T={T} C={C}", flush=True)
    x = randn_bf16((B, T, C), 100 + T)
    w = randn_bf16((C,), 7, scale=0.02, mean=1.0)
    out = cke.rms_norm(x.to(gpu), w.to(gpu), 1e-5)
    torch.cuda.synchronize()
    assert out.shape == x.shape and out.dtype == torch.bfloat16 and out.is_contiguous()
    assert_within_ulps(out, rms_norm_ref(t2f32(x), t2f32(w), 1e-5), 1, what=f"rms {B}x{T}x{C}")


@pytest.mark.parametrize("C", [8, 64, 100, 136, 2056, 5120, 8192, 8200, 16384])
@pytest.mark.parametrize("rows", [3, 1100, 2500])
def test_rms_norm_other_widths(gpu, C, rows):
    """Widths off the fast paths: not a multiple of 8 (2-byte path), wider than the
    register-resident limit, and tiny."""
    from custom_kernels import custom_kernels_extension as cke

    print(f"rms_norm rows={rows} C={C}", flush=True)
    x = randn_bf16((1, rows, C), C)
    w = randn_bf16((C,), 8, scale=0.5, mean=0.0)
    out = cke.rms_norm(x.to(gpu), w.to(gpu), 1e-5)
    torch.cuda.synchronize()
    assert_within_ulps(out, rms_norm_ref(t2f32(x), t2f32(w), 1e-5), 1, what=f"rms rows{rows} C{C}")


def test_rms_norm_adversarial_rows(gpu):
    from custom_kernels import custom_kernels_extension as cke

    C = 4096
    rows = []
    g = torch.Generator().manual_seed(0)
    rows.append(torch.randn(C, generator=g) * torch.logspace(-6, 6, C))          # 12 decades of range
    rows.append(torch.full((C,), 3.0))                                           # constant
    rows.append(torch.zeros(C))                                                  # eps only
    onehot = torch.zeros(C); onehot[123] = -7.0; rows.append(onehot)
    rows.append(torch.randn(C, generator=g) * 1e-4)                              # eps comparable to mean(x^2)
    rows.append(torch.randn(C, generator=g) * 1e4)
    alt = torch.ones(C); alt[::2] = -1.0; rows.append(alt * 255.0)
    x = torch.stack(rows).to(torch.bfloat16).unsqueeze(0)
    w = randn_bf16((C,), 9, scale=1.0)
    out = cke.rms_norm(x.to(gpu), w.to(gpu), 1e-5)
    torch.cuda.synchronize()
    assert_within_ulps(out, rms_norm_ref(t2f32(x), t2f32(w), 1e-5), 1, what="adversarial rows")
    assert torch.all(out[0, 2] == 0)
    # non-contiguous input is accepted (made contiguous), weight of ones is the identity scaling
    xt = randn_bf16((4, 2, 2048), 3).to(gpu).transpose(0, 1)
    o2 = cke.rms_norm(xt, torch.ones(2048, dtype=torch.bfloat16, device=gpu), 1e-5)
    assert_within_ulps(o2, rms_norm_ref(t2f32(xt), np.ones(2048), 1e-5), 1, what="transposed input")
    with pytest.raises(RuntimeError):
        cke.rms_norm(xt, torch.ones(100, dtype=torch.bfloat16, device=gpu), 1e-5)


# --------------------------------------------------------------------------------- RoPE
def _qkv_views(B, T, HD, seed, device=None):
    """q (32 heads) and k (8 heads) as views into a fused projection output (model.py:95-97)."""
    buf = randn_bf16((B, T, (32 + 16) * HD), seed)
    if device is not None:
        buf = buf.to(device)
    q, k, _ = buf.split([32 * HD, 8 * HD, 8 * HD], dim=-1)
    return q.view(B, T, 32, HD), k.view(B, T, 8, HD)


@pytest.mark.parametrize("HD", [64, 128])
@pytest.mark.parametrize("shape", [(1, 1), (64, 1), (1, 64), (1, 256), (2, 2048)])
def test_rot_embed_config_shapes(gpu, HD, shape):
    from custom_kernels import custom_kernels_extension as cke

    B, T = shape
    start = 0 if T > 1 else 4321
    print(f"rot_embed B={B} T={T} HD={HD} start={start}", flush=True)
    tab = precompute_freqs_cis_ref(HD, start + T, theta=500000.0, use_scaled=True, scale_factor=32.0)[start:]
    tab_g = torch.from_numpy(tab).to(gpu)
    for x, xg in zip(_qkv_views(B, T, HD, 5), _qkv_views(B, T, HD, 5, device=gpu)):
        assert not xg.is_contiguous() or B * T == 1
        out = cke.rot_embed(xg, tab_g)
        torch.cuda.synchronize()
        assert out.shape == x.shape and out.is_contiguous() and out.dtype == torch.bfloat16
        assert_within_ulps(out, rot_embed_ref(t2f32(x), tab), 1, what=f"rope {tuple(x.shape)}")
        # the same values from a contiguous tensor give the same bits
        out_c = cke.rot_embed(xg.contiguous(), tab_g)
        np.testing.assert_array_equal(t2bits(out), t2bits(out_c))


@pytest.mark.parametrize("B,T,NH,HD", [(3, 1501, 32, 128),    # 2 tokens per workgroup, odd T: a half-filled last block
                                        (2, 3100, 20, 128),    # 80 threads per token: 3 tokens per workgroup, idle lanes
                                        (5, 7000, 8, 64),      # 16 tokens per workgroup
                                        (2, 5200, 6, 128),     # head pairs, 48 threads per token
                                        (1, 9001, 7, 64)])     # single heads, 56 threads per token
def test_rot_embed_many_tokens(gpu, B, T, NH, HD):
    """Thousands of tokens per batch row with head counts that give 2, 3, 4, 5 and 16 tokens per
    workgroup, idle lanes, and token counts that do not fill the last workgroup."""
    from custom_kernels import custom_kernels_extension as cke

    print(f"rot_embed B={B} T={T} NH={NH} HD={HD}", flush=True)
    tab = precompute_freqs_cis_ref(HD, T, theta=500000.0, use_scaled=True, scale_factor=32.0)
    wide = randn_bf16((B, T, NH * HD + 2 * HD), 77)      # a view into wider rows, as q is into qkv
    x = wide[..., :NH * HD].view(B, T, NH, HD)
    xg = wide.to(gpu)[..., :NH * HD].view(B, T, NH, HD)
    out = cke.rot_embed(xg, torch.from_numpy(np.ascontiguousarray(tab)).to(gpu))
    torch.cuda.synchronize()
    assert out.is_contiguous()
    assert_within_ulps(out, rot_embed_ref(t2f32(x), tab), 1, what=f"rope {tuple(x.shape)}")


def test_rot_embed_identity_at_position_zero_and_norms(gpu):
    from custom_kernels import custom_kernels_extension as cke

    HD = 64
    x = randn_bf16((2, 3, 8, HD), 11)
    tab = precompute_freqs_cis_ref(HD, 3, theta=500000.0, use_scaled=True, scale_factor=32.0)
    out = cke.rot_embed(x.to(gpu), torch.from_numpy(tab).to(gpu))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(t2bits(out[:, 0]), t2bits(x[:, 0]))   # cos 1, sin 0: bit-exact identity
    o = t2f32(out).astype(np.float64)
    xi = t2f32(x).astype(np.float64)
    n_out = o[..., 0::2] ** 2 + o[..., 1::2] ** 2
    n_in = xi[..., 0::2] ** 2 + xi[..., 1::2] ** 2
    np.testing.assert_allclose(n_out, n_in, rtol=2.0 ** -6, atol=1e-6)   # rotation keeps pair norms (bf16 rounding)


def test_rot_embed_cancellation_stays_within_one_ulp(gpu):
    """Pairs built so that x0*cos - x1*sin nearly cancels: the float32 evaluation must keep the
    error relative to the (small) result."""
    from custom_kernels import custom_kernels_extension as cke

    HD, T = 64, 2048
    tab = precompute_freqs_cis_ref(HD, T, theta=500000.0, use_scaled=True, scale_factor=32.0)
    c, s = tab[:, 0::2].astype(np.float64), tab[:, 1::2].astype(np.float64)
    x = np.zeros((1, T, 1, HD))
    x[0, :, 0, 0::2] = s          # x0 = sin, x1 = cos  ->  y0 = sin*cos - cos*sin ~ 0 after bf16 rounding of x
    x[0, :, 0, 1::2] = c
    xb = torch.from_numpy(x).to(torch.bfloat16)
    out = cke.rot_embed(xb.to(gpu), torch.from_numpy(tab).to(gpu))
    torch.cuda.synchronize()
    assert_within_ulps(out, rot_embed_ref(t2f32(xb), tab), 1, what="cancelling pairs")


@pytest.mark.parametrize("B,T,NH,HD", [(2, 37, 80, 128), (1, 300, 132, 64), (3, 5, 96, 128)])
def test_rot_embed_many_heads(gpu, B, T, NH, HD):
    """More heads than a workgroup's threads can share per token (16-byte chunks x head groups > 256):
    the flat one-item-per-lane kernel."""
    from custom_kernels import custom_kernels_extension as cke

    print(f"rot_embed B={B} T={T} NH={NH} HD={HD}", flush=True)
    tab = precompute_freqs_cis_ref(HD, 100 + T, theta=500000.0, use_scaled=True, scale_factor=32.0)[100:]
    wide = randn_bf16((B, T, NH * HD + 64), 91)
    x = wide[..., :NH * HD].view(B, T, NH, HD)
    xg = wide.to(gpu)[..., :NH * HD].view(B, T, NH, HD)
    out = cke.rot_embed(xg, torch.from_numpy(np.ascontiguousarray(tab)).to(gpu))
    torch.cuda.synchronize()
    assert out.is_contiguous()
    assert_within_ulps(out, rot_embed_ref(t2f32(x), tab), 1, what=f"rope {tuple(x.shape)}")


def test_rot_embed_pair_path_and_errors(gpu):
    from custom_kernels import custom_kernels_extension as cke

    # head size 6 and a token stride that is not a multiple of 8: the 4-byte path
    buf = randn_bf16((2, 5, 3 * 6 + 2), 13)
    x = buf[..., : 3 * 6].view(2, 5, 3, 6)
    ang = np.random.default_rng(1).uniform(-3, 3, size=(5, 3))
    tab = np.empty((5, 6), dtype=np.float32); tab[:, 0::2] = np.cos(ang); tab[:, 1::2] = np.sin(ang)
    out = cke.rot_embed(to_device_like(x, gpu), torch.from_numpy(tab).to(gpu))
    torch.cuda.synchronize()
    assert_within_ulps(out, rot_embed_ref(t2f32(x), tab), 1, what="pair path")
    with pytest.raises(RuntimeError):
        cke.rot_embed(to_device_like(x, gpu), torch.from_numpy(tab[:4]).to(gpu))
    with pytest.raises(RuntimeError):
        cke.rot_embed(to_device_like(x, gpu).float(), torch.from_numpy(tab).to(gpu))


@pytest.mark.parametrize("HD,NH,KVH", [(64, 32, 8), (128, 32, 8), (64, 4, 4)])
def test_rot_embed_append_fuses_rope_and_cache_write(gpu, HD, NH, KVH):
    """Against the unfused sequence of model.py:100-106: rot_embed(q), rot_embed(k), two cache
    slice assignments -- q, the cache row at `pos`, and every other cache row (untouched)."""
    from custom_kernels import custom_kernels_extension as cke

    B, maxB, L = 3, 4, 40
    tab = precompute_freqs_cis_ref(HD, 64, theta=500000.0, use_scaled=True, scale_factor=32.0)
    tab_g = torch.from_numpy(tab).to(gpu)
    qkv = randn_bf16((B, 1, (NH + 2 * KVH) * HD), 17)
    ck0 = randn_bf16((maxB, L, KVH, HD), 18)
    cv0 = randn_bf16((maxB, L, KVH, HD), 19)
    pos = torch.zeros(1, dtype=torch.int32, device=gpu)
    for p in (0, 7, L - 1):
        ck, cv = ck0.to(gpu), cv0.to(gpu)
        pos.fill_(p)
        q_out = cke.rot_embed_append(qkv.to(gpu), tab_g, ck, cv, pos, NH)
        torch.cuda.synchronize()
        q, k, v = qkv.split([NH * HD, KVH * HD, KVH * HD], dim=-1)
        q, k, v = (t.view(B, 1, -1, HD) for t in (q, k, v))
        assert q_out.shape == (B, 1, NH, HD) and q_out.is_contiguous()
        assert_within_ulps(q_out, rot_embed_ref(t2f32(q), tab[p:p + 1]), 1, what="q")
        assert_within_ulps(ck[:B, p:p + 1].contiguous(), rot_embed_ref(t2f32(k), tab[p:p + 1]), 1, what="k row")
        np.testing.assert_array_equal(t2bits(cv[:B, p]), t2bits(v[:, 0]))
        # bit-identical to the unfused operator
        np.testing.assert_array_equal(t2bits(q_out), t2bits(cke.rot_embed(q.to(gpu), tab_g[p:p + 1])))
        keep = [i for i in range(L) if i != p]
        np.testing.assert_array_equal(t2bits(ck[:, keep]), t2bits(ck0[:, keep]))
        np.testing.assert_array_equal(t2bits(cv[:, keep]), t2bits(cv0[:, keep]))
        np.testing.assert_array_equal(t2bits(ck[B:]), t2bits(ck0[B:]))
    # a position outside the cache writes nothing
    ck, cv = ck0.to(gpu), cv0.to(gpu)
    pos.fill_(L)
    cke.rot_embed_append(qkv.to(gpu), tab_g, ck, cv, pos, NH)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(t2bits(ck), t2bits(ck0))


@pytest.mark.parametrize("shape", [(1, 1, 2048), (64, 1, 2048), (2, 700, 4096), (1, 3, 136), (1, 5, 100), (1, 2, 8200),
                                   (4, 1024, 2048), (3, 1001, 1000), (2, 2048, 4096)])
def test_add_rms_norm_equals_add_then_norm(gpu, shape):
    from custom_kernels import custom_kernels_extension as cke

    B, T, C = shape
    print(f"add_rms_norm {shape}", flush=True)
    x = randn_bf16(shape, 71)
    r = randn_bf16(shape, 72, scale=0.5)
    w = randn_bf16((C,), 73, scale=0.02, mean=1.0)
    s, y = cke.add_rms_norm(x.to(gpu), r.to(gpu), w.to(gpu), 1e-5)
    torch.cuda.synchronize()
    # the sum is torch's bf16 addition, bit for bit
    s_ref = (x.to(gpu) + r.to(gpu))
    np.testing.assert_array_equal(t2bits(s), t2bits(s_ref))
    # the norm is the unfused kernel on that sum, bit for bit, and within 1 ulp of the oracle
    np.testing.assert_array_equal(t2bits(y), t2bits(cke.rms_norm(s_ref, w.to(gpu), 1e-5)))
    assert_within_ulps(y, rms_norm_ref(t2f32(s_ref), t2f32(w), 1e-5), 1, what=f"add_rms_norm {shape}")
    with pytest.raises(RuntimeError):
        cke.add_rms_norm(x.to(gpu), r.to(gpu)[:, :, : C // 2], w.to(gpu), 1e-5)


@pytest.mark.parametrize("shape", [(1, 1, 8192), (64, 1, 8192), (2, 300, 1000), (3, 7, 13)])
def test_silu_mul_matches_torch(gpu, shape):
    from custom_kernels import custom_kernels_extension as cke
    import torch.nn.functional as F

    a = randn_bf16(shape, 81, scale=3.0).to(gpu)
    b = randn_bf16(shape, 82).to(gpu)
    y = cke.silu_mul(a, b)
    torch.cuda.synchronize()
    ref = F.silu(a) * b
    d = bf16_ulp(y, ref)
    assert d.max() <= 1 and (d > 0).mean() < 1e-3, f"silu_mul differs from torch: max {d.max()} ulp, {(d > 0).mean():.2e} of elements"
    # and against exact arithmetic with the same two roundings
    af, bf = t2f32(a).astype(np.float64), t2f32(b).astype(np.float64)
    s = round_to_bf16(af / (1.0 + np.exp(-af))).astype(np.float64)
    assert_within_ulps(y, s * bf, 1, what=f"silu_mul {shape}")


@pytest.mark.parametrize("rows,V", [(1, 128256), (64, 128256), (3, 1000), (2, 2048), (5, 2049), (1, 7)])
def test_argmax_first_maximum(gpu, rows, V):
    from custom_kernels import custom_kernels_extension as cke

    x = randn_bf16((rows, V), 91)
    # plant ties of the row maximum: the first one must win
    for r in range(rows):
        top = x[r].float().max().item() + 1.0
        pos = sorted({(r * 37 + 5) % V, (V - 1 - r) % V, V // 2})
        for p in pos:
            x[r, p] = top
    out = cke.argmax(x.to(gpu))
    torch.cuda.synchronize()
    want = torch.argmax(x.float(), dim=-1)
    first = torch.tensor([int(np.flatnonzero(t2f32(x[r]) == t2f32(x[r]).max())[0]) for r in range(rows)])
    assert out.dtype == torch.int64
    np.testing.assert_array_equal(out.cpu().numpy(), first.numpy())
    np.testing.assert_array_equal(out.cpu().numpy(), want.numpy())
    # strided rows (a slice of a wider matrix)
    wide = randn_bf16((rows, V + 9), 92).to(gpu)
    np.testing.assert_array_equal(cke.argmax(wide[:, :V]).cpu().numpy(),
                                  torch.argmax(wide[:, :V].float(), dim=-1).cpu().numpy())


def test_argmax_treats_nan_as_the_maximum_like_torch(gpu):
    """A NaN logit wins (the first one), as in torch.argmax: a numerical blow-up picks the same
    token on the graph-replayed and the eager path."""
    from custom_kernels import custom_kernels_extension as cke

    V = 5000
    x = randn_bf16((6, V), 93)
    x[0, 4000] = float("nan")                       # one NaN beats every number ...
    x[1, 4100] = float("nan"); x[1, 17] = float("nan"); x[1, 2500] = float("inf")   # ... the first of several wins, inf included
    x[2, :] = float("nan")                          # a row of NaNs: index 0
    x[3, 7] = float("inf"); x[3, 9] = float("inf")  # no NaN: first maximum
    x[4, :] = float("-inf")                         # all equal: index 0
    x[5, V - 1] = float("nan")                      # in the last chunk
    out = cke.argmax(x.to(gpu)).cpu()
    want = torch.argmax(x.float(), dim=-1)
    np.testing.assert_array_equal(out.numpy(), want.numpy())
    np.testing.assert_array_equal(out.numpy(), np.array([4000, 17, 0, 7, 0, V - 1]))


@pytest.mark.parametrize("rows,V,L,pos0", [(1, 128256, 256, 127), (64, 128256, 256, 200), (5, 1000, 20, 7), (3, 50, 9, 8)])
def test_greedy_step_matches_generate_bookkeeping(gpu, rows, V, L, pos0):
    """argmax + the per-token bookkeeping of generate() (model.py:371-378) in place on the device,
    against the same steps written with torch operators; two steps in a row."""
    from custom_kernels import custom_kernels_extension as cke

    g = torch.Generator().manual_seed(rows * 1000 + V)
    tokens = torch.randint(0, V, (rows, L), generator=g)
    text_mask = torch.rand((rows, L), generator=g) < 0.5
    eos = torch.zeros(rows, dtype=torch.bool)
    state = dict(tokens=tokens.to(gpu), text_mask=text_mask.to(gpu), tok=torch.zeros((rows, 1), dtype=torch.long, device=gpu),
                 pos=torch.tensor([pos0], dtype=torch.int32, device=gpu),
                 kv_len=torch.tensor([pos0 + 1], dtype=torch.int32, device=gpu), eos=eos.to(gpu))
    ref_tokens, ref_eos, ref_pos = tokens.clone(), eos.clone(), pos0
    for step in range(2):
        logits = randn_bf16((rows, V), 7 + step)
        want = torch.argmax(logits.float(), dim=-1)
        # every second row's pick is declared a stop token
        stop = torch.unique(torch.cat([want[::2], torch.tensor([V + 5])]))
        cke.greedy_step(logits.to(gpu), state["tokens"], state["text_mask"], state["tok"], state["pos"],
                        state["kv_len"], state["eos"], stop.to(gpu))
        torch.cuda.synchronize()
        cur = min(ref_pos + 1, L - 1)
        keep = text_mask[:, cur]
        nxt = torch.where(keep, ref_tokens[:, cur], want)
        ref_tokens[:, cur] = nxt
        ref_eos |= ~keep & torch.isin(nxt, stop)
        ref_pos += 1
        assert torch.equal(state["tokens"].cpu(), ref_tokens), f"tokens after step {step}"
        assert torch.equal(state["tok"].cpu().view(-1), nxt)
        assert torch.equal(state["eos"].cpu(), ref_eos)
        assert state["pos"].item() == ref_pos and state["kv_len"].item() == ref_pos + 1
