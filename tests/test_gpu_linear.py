"""GPU parity: the decode-step linear kernels (through the C ABI) against the float64 oracle."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import bf16_ulp_distance, randn_bf16, t2bits, t2f32
from oracle import linear_ref, swiglu_linear_ref

pytestmark = pytest.mark.gpu


def assert_linear_close(y, ref, what):
    """Within 1 bf16 ulp of the float64 result, except where the sum cancels to (nearly) nothing:
    there the float32 accumulation error, about 2^-24 per term relative to the LARGEST partial
    sum, can exceed the tiny result's own ulp, so an absolute 2^-18 of the row's largest |y| also
    passes."""
    ref = np.asarray(ref, dtype=np.float64)
    got = t2f32(y).astype(np.float64)
    d = bf16_ulp_distance(t2bits(y), t2bits(torch.from_numpy(ref.astype(np.float32)).to(torch.bfloat16)))
    slack = 2.0 ** -18 * np.abs(ref).max(axis=-1, keepdims=True)
    bad = (d > 1) & (np.abs(got - ref) > slack)
    assert not bad.any(), f"{what}: {bad.sum()} elements off by more than 1 ulp and the cancellation slack; " \
                          f"max distance {d.max()} ulp"

# (M, N, K): the 1B-architecture decode shapes (qkv, out projection, MLP down projection, lm head),
# batch sizes up to 64, and shapes off every multiple the kernel tiles by
# (rows above 16 are served by the split-K kernel and its finishing pass: N % 8 == 0, K % 128 == 0)
SHAPES = [(1, 3072, 2048), (1, 2048, 2048), (1, 2048, 8192), (1, 128256, 2048), (3, 1024, 512), (16, 3072, 2048),
          (17, 512, 256), (64, 3072, 2048), (64, 2048, 8192), (5, 20, 32), (2, 36, 64), (33, 104, 384),
          (64, 16, 4096), (1, 16, 32), (8, 6144, 4096), (4, 2048, 8192), (4, 20, 128), (2, 3072, 2048), (3, 4, 384),
          (16, 100, 96), (40, 2048, 2048), (64, 32768, 2048), (17, 20000, 1152), (33, 16384, 384)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_linear_decode_against_oracle(gpu, M, N, K):
    from custom_kernels import custom_kernels_extension as cke

    print(f"linear_decode M={M} N={N} K={K}", flush=True)
    x = randn_bf16((M, K), 11)
    w = randn_bf16((N, K), 12, scale=0.05)
    y = cke.linear_decode(x.to(gpu), w.to(gpu))
    torch.cuda.synchronize()
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    assert_linear_close(y, linear_ref(t2f32(x), t2f32(w)), f"linear {M}x{N}x{K}")


def test_linear_decode_layouts_and_errors(gpu):
    from custom_kernels import custom_kernels_extension as cke

    M, N, K = 4, 256, 512
    w = randn_bf16((N, K), 21, scale=0.05).to(gpu)
    buf = randn_bf16((M, 1, K + 64), 22).to(gpu)
    x = buf[..., :K]                                   # (M, 1, K) rows with a padded stride
    y = cke.linear_decode(x, w)
    assert y.shape == (M, 1, N)
    dense = cke.linear_decode(x.contiguous(), w)
    assert torch.equal(y, dense)
    wide = randn_bf16((N, K + 32), 23, scale=0.05).to(gpu)
    ys = cke.linear_decode(x, wide[:, :K])             # weight rows with a padded stride
    assert_linear_close(ys, linear_ref(t2f32(x), t2f32(wide[:, :K])), "strided weight")
    # the rows of a batch do not influence each other: row 2 alone gives the same bits
    assert torch.equal(cke.linear_decode(x[2:3], w), y[2:3])
    with pytest.raises(RuntimeError):
        cke.linear_decode(randn_bf16((65, K), 1).to(gpu), w)          # too many rows for this entry point
    with pytest.raises(RuntimeError):                                 # 17..64 rows need N % 8 == 0 and K % 128 == 0
        cke.linear_decode(randn_bf16((20, 96), 1).to(gpu), randn_bf16((64, 96), 2).to(gpu))
    with pytest.raises(RuntimeError):
        cke.linear_decode(randn_bf16((2, 48), 1).to(gpu), randn_bf16((8, 48), 2).to(gpu))   # K % 32 != 0
    with pytest.raises(RuntimeError):
        cke.linear_decode(randn_bf16((2, K + 32), 1).to(gpu), w)      # K mismatch
    with pytest.raises(RuntimeError):
        cke.linear_decode(randn_bf16((2, K), 1), w)                   # CPU tensor


@pytest.mark.parametrize("M,N,K", [(1, 8192, 2048), (12, 8192, 2048), (7, 1024, 256), (16, 14336, 4096), (9, 52, 64),
                                   (4, 1684, 1024), (2, 1684, 2048), (13, 3420, 4096), (4, 4680, 3072),
                                   (15, 3804, 4096)])
def test_linear_swiglu_decode(gpu, M, N, K):
    from custom_kernels import custom_kernels_extension as cke

    print(f"linear_swiglu_decode M={M} N={N} K={K}", flush=True)
    x = randn_bf16((M, K), 31)
    wg = randn_bf16((N, K), 32, scale=0.05)
    wu = randn_bf16((N, K), 33, scale=0.05)
    xd, wgd, wud = x.to(gpu), wg.to(gpu), wu.to(gpu)
    y = cke.linear_swiglu_decode(xd, wgd, wud)
    torch.cuda.synchronize()
    assert y.shape == (M, N)
    # The three-operator sequence has the same rounding points.  The sums over K are not added up in
    # the same order, though (the fused form deals its wavefronts over two matrices, and up to 4 rows
    # the plain linear splits the k range of a small matrix further): a gate or up value whose float32
    # sum straddles a bf16 rounding boundary rounds the other way now and then, and the product follows.
    seq = cke.silu_mul(cke.linear_decode(xd, wgd), cke.linear_decode(xd, wud))
    dseq = bf16_ulp_distance(t2bits(y), t2bits(seq))
    assert (dseq > 0).mean() < 0.02 and (dseq > 2).mean() < 2e-3
    # against exact arithmetic with the same rounding points: a gate or up value that rounds the other
    # way moves the product by about one ulp of that factor
    ref = swiglu_linear_ref(t2f32(x), t2f32(wg), t2f32(wu))
    d = bf16_ulp_distance(t2bits(y), t2bits(torch.from_numpy(ref.astype(np.float32)).to(torch.bfloat16)))
    assert (d > 2).mean() < 2e-3 and np.abs(t2f32(y) - ref).max() <= 0.02 * max(1.0, np.abs(ref).max())
    # and torch's own three operators on the same device
    lib = F.silu(F.linear(xd, wgd)) * F.linear(xd, wud)
    assert (y.float() - lib.float()).abs().max().item() <= 0.02 * max(1.0, lib.float().abs().max().item())


@pytest.mark.parametrize("M,N,K", [(1, 3072, 2048), (8, 3072, 2048), (11, 512, 2048), (1, 2048, 8192), (2, 128, 8192),
                                   (16, 100, 512), (3, 128256, 2048), (5, 64, 1536), (5, 4096, 4096), (5, 2048, 4096)])
def test_linear_fused_input_norm(gpu, M, N, K):
    from custom_kernels import custom_kernels_extension as cke
    from oracle import rms_norm_ref, round_to_bf16

    print(f"linear_decode_fused norm M={M} N={N} K={K}", flush=True)
    x = randn_bf16((M, 1, K), 41, scale=2.0)
    nw = randn_bf16((K,), 42, scale=0.1, mean=1.0)
    w = randn_bf16((N, K), 43, scale=0.05)
    xd, nwd, wd = x.to(gpu), nw.to(gpu), w.to(gpu)
    y = cke.linear_decode_fused(xd, wd, norm_weight=nwd, eps=1e-5)
    torch.cuda.synchronize()
    assert y.shape == (M, 1, N)
    # the two separate operators: the same bits except where the row's inverse rms differs in its
    # last float32 bit (the two kernels add the squares in different orders)
    seq = cke.linear_decode(cke.rms_norm(xd, nwd, 1e-5), wd)
    d = bf16_ulp_distance(t2bits(y), t2bits(seq))
    assert d.max() <= 1 and (d > 0).mean() < 0.02, f"fused norm vs sequence: max {d.max()} ulp, {(d > 0).mean():.3f} differ"
    # exact arithmetic with the rounding point of the stand-alone norm
    h = round_to_bf16(rms_norm_ref(t2f32(x), t2f32(nw), 1e-5))
    ref = linear_ref(h, t2f32(w))
    err = np.abs(t2f32(y).astype(np.float64) - ref)
    assert err.max() <= 2.0 ** -6 * max(1.0, np.abs(ref).max()), f"fused norm vs oracle: max err {err.max()}"


@pytest.mark.parametrize("M,N,K", [(1, 8192, 2048), (4, 1024, 512), (11, 8192, 2048), (16, 260, 256)])
@pytest.mark.parametrize("with_norm", [False, True])
def test_linear_fused_swiglu_with_residual(gpu, M, N, K, with_norm):
    """The SwiGLU form and the residual in one call (with and without the input norm): every
    optional part of linear_decode_fused applies whatever the others are."""
    from custom_kernels import custom_kernels_extension as cke

    if with_norm and M > cke.linear_decode_fused_max_rows(K):
        pytest.skip("more rows than the input norm stages")
    print(f"linear_decode_fused swiglu+residual M={M} N={N} K={K} norm={with_norm}", flush=True)
    x = randn_bf16((M, 1, K), 54).to(gpu)
    nw = randn_bf16((K,), 55, scale=0.1, mean=1.0).to(gpu) if with_norm else None
    wg = randn_bf16((N, K), 56, scale=0.05).to(gpu)
    wu = randn_bf16((N, K), 57, scale=0.05).to(gpu)
    r = randn_bf16((M, 1, N), 58, scale=3.0).to(gpu)
    y = cke.linear_decode_fused(x, wg, norm_weight=nw, w_up=wu, residual=r)
    t = cke.linear_decode_fused(x, wg, norm_weight=nw, w_up=wu)
    torch.cuda.synchronize()
    assert not torch.equal(y, t)                 # a dropped residual would pass every tolerance but this
    assert torch.equal(y, r + t)                 # torch's bf16 add: float sum, one rounding
    with pytest.raises(RuntimeError):            # more than 16 rows: no SwiGLU form, and nothing is dropped silently
        cke.linear_decode_fused(randn_bf16((17, K), 1).to(gpu), wg, w_up=wu, residual=randn_bf16((17, N), 2).to(gpu))


@pytest.mark.parametrize("M,N,K", [(1, 2048, 2048), (1, 2048, 8192), (9, 2048, 8192), (16, 256, 512), (64, 2048, 8192)])
def test_linear_fused_residual(gpu, M, N, K):
    from custom_kernels import custom_kernels_extension as cke

    print(f"linear_decode_fused residual M={M} N={N} K={K}", flush=True)
    x = randn_bf16((M, 1, K), 51).to(gpu)
    w = randn_bf16((N, K), 52, scale=0.05).to(gpu)
    r = randn_bf16((M, 1, N), 53, scale=3.0).to(gpu)
    y = cke.linear_decode_fused(x, w, residual=r)
    torch.cuda.synchronize()
    assert torch.equal(y, r + cke.linear_decode(x, w))    # torch's bf16 add: float sum, one rounding


def test_linear_fused_whole_mlp_and_limits(gpu):
    """ln_2 -> SwiGLU -> down projection + residual as the decode step chains them, against the
    separate operators; and the row limit of the input norm."""
    from custom_kernels import custom_kernels_extension as cke

    M, C, H = 4, 2048, 8192
    x = randn_bf16((M, 1, C), 61).to(gpu)
    nw = randn_bf16((C,), 62, scale=0.1, mean=1.0).to(gpu)
    wg = randn_bf16((H, C), 63, scale=0.03).to(gpu)
    wu = randn_bf16((H, C), 64, scale=0.03).to(gpu)
    wd = randn_bf16((C, H), 65, scale=0.03).to(gpu)
    t = cke.linear_decode_fused(x, wg, norm_weight=nw, eps=1e-5, w_up=wu)
    y = cke.linear_decode_fused(t, wd, residual=x)
    h = cke.rms_norm(x, nw, 1e-5)
    t_seq = cke.silu_mul(cke.linear_decode(h, wg), cke.linear_decode(h, wu))
    y_seq = x + cke.linear_decode(t_seq, wd)
    torch.cuda.synchronize()
    assert (t.float() - t_seq.float()).abs().max().item() <= 2.0 ** -7 * max(1.0, t_seq.float().abs().max().item())
    assert (y.float() - y_seq.float()).abs().max().item() <= 2.0 ** -6 * max(1.0, y_seq.float().abs().max().item())
    assert cke.linear_decode_fused_max_rows(2048) == 11 and cke.linear_decode_fused_max_rows(8192) == 2
    with pytest.raises(RuntimeError):
        cke.linear_decode_fused(randn_bf16((12, C), 1).to(gpu), wg, norm_weight=nw)   # too many rows to stage
    with pytest.raises(RuntimeError):
        cke.linear_decode_fused(x, wg, norm_weight=nw[:100])
    with pytest.raises(RuntimeError):                                                  # width not a multiple of 512
        cke.linear_decode_fused(randn_bf16((2, 1056), 1).to(gpu), randn_bf16((64, 1056), 2).to(gpu),
                                norm_weight=randn_bf16((1056,), 3).to(gpu))


@pytest.mark.parametrize("B,NH,KVH,HD,K,norm", [(1, 32, 8, 64, 2048, True), (8, 32, 8, 64, 2048, True),
                                                (16, 32, 8, 64, 2048, False), (3, 8, 2, 128, 512, True),
                                                (13, 32, 8, 64, 2048, False), (2, 4, 4, 64, 96, False)])
def test_linear_qkv_rope_append_equals_the_separate_operators(gpu, B, NH, KVH, HD, K, norm):
    from custom_kernels import custom_kernels_extension as cke
    from custom_kernels import precompute_freqs_cis

    print(f"linear_qkv_rope_append B={B} NH={NH} KVH={KVH} HD={HD} K={K} norm={norm}", flush=True)
    L, pos_val = 40, 17
    x = randn_bf16((B, 1, K), 71).to(gpu)
    w = randn_bf16(((NH + 2 * KVH) * HD, K), 72, scale=0.05).to(gpu)
    nw = randn_bf16((K,), 73, scale=0.1, mean=1.0).to(gpu) if norm else None
    table = precompute_freqs_cis(HD, 64, 500000.0, True, scale_factor=32.0, device=gpu)
    pos = torch.tensor([pos_val], dtype=torch.int32, device=gpu)
    base_k = randn_bf16((B + 1, L, KVH, HD), 74).to(gpu)
    base_v = randn_bf16((B + 1, L, KVH, HD), 75).to(gpu)

    ck1, cv1 = base_k.clone(), base_v.clone()
    q1 = cke.linear_qkv_rope_append(x, w, table, ck1, cv1, pos, NH, norm_weight=nw, eps=1e-5)
    ck2, cv2 = base_k.clone(), base_v.clone()
    qkv = cke.linear_decode_fused(x, w, norm_weight=nw, eps=1e-5) if norm else cke.linear_decode(x, w)
    q2 = cke.rot_embed_append(qkv, table, ck2, cv2, pos, NH)
    torch.cuda.synchronize()
    assert q1.shape == (B, 1, NH, HD)
    assert torch.equal(q1, q2)
    assert torch.equal(ck1, ck2) and torch.equal(cv1, cv2)
    # only token `pos` of the first B cache rows changed
    changed_k = (ck1 != base_k).any(dim=-1).any(dim=-1)
    assert changed_k[:B, pos_val].all() and changed_k.sum().item() == B
    # a position outside the cache writes nothing
    ck3, cv3 = base_k.clone(), base_v.clone()
    cke.linear_qkv_rope_append(x, w, table, ck3, cv3, torch.tensor([L], dtype=torch.int32, device=gpu), NH,
                               norm_weight=nw, eps=1e-5)
    torch.cuda.synchronize()
    assert torch.equal(ck3, base_k) and torch.equal(cv3, base_v)


# ---- split-K linear for 17..64 rows and the operators that add its splits up
def _sum_in_split_order(part):
    acc = part[0].clone()
    for s in range(1, part.shape[0]):
        acc += part[s]
    return acc


@pytest.mark.parametrize("M,N,K,ksplit", [(64, 3072, 2048, 0), (64, 2048, 2048, 0), (64, 2048, 8192, 0), (17, 2048, 2048, 4),
                                          (40, 264, 384, 1), (33, 8, 128, 1), (64, 16384, 2048, 4), (64, 2048, 2048, 16),
                                          (20, 1000, 1280, 3), (20, 1000, 1280, 2), (33, 512, 896, 1), (17, 256, 768, 1),
                                          (64, 2048, 8192, 8), (24, 8192, 384, 1), (64, 3072, 2048, 2)])
def test_linear_splitk_against_oracle(gpu, M, N, K, ksplit):
    from custom_kernels import custom_kernels_extension as cke

    print(f"linear_splitk M={M} N={N} K={K} ksplit={ksplit}", flush=True)
    x = randn_bf16((M, K), 81)
    w = randn_bf16((N, K), 82, scale=0.05)
    part = cke.linear_splitk(x.to(gpu), w.to(gpu), ksplit)
    torch.cuda.synchronize()
    assert part.dtype == torch.float32 and part.shape[1:] == (M, N) and (ksplit == 0 or part.shape[0] == ksplit)
    y = _sum_in_split_order(part).to(torch.bfloat16)
    assert_linear_close(y, linear_ref(t2f32(x), t2f32(w)), f"splitk {M}x{N}x{K}")
    # every split alone is the product over its own k range
    per = -(-(K // 128) // part.shape[0]) * 128
    s = part.shape[0] - 1
    ref_last = linear_ref(t2f32(x)[:, s * per:], t2f32(w)[:, s * per:])
    assert np.abs(part[s].cpu().numpy() - ref_last).max() <= 1e-4 * max(1.0, np.abs(ref_last).max())


@pytest.mark.parametrize("M,N,K,with_res", [(64, 2048, 8192, True), (64, 3072, 2048, False), (17, 256, 128, True),
                                            (33, 2048, 2048, True)])
def test_linear_splitk_finish_equals_the_unsplit_linear(gpu, M, N, K, with_res):
    """Split-K + finish against the float64 oracle, and the residual form against a bf16 linear
    followed by a bf16 addition (the two roundings of model.py:147-148)."""
    from custom_kernels import custom_kernels_extension as cke

    print(f"linear_splitk_finish M={M} N={N} K={K} residual={with_res}", flush=True)
    x = randn_bf16((M, 1, K), 41)
    w = randn_bf16((N, K), 42, scale=0.05)
    part = cke.linear_splitk(x.to(gpu), w.to(gpu))
    y = cke.linear_splitk_finish(part)
    torch.cuda.synchronize()
    assert y.shape == (M, N)
    assert_linear_close(y, linear_ref(t2f32(x), t2f32(w)).reshape(M, N), "split-K + finish")
    assert torch.equal(y, _sum_in_split_order(part).to(torch.bfloat16))
    assert torch.equal(cke.linear_decode(x.to(gpu), w.to(gpu)).view(M, N), y)      # what linear_decode does at these rows
    if with_res:
        res = randn_bf16((M, 1, N), 43).to(gpu)
        yr = cke.linear_splitk_finish(part, res)
        assert torch.equal(yr, (res.view(M, N) + y))
        assert torch.equal(cke.linear_decode_fused(x.to(gpu), w.to(gpu), residual=res).view(M, N), yr)
    with pytest.raises(RuntimeError):
        cke.linear_splitk_finish(part.to(torch.bfloat16))
    with pytest.raises(RuntimeError):
        cke.linear_splitk_finish(part, randn_bf16((M, N + 8), 44).to(gpu))


def test_linear_splitk_errors(gpu):
    from custom_kernels import custom_kernels_extension as cke

    w = randn_bf16((256, 2048), 1).to(gpu)
    with pytest.raises(RuntimeError):
        cke.linear_splitk(randn_bf16((64, 2048), 2).to(gpu), w, 1)        # 2048 k per workgroup: more than it stages
    with pytest.raises(RuntimeError):
        cke.linear_splitk(randn_bf16((64, 2048), 2).to(gpu), w, 17)       # more splits than 128-k chunks
    with pytest.raises(RuntimeError):
        cke.linear_splitk(randn_bf16((64, 96), 2).to(gpu), randn_bf16((256, 96), 3).to(gpu))   # K % 128 != 0
    with pytest.raises(RuntimeError):
        cke.linear_splitk(randn_bf16((65, 2048), 2).to(gpu), w)


@pytest.mark.parametrize("rows,C,ksplit", [(64, 2048, 16), (17, 2048, 4), (64, 4096, 8), (3, 8, 1), (5, 8192, 2)])
def test_add_rms_norm_partials_equals_sum_then_add_rms_norm(gpu, rows, C, ksplit):
    from custom_kernels import custom_kernels_extension as cke

    x = randn_bf16((rows, 1, C), 91).to(gpu)
    w = randn_bf16((C,), 92, scale=0.1, mean=1.0).to(gpu)
    part = (torch.randn((ksplit, rows, C), generator=torch.Generator().manual_seed(93)) * 0.7).to(gpu)
    s1, y1 = cke.add_rms_norm_partials(x, part, w, 1e-5)
    r = _sum_in_split_order(part).to(torch.bfloat16).view(rows, 1, C)
    s2, y2 = cke.add_rms_norm(x, r, w, 1e-5)
    torch.cuda.synchronize()
    assert torch.equal(s1, s2)
    d = bf16_ulp_distance(t2bits(y1), t2bits(y2))     # the two kernels add the squares in different orders
    assert d.max() <= 1 and (d > 0).mean() < 0.02


@pytest.mark.parametrize("B,NH,KVH,HD,ksplit", [(64, 32, 8, 64, 8), (17, 8, 2, 128, 3), (2, 4, 4, 64, 1)])
def test_rot_embed_append_partials_equals_sum_then_rot_embed_append(gpu, B, NH, KVH, HD, ksplit):
    from custom_kernels import custom_kernels_extension as cke
    from custom_kernels import precompute_freqs_cis

    L, pos_val = 24, 11
    N = (NH + 2 * KVH) * HD
    part = torch.randn((ksplit, B, N), generator=torch.Generator().manual_seed(95)).to(gpu)
    table = precompute_freqs_cis(HD, 64, 500000.0, True, scale_factor=32.0, device=gpu)
    pos = torch.tensor([pos_val], dtype=torch.int32, device=gpu)
    base_k = randn_bf16((B, L, KVH, HD), 96).to(gpu)
    base_v = randn_bf16((B, L, KVH, HD), 97).to(gpu)
    ck1, cv1 = base_k.clone(), base_v.clone()
    q1 = cke.rot_embed_append_partials(part, table, ck1, cv1, pos, NH)
    ck2, cv2 = base_k.clone(), base_v.clone()
    qkv = _sum_in_split_order(part).to(torch.bfloat16).view(B, 1, N)
    q2 = cke.rot_embed_append(qkv, table, ck2, cv2, pos, NH)
    torch.cuda.synchronize()
    assert torch.equal(q1, q2) and torch.equal(ck1, ck2) and torch.equal(cv1, cv2)
