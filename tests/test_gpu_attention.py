"""GPU parity: split-KV decode attention + combine (through the C ABI) against the float64
oracle on the same seeded inputs.  Tolerance: atol 2e-2 / rtol 1.6e-2 on the bf16 output
(helpers.ATTN_ATOL / ATTN_RTOL)."""

import numpy as np
import pytest
import torch

from helpers import ATTN_REG_ATOL, ATTN_REG_FEW_TOKENS, ATTN_REG_RTOL, assert_attn_close, make_qkv, randn_bf16, t2bits, t2f32
from oracle import attention_decode_ref

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("attn_kernel")]


def _run(gpu, B, QH, KVH, S, HD, seed=42, cache_len=None, splits=0, tweak=None):
    from custom_kernels import custom_kernels_extension as cke

    print(f"attention B={B} QH={QH} KVH={KVH} S={S} HD={HD} L={cache_len} splits={splits} seed={seed}", flush=True)
    q, k, v = make_qkv(B, QH, KVH, S, HD, seed=seed, cache_len=cache_len)
    if tweak is not None:
        tweak(q, k, v)
    qg, kg, vg = make_qkv(B, QH, KVH, S, HD, seed=seed, cache_len=cache_len, device=gpu)
    if tweak is not None:
        tweak(qg, kg, vg)
    out = cke.flash_attention_decode(qg, kg, vg, splits)
    torch.cuda.synchronize()
    assert out.shape == qg.shape and out.stride() == qg.stride()
    ref = attention_decode_ref(t2f32(q), t2f32(k), t2f32(v))
    err = assert_attn_close(out, ref, what=f"B{B} QH{QH} KVH{KVH} S{S} HD{HD} splits{splits}", min_kv_len=S)
    return out, ref, err


@pytest.mark.parametrize("HD", [64, 128])
@pytest.mark.parametrize("S", [1, 2, 7, 31, 32, 33, 63, 64, 65, 127, 128, 129, 200, 257, 1000])
def test_ragged_lengths(gpu, HD, S):
    _run(gpu, 2, 8, 2, S, HD, seed=S)


@pytest.mark.parametrize("HD,QH,KVH", [(64, 4, 4), (64, 8, 4), (64, 12, 4), (64, 32, 8), (64, 16, 2),
                                        (128, 4, 4), (128, 4, 2), (128, 24, 8), (128, 32, 8), (128, 64, 8),
                                        (64, 6, 3), (128, 6, 6), (64, 5, 5), (128, 16, 16), (64, 32, 16),
                                        (128, 8, 1), (64, 7, 7)])
@pytest.mark.parametrize("splits", [0, 1, 4])
def test_head_ratios(gpu, HD, QH, KVH, splits):
    _run(gpu, 2, QH, KVH, 333, HD, seed=QH + KVH, splits=splits)


@pytest.mark.parametrize("B,QH,KVH,S,HD,splits", [(40, 32, 8, 300, 64, 2), (40, 32, 8, 300, 128, 3),
                                                   (130, 8, 8, 97, 64, 2), (33, 32, 4, 1000, 128, 31),
                                                   (515, 2, 2, 70, 64, 2), (36, 32, 8, 2100, 128, 32),
                                                   (100, 32, 8, 1024, 128, 0),
                                                   (4, 64, 16, 500, 64, 3), (2, 32, 32, 300, 128, 2),
                                                   (16, 16, 4, 400, 64, 5), (8, 24, 8, 350, 128, 4)])
def test_many_sequences_with_few_splits(gpu, attn_kernel, B, QH, KVH, S, HD, splits):
    """A thousand or more (batch, query head) pairs with 2 ... 32 splits each: the combine runs with a
    wavefront per pair (515 x 2 pairs do not fill its last workgroup); the case with 0 splits takes the plan's
    own choice for 100 long sequences (two splits with the MFMA kernel); the last four (and the first two)
    have (head groups x batch) a multiple of 8, where the combine deals its pairs to the XCD whose split
    workgroups wrote them: one, two and four head groups of eight kv heads, four kv heads, head ratio 3."""
    if splits == 0:
        from custom_kernels import custom_kernels_extension as cke
        assert cke.attention_num_splits(B, KVH, S, HD, 256) == (2 if attn_kernel == "mfma" else 1)
        q, k, v = make_qkv(B, QH, KVH, S, HD, seed=9)
        qg, kg, vg = make_qkv(B, QH, KVH, S, HD, seed=9, device=gpu)
        out = cke.flash_attention_decode(qg, kg, vg)
        torch.cuda.synchronize()
        rows = [0, 1, 50, B - 1]                      # the oracle on a few sequences only
        ref = attention_decode_ref(t2f32(q[rows]), t2f32(k[rows]), t2f32(v[rows]))
        assert_attn_close(out[rows], ref, what="100 long sequences", min_kv_len=S)
        return
    _run(gpu, B, QH, KVH, S, HD, seed=B + splits, splits=splits)


@pytest.mark.parametrize("B,QH,KVH,S,HD", [(1, 32, 8, 513, 128), (1, 32, 8, 1000, 128), (1, 32, 8, 2048, 128),
                                            (1, 32, 8, 4097, 128), (1, 32, 8, 8192, 128), (1, 32, 8, 600, 64),
                                            (1, 32, 8, 1024, 64), (1, 32, 8, 3000, 64), (1, 32, 8, 4096, 64),
                                            (3, 8, 2, 777, 128), (2, 32, 8, 1500, 64), (5, 6, 3, 290, 128),
                                            (1, 8, 1, 5000, 128), (64, 8, 2, 300, 128)])
def test_medium_sequences_over_few_heads(gpu, attn_kernel, B, QH, KVH, S, HD):
    """The plan's own choice for medium lengths over few (batch, kv head) pairs: with the MFMA kernel,
    cooperative workgroups over several splits (one merged partial row per workgroup) plus the combine.
    Checked against the oracle and against a forced split count, which takes the streaming form."""
    from custom_kernels import custom_kernels_extension as cke

    if attn_kernel == "mfma":
        assert cke.attention_num_splits(B, KVH, S, HD, 256) > 1
    out, ref, _ = _run(gpu, B, QH, KVH, S, HD, seed=S + HD)
    qg, kg, vg = make_qkv(B, QH, KVH, S, HD, seed=S + HD, device=gpu)
    forced = cke.flash_attention_decode(qg, kg, vg, 5)
    torch.cuda.synchronize()
    assert (out.float() - forced.float()).abs().max().item() <= 2.0 ** -7 * max(1.0, np.abs(ref).max())


@pytest.mark.parametrize("HD", [64, 128])
@pytest.mark.parametrize("splits", [1, 2, 5, 16, 512])
def test_result_independent_of_split_count(gpu, HD, splits):
    base, ref, _ = _run(gpu, 1, 32, 8, 2048, HD, seed=5, splits=1)
    out, _, _ = _run(gpu, 1, 32, 8, 2048, HD, seed=5, splits=splits)
    d = np.abs(t2f32(out).astype(np.float64) - t2f32(base).astype(np.float64))
    assert d.max() <= 2.0 ** -7 * max(1.0, np.abs(ref).max()), "split count changes the result beyond bf16 rounding"


@pytest.mark.parametrize("HD", [64, 128])
def test_dominant_key_in_a_late_split(gpu, HD):
    """One key far above the rest, sitting in the last split: the log-sum-exp combine must
    hand that split ~all the weight.  A combine that reuses split 0's statistics for every
    split (custom_kernels.cu:184,201,209) returns the mean of the splits and fails this."""
    S = 1500

    def tweak(q, k, v):
        k[0, 1, S - 10] = q[0, 5, 0] * 4.0   # query head 5 -> kv head 1

    out, ref, _ = _run(gpu, 1, 32, 8, S, HD, seed=3, splits=8, tweak=tweak)
    q, k, v = make_qkv(1, 32, 8, S, HD, seed=3)
    got = t2f32(out)[0, 5, 0]
    assert np.abs(got - t2f32(v)[0, 1, S - 10]).max() < 0.05
    assert np.abs(ref[0, 5, 0] - t2f32(v)[0, 1, S - 10]).max() < 0.05


@pytest.mark.parametrize("HD", [64, 128])
def test_cache_view_and_dense_layouts_give_identical_bits(gpu, HD):
    """Same values through three layouts: a slice of a longer cache (batch stride L*KVH*HD,
    model.py:89,107), the benchmark's token-major tensor (benchmark_kernel.py:165-173) and
    a head-major contiguous (B, KVH, S, HD) tensor."""
    from custom_kernels import custom_kernels_extension as cke

    B, QH, KVH, S = 3, 32, 8, 777
    q, k, v = make_qkv(B, QH, KVH, S, HD, seed=9, cache_len=1024, device=gpu)
    a = cke.flash_attention_decode(q, k, v)
    kt = k.transpose(1, 2).contiguous().transpose(1, 2)
    vt = v.transpose(1, 2).contiguous().transpose(1, 2)
    b = cke.flash_attention_decode(q, kt, vt)
    c = cke.flash_attention_decode(q.contiguous(), k.contiguous(), v.contiguous())
    torch.cuda.synchronize()
    assert k.stride() != kt.stride() != k.contiguous().stride()
    np.testing.assert_array_equal(t2bits(a), t2bits(b))
    np.testing.assert_array_equal(t2bits(a), t2bits(c))


def test_equal_value_rows_return_that_row(gpu):
    from custom_kernels import custom_kernels_extension as cke

    q, k, v = make_qkv(2, 32, 8, 4096, 128, seed=1, device=gpu)
    row = randn_bf16((2, 8, 1, 128), 77).to(gpu)
    v_const = row.expand(2, 8, 4096, 128).transpose(1, 2).contiguous().transpose(1, 2)
    out = cke.flash_attention_decode(q, k, v_const)
    torch.cuda.synchronize()
    want = row.repeat_interleave(4, dim=1)
    # a convex combination of identical rows: only bf16 rounding of the normalised sum remains
    assert (out.float() - want.float()).abs().max().item() <= 2.0 ** -7 * want.float().abs().max().item()


def test_very_long_sequence_by_property(gpu):
    """KV length 131072 at head size 128 (0.5 GB of K+V): too large for the float64 oracle to be
    worth it, so the result is pinned by a size-independent property -- with identical V rows per
    head the output must be that row whatever the scores are -- plus agreement between the
    automatic plan and a forced, different split count."""
    from custom_kernels import custom_kernels_extension as cke

    B, QH, KVH, S, HD = 1, 32, 8, 131072, 128
    g = torch.Generator(device="cpu").manual_seed(5)
    q = torch.randn((B, 1, QH, HD), generator=g).to(torch.bfloat16).to(gpu).transpose(1, 2)
    k = torch.randn((B, S, KVH, HD), generator=g).to(torch.bfloat16).to(gpu).transpose(1, 2)
    row = torch.randn((B, 1, KVH, HD), generator=g).to(torch.bfloat16).to(gpu)
    v = row.expand(B, S, KVH, HD).contiguous().transpose(1, 2)
    out = cke.flash_attention_decode(q, k, v)
    want = row.transpose(1, 2).repeat_interleave(QH // KVH, dim=1)
    assert (out.float() - want.float()).abs().max().item() <= 2.0 ** -7 * want.float().abs().max().item()
    v2 = torch.randn((B, S, KVH, HD), generator=g).to(torch.bfloat16).to(gpu).transpose(1, 2)
    a = cke.flash_attention_decode(q, k, v2)
    b2 = cke.flash_attention_decode(q, k, v2, 37)
    torch.cuda.synchronize()
    assert (a.float() - b2.float()).abs().max().item() <= 2.0 ** -7


def test_inputs_are_not_modified_and_errors_are_raised(gpu):
    from custom_kernels import custom_kernels_extension as cke

    q, k, v = make_qkv(1, 32, 8, 300, 64, seed=2, device=gpu)
    qb, kb, vb = t2bits(q), t2bits(k), t2bits(v)
    cke.flash_attention_decode(q, k, v)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(t2bits(q), qb)
    np.testing.assert_array_equal(t2bits(k), kb)
    np.testing.assert_array_equal(t2bits(v), vb)
    with pytest.raises(RuntimeError, match="Unsupported head size"):
        cke.flash_attention_decode(*make_qkv(1, 8, 2, 16, 96, device=gpu))
    with pytest.raises(RuntimeError, match="Unsupported QKV head ratio"):
        cke.flash_attention_decode(*make_qkv(1, 10, 2, 16, 64, device=gpu))
    with pytest.raises(RuntimeError, match="BFloat16"):
        cke.flash_attention_decode(q.float(), k, v)
    # a token stride of 2^24 elements or more is refused (a tile's rows are addressed with 32-bit
    # offsets); nothing is read through the view
    wide = torch.zeros((1 << 24) + 8 * 64, device=gpu, dtype=torch.bfloat16).as_strided((1, 8, 2, 64), (0, 64, 1 << 24, 1))
    with pytest.raises(RuntimeError, match="stride"):
        cke.flash_attention_decode(q, wide, wide)


def test_more_sequences_than_one_grid_dimension_holds(gpu):
    """The batch index is a grid dimension of at most 65535 entries; a larger batch goes out in slices.
    Every sequence, those of the second slice included, must match the oracle."""
    from custom_kernels import custom_kernels_extension as cke

    B, QH, KVH, S, HD = 65535 + 70, 2, 1, 40, 64
    q, k, v = make_qkv(B, QH, KVH, S, HD, seed=77)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    for splits in (1, 2):
        out = cke.flash_attention_decode(qg, kg, vg, splits)
        torch.cuda.synchronize()
        tail = slice(B - 200, B)
        ref = attention_decode_ref(t2f32(q[tail]), t2f32(k[tail]), t2f32(v[tail]))
        assert_attn_close(out[tail], ref, what=f"last 200 of {B} sequences, splits {splits}", min_kv_len=S)
        head = slice(0, 64)
        ref = attention_decode_ref(t2f32(q[head]), t2f32(k[head]), t2f32(v[head]))
        assert_attn_close(out[head], ref, what=f"first 64 of {B} sequences, splits {splits}", min_kv_len=S)


def test_runs_on_the_current_stream(gpu):
    from custom_kernels import custom_kernels_extension as cke

    q, k, v = make_qkv(2, 32, 8, 512, 64, seed=4, device=gpu)
    ref = cke.flash_attention_decode(q, k, v)
    torch.cuda.synchronize()
    s = torch.cuda.Stream(device=gpu)
    with torch.cuda.stream(s):
        out = cke.flash_attention_decode(q, k, v)
    s.synchronize()
    np.testing.assert_array_equal(t2bits(out), t2bits(ref))


# ---- the benchmark configurations at full size (oracle in float64, chunked over the batch)
# name: (B, QH, KVH, S, HD, splits the MFMA plan makes on 256 compute units when the workspace carries
# arrival counters, launches of that plan).  Every shape the benchmark line reports is here at its own size.
FULL = {
    "c1": (1, 32, 8, 256, 64, 1, 1),
    "c2_s512": (1, 32, 8, 512, 128, 8, 1),
    "c2_s1024": (1, 32, 8, 1024, 128, 16, 1),
    "c2_s2048": (1, 32, 8, 2048, 128, 32, 1),
    "c2_s4096": (1, 32, 8, 4096, 128, 32, 1),
    "c2_s8192": (1, 32, 8, 8192, 128, 32, 1),
    "c2_s16384": (1, 32, 8, 16384, 128, 32, 1),
    "c2_s32768": (1, 32, 8, 32768, 128, 32, 1),
    "hd128_s65536": (1, 32, 8, 65536, 128, 205, 2),
    "hd64_s4096": (1, 32, 8, 4096, 64, 32, 1),
    "hd64_s8192": (1, 32, 8, 8192, 64, 32, 1),
    "hd64_s16384": (1, 32, 8, 16384, 64, 32, 1),
    "hd64_s32768": (1, 32, 8, 32768, 64, 171, 2),
    "hd64_s65536": (1, 32, 8, 65536, 64, 205, 2),
    "c3a": (256, 32, 8, 256, 64, 1, 1),
    "c3b": (16, 32, 8, 4096, 64, 11, 2),
}


@pytest.mark.parametrize("name", list(FULL))
def test_baseline_shapes_full_size(gpu, attn_kernel, name):
    from custom_kernels import _l3lib
    from custom_kernels import custom_kernels_extension as cke

    B, QH, KVH, S, HD, plan_splits, plan_launches = FULL[name]
    print(f"full-size {name}: B={B} S={S} HD={HD}", flush=True)
    if attn_kernel == "mfma":
        # the test follows the plan: these are the split counts and launch counts the benchmark line reports
        W = _l3lib.L3_ATTN_FLAG_WS_COUNTERS
        assert cke.attention_num_splits(B, KVH, S, HD, 256, flags=W) == plan_splits
        if torch.cuda.get_device_properties(gpu).multi_processor_count == 256:
            assert _l3lib.load().l3_attn_launches(B, QH, KVH, S, HD, 0, W) == plan_launches
    q, k, v = make_qkv(B, QH, KVH, S, HD, seed=42)
    qg, kg, vg = make_qkv(B, QH, KVH, S, HD, seed=42, device=gpu)
    out = cke.flash_attention_decode(qg, kg, vg)
    torch.cuda.synchronize()
    worst = 0.0
    for b0 in range(0, B, 32):
        sl = slice(b0, min(B, b0 + 32))
        ref = attention_decode_ref(t2f32(q[sl]), t2f32(k[sl]), t2f32(v[sl]))
        worst = max(worst, assert_attn_close(out[sl], ref, what=f"full-size {name}", min_kv_len=S))
    print(f"  max abs err {worst:.3e}", flush=True)


# ---- the two stages on their own (sequence held in several pieces)
@pytest.mark.parametrize("HD", [64, 128])
def test_split_stage_partials_match_oracle(gpu, HD):
    from custom_kernels import custom_kernels_extension as cke
    from oracle import attention_split_partials_ref

    B, QH, KVH, S = 2, 8, 2, 150
    q, k, v = make_qkv(B, QH, KVH, S, HD, seed=21)
    qg, kg, vg = make_qkv(B, QH, KVH, S, HD, seed=21, device=gpu)
    po, pml = cke.flash_attention_split(qg, kg, vg, 1)
    torch.cuda.synchronize()
    assert po.shape == (B, QH, 1, HD) and pml.shape == (B, QH, 1, 2)
    o, m, l = attention_split_partials_ref(t2f32(q), t2f32(k), t2f32(v), [0, S])
    LOG2E = 1.4426950408889634
    np.testing.assert_allclose(pml[:, :, 0, 0].cpu().numpy(), m[0] * LOG2E, rtol=1e-5, atol=1e-4)
    # P is rounded to bf16 before the second product on the MFMA path: 2^-8 relative per term
    np.testing.assert_allclose(pml[:, :, 0, 1].cpu().numpy(), l[0], rtol=2e-5)
    np.testing.assert_allclose(po[:, :, 0].cpu().numpy(), o[0], rtol=0, atol=8e-3 * np.abs(o[0]).max())


@pytest.mark.parametrize("HD", [64, 128])
def test_pieces_of_a_sequence_combine_to_the_whole(gpu, HD):
    """Token ranges processed separately (as if on different devices), partials concatenated
    along the split axis, one combine: equals attention over the whole sequence."""
    from custom_kernels import custom_kernels_extension as cke

    B, QH, KVH, S = 2, 32, 8, 1000
    q, k, v = make_qkv(B, QH, KVH, S, HD, seed=31)
    k[0, 3, 900] = q[0, 13, 0] * 4.0          # a dominant key in the last piece
    qg, kg, vg = make_qkv(B, QH, KVH, S, HD, seed=31, device=gpu)
    kg[0, 3, 900] = qg[0, 13, 0] * 4.0
    pieces = [(0, 333), (333, 400), (400, 1000)]
    parts = [cke.flash_attention_split(qg, kg[:, :, a:b], vg[:, :, a:b], ns) for (a, b), ns in zip(pieces, (0, 1, 5))]
    po = torch.cat([p[0] for p in parts], dim=2)
    pml = torch.cat([p[1] for p in parts], dim=2)
    out = cke.flash_attention_combine(po, pml)
    torch.cuda.synchronize()
    assert out.shape == (B, QH, 1, HD) and out.stride() == qg.stride()
    assert_attn_close(out, attention_decode_ref(t2f32(q), t2f32(k), t2f32(v)), what="pieces")
    whole = cke.flash_attention_decode(qg, kg, vg)
    assert (out.float() - whole.float()).abs().max().item() <= 2.0 ** -7 * max(1.0, whole.float().abs().max().item())


# ---- KV length read from device memory (one recorded launch serves a growing cache)
@pytest.mark.parametrize("HD,B,L", [(64, 1, 256), (64, 3, 300), (128, 2, 1024), (64, 64, 256), (128, 40, 200)])
def test_device_side_kv_length(gpu, HD, B, L):
    from custom_kernels import custom_kernels_extension as cke

    QH, KVH = 32, 8
    q, k, v = make_qkv(B, QH, KVH, L, HD, seed=41)
    qg, kg, vg = make_qkv(B, QH, KVH, L, HD, seed=41, device=gpu)
    kv_len = torch.zeros(1, dtype=torch.int32, device=gpu)
    for S in (1, 2, 63, 64, 65, 129, L - 1, L):
        kv_len.fill_(S)
        out = cke.flash_attention_decode_devlen(qg, kg, vg, kv_len)
        torch.cuda.synchronize()
        ref = attention_decode_ref(t2f32(q), t2f32(k[:, :, :S]), t2f32(v[:, :, :S]))
        assert_attn_close(out, ref, what=f"devlen S={S} of L={L}", min_kv_len=S)
        # a forced split count (streaming form of the kernel) agrees to bf16 rounding
        forced = cke.flash_attention_decode_devlen(qg, kg, vg, kv_len, 3)
        assert (out.float() - forced.float()).abs().max().item() <= 2.0 ** -7 * max(1.0, np.abs(ref).max())


@pytest.mark.parametrize("splits", [0, 4])
def test_device_side_kv_length_below_one_attends_to_the_first_token(gpu, splits):
    """*kv_len <= 0 is clamped to 1: the output is V[:, :, 0] (softmax over one token), never stale
    partials or a 0/0."""
    from custom_kernels import custom_kernels_extension as cke

    qg, kg, vg = make_qkv(2, 32, 8, 512, 64, seed=43, device=gpu)
    kv_len = torch.zeros(1, dtype=torch.int32, device=gpu)
    for n in (0, -7):
        kv_len.fill_(n)
        out = cke.flash_attention_decode_devlen(qg, kg, vg, kv_len, splits)
        torch.cuda.synchronize()
        want = vg[:, :, 0].repeat_interleave(4, dim=1).unsqueeze(2)       # query head h reads kv head h // 4
        assert torch.equal(out, want), f"kv_len={n} splits={splits}"


def test_caller_supplied_outputs_are_validated(gpu):
    """A wrong `out` would be written through its raw pointer with the query's shape."""
    from custom_kernels import custom_kernels_extension as cke

    qg, kg, vg = make_qkv(2, 32, 8, 256, 64, seed=44, device=gpu)
    kv_len = torch.full((1,), 256, dtype=torch.int32, device=gpu)
    good = torch.empty_like(qg)
    assert cke.flash_attention_decode_devlen(qg, kg, vg, kv_len, out=good) is good
    bad_outs = [torch.empty((2, 32, 1, 32), dtype=torch.bfloat16, device=gpu),        # too small
                torch.empty(qg.shape, dtype=torch.float16, device=gpu),              # wrong dtype
                torch.empty(qg.shape, dtype=torch.bfloat16),                          # wrong device
                torch.empty((2, 32, 1, 128), dtype=torch.bfloat16, device=gpu)[..., ::2],   # strided last dim
                torch.empty((2, 32, 1, 68), dtype=torch.bfloat16, device=gpu)[..., :64]]    # rows off 16-byte boundaries
    for bad in bad_outs:
        with pytest.raises(RuntimeError):
            cke.flash_attention_decode_devlen(qg, kg, vg, kv_len, out=bad)
        with pytest.raises(RuntimeError):
            cke.flash_attention_decode_static(qg, kg, vg, bad)
    with pytest.raises(RuntimeError):
        cke.flash_attention_decode_devlen(qg, kg, vg, kv_len.cpu())
    qkv = randn_bf16((2, 1, 48 * 64), 45).to(gpu)
    cache = torch.zeros((2, 16, 8, 64), dtype=torch.bfloat16, device=gpu)
    table = torch.zeros((16, 64), dtype=torch.float32, device=gpu)
    pos = torch.zeros(1, dtype=torch.int32, device=gpu)
    for bad in (torch.empty((2, 1, 32, 32), dtype=torch.bfloat16, device=gpu),
                torch.empty((2, 1, 32, 64), dtype=torch.float16, device=gpu),
                torch.empty((2, 1, 32, 64), dtype=torch.bfloat16)):
        with pytest.raises(RuntimeError):
            cke.rot_embed_append(qkv, table, cache, cache.clone(), pos, 32, out=bad)
    with pytest.raises(RuntimeError):
        cke.rot_embed_append(qkv, table, cache, cache.clone(), pos.cpu(), 32)


def test_concurrent_streams_do_not_share_scratch(gpu):
    """Two streams run split + combine calls at the same time; each stream has its own workspace
    in the shim, so the results must equal the serial ones bit for bit."""
    from custom_kernels import custom_kernels_extension as cke

    a = make_qkv(1, 32, 8, 6000, 128, seed=51, device=gpu)
    b = make_qkv(1, 32, 8, 5000, 128, seed=52, device=gpu)
    ra, rb = cke.flash_attention_decode(*a), cke.flash_attention_decode(*b)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(device=gpu), torch.cuda.Stream(device=gpu)
    outs_a, outs_b = [], []
    for _ in range(20):
        with torch.cuda.stream(s1):
            outs_a.append(cke.flash_attention_decode(*a))
        with torch.cuda.stream(s2):
            outs_b.append(cke.flash_attention_decode(*b))
    torch.cuda.synchronize()
    for o in outs_a:
        np.testing.assert_array_equal(t2bits(o), t2bits(ra))
    for o in outs_b:
        np.testing.assert_array_equal(t2bits(o), t2bits(rb))


# ---- causal prefill (T > 1) through the same tile loop
@pytest.mark.parametrize("HD", [64, 128])
@pytest.mark.parametrize("B,QH,KVH,T,S", [(1, 32, 8, 128, 128), (2, 8, 2, 37, 37), (1, 4, 4, 16, 16), (3, 24, 8, 5, 5),
                                           (1, 16, 2, 130, 130), (2, 32, 8, 64, 200), (1, 8, 8, 2, 2),
                                           (1, 32, 8, 1000, 1000), (1, 6, 3, 33, 40), (1, 16, 16, 300, 300),
                                           (1, 16, 2, 257, 321), (3, 32, 8, 300, 300), (4, 8, 2, 100, 164),
                                           (8, 32, 8, 64, 64)])
def test_prefill_against_oracle(gpu, prefill_form, HD, B, QH, KVH, T, S):
    from custom_kernels import custom_kernels_extension as cke
    from oracle import attention_prefill_ref

    print(f"prefill form={prefill_form} B={B} QH={QH} KVH={KVH} T={T} S={S} HD={HD}", flush=True)
    L = S + 7   # the cache is longer than what is attended
    q = randn_bf16((B, T, QH, HD), 61)
    kc = randn_bf16((B, L, KVH, HD), 62)
    vc = randn_bf16((B, L, KVH, HD), 63)
    out = cke.flash_attention_prefill(q.to(gpu).transpose(1, 2), kc.to(gpu)[:, :S].transpose(1, 2),
                                      vc.to(gpu)[:, :S].transpose(1, 2))
    torch.cuda.synchronize()
    assert out.shape == (B, QH, T, HD) and out.transpose(1, 2).is_contiguous()
    ref = attention_prefill_ref(t2f32(q.transpose(1, 2)), t2f32(kc[:, :S].transpose(1, 2)),
                                t2f32(vc[:, :S].transpose(1, 2)))
    assert_attn_close(out, ref, what=f"prefill T={T} S={S} HD={HD}")


@pytest.mark.parametrize("HD", [64, 128])
@pytest.mark.parametrize("gain", [3.0, 8.0])
def test_prefill_wide_score_range(gpu, prefill_form, HD, gain):
    """Scores spread over tens of powers of two (queries scaled up), and one key that dominates every
    query from token 700 on: the running maximum moves both by less and by more than the tiled kernel's
    2^8 rescaling slack, early and late in a row."""
    from custom_kernels import custom_kernels_extension as cke
    from oracle import attention_prefill_ref

    B, QH, KVH, T = 1, 8, 2, 900
    print(f"prefill wide range form={prefill_form} HD={HD} gain={gain}", flush=True)
    q = (randn_bf16((B, T, QH, HD), 91).float() * gain).to(torch.bfloat16)
    k = randn_bf16((B, T, KVH, HD), 92)
    v = randn_bf16((B, T, KVH, HD), 93)
    k[0, 700, 1] = (q[0, 800, 5].float() / gain * 2.0).to(torch.bfloat16)   # aligned with one query, large for all of its group
    out = cke.flash_attention_prefill(q.to(gpu).transpose(1, 2), k.to(gpu).transpose(1, 2), v.to(gpu).transpose(1, 2))
    torch.cuda.synchronize()
    ref = attention_prefill_ref(t2f32(q.transpose(1, 2)), t2f32(k.transpose(1, 2)), t2f32(v.transpose(1, 2)))
    assert_attn_close(out, ref, what=f"prefill wide range HD={HD} gain={gain}")


def test_prefill_forms_agree_on_a_long_prompt(gpu):
    """2048 tokens (the auto choice is the tiled form): the tiled and the wavefront-private form against
    each other, and sampled rows against the float64 oracle."""
    from custom_kernels import custom_kernels_extension as cke
    from oracle import attention_decode_ref

    B, QH, KVH, T, HD = 2, 32, 8, 2048, 128
    q = randn_bf16((B, T, QH, HD), 81)
    k = randn_bf16((B, T, KVH, HD), 82)
    v = randn_bf16((B, T, KVH, HD), 83)
    qd, kd, vd = (t.to(gpu).transpose(1, 2) for t in (q, k, v))
    outs = {}
    for name in ("auto", "wave", "tiled"):
        print(f"long prefill form={name}", flush=True)
        with cke.attention_flags(prefill=name):
            outs[name] = cke.flash_attention_prefill(qd, kd, vd).float().cpu()
    assert torch.equal(outs["auto"], outs["tiled"])
    assert (outs["wave"] - outs["tiled"]).abs().max().item() <= 2.0 ** -6
    for i in (0, 1, 63, 64, 65, 1000, 2047):
        ref = attention_decode_ref(t2f32(q[:, i:i + 1].transpose(1, 2)), t2f32(k[:, :i + 1].transpose(1, 2)),
                                   t2f32(v[:, :i + 1].transpose(1, 2)))
        assert_attn_close(outs["tiled"][:, :, i:i + 1], ref, what=f"long prefill row {i} (tiled)")
        assert_attn_close(outs["wave"][:, :, i:i + 1], ref, what=f"long prefill row {i} (wave)")


@pytest.mark.parametrize("HD", [64, 128])
@pytest.mark.parametrize("where", [(70,), (1500,), (2047,), (100, 900, 1800), (64, 65, 127, 128)])
def test_prefill_scores_that_outgrow_the_reference(gpu, HD, where):
    """A long prompt in which a few keys, past the first 64 tokens, each score some twenty nats above everything
    before them for the queries of their group: the tiles that take no maximum (forced here; the library turns
    to them only for large launches) have to notice, and go on with the maximum taken first from that tile
    on without losing what they had.  Wavefronts of one workgroup meet such a key at different tiles or not
    at all (queries before it never see it)."""
    from custom_kernels import custom_kernels_extension as cke
    from oracle import attention_prefill_ref

    B, QH, KVH, T = 1, 8, 2, 2048
    print(f"prefill outgrown reference HD={HD} where={where}", flush=True)
    q = randn_bf16((B, T, QH, HD), 94)
    k = randn_bf16((B, T, KVH, HD), 95)
    v = randn_bf16((B, T, KVH, HD), 96)
    unit = q[0, T - 1, 5].float() * (HD ** 0.5 / float((q[0, T - 1, 5].float() ** 2).sum()))   # scores 1 with that query
    for n, w in enumerate(where):
        k[0, w, 1] = (unit * 20.0 * (n + 1)).to(torch.bfloat16)
    ref = attention_prefill_ref(t2f32(q.transpose(1, 2)), t2f32(k.transpose(1, 2)), t2f32(v.transpose(1, 2)))
    outs = {}
    for form in ("tiled", "tiled-no-max"):
        with cke.attention_flags(prefill=form):
            outs[form] = cke.flash_attention_prefill(q.to(gpu).transpose(1, 2), k.to(gpu).transpose(1, 2),
                                                     v.to(gpu).transpose(1, 2))
        torch.cuda.synchronize()
        assert_attn_close(outs[form], ref, what=f"prefill outgrown reference HD={HD} where={where} {form}", regression=False)
        # the last query of head 5 puts nearly all its weight on the last of those keys
        assert np.abs(t2f32(outs[form])[0, 5, T - 1] - t2f32(v)[0, where[-1], 1]).max() < 0.05


@pytest.mark.parametrize("B,T,HD,gain", [(2, 2048, 64, 1.0), (1, 8192, 128, 1.0), (1, 8192, 64, 1.0),
                                         (1, 8192, 128, 3.0), (1, 8192, 64, 3.0)])
def test_prefill_timed_shapes_by_sampled_rows(gpu, B, T, HD, gain):
    """The prompt shapes the benchmark times, at their own size: rows either side of every kind of tile
    edge and the last rows against the float64 oracle, with unit-variance queries and with queries scaled
    so that a row's maximum keeps moving by more than the kernel's rescaling slack over 128 tiles.  With
    the scaled queries a few keys carry a row, and the head-size-128 kernel, which exponentiates against the
    previous tile's reference, rounds the dominant weight to bf16 (2^-9 relative) where a maximum-first
    kernel holds it as exactly 1: those rows are held to twice the regression bound's absolute part."""
    from custom_kernels import custom_kernels_extension as cke
    from oracle import attention_decode_ref

    QH, KVH = 32, 8
    print(f"prefill timed shape B={B} T={T} HD={HD} gain={gain}", flush=True)
    q = (randn_bf16((B, T, QH, HD), 84).float() * gain).to(torch.bfloat16)
    k = randn_bf16((B, T, KVH, HD), 85)
    v = randn_bf16((B, T, KVH, HD), 86)
    out = cke.flash_attention_prefill(q.to(gpu).transpose(1, 2), k.to(gpu).transpose(1, 2),
                                      v.to(gpu).transpose(1, 2)).float().cpu()
    rows = sorted({0, 15, 16, 63, 64, 65, 127, 128, 129, 255, 256, T // 2 - 1, T // 2, T // 2 + 1, T - 130,
                   T - 65, T - 64, T - 2, T - 1})
    for i in rows:
        ref = attention_decode_ref(t2f32(q[:, i:i + 1].transpose(1, 2)), t2f32(k[:, :i + 1].transpose(1, 2)),
                                   t2f32(v[:, :i + 1].transpose(1, 2)))
        what = f"prefill B={B} T={T} HD={HD} gain={gain} row {i}"
        assert_attn_close(out[:, :, i:i + 1], ref, what=what, min_kv_len=i + 1, regression=gain == 1.0)
        if gain != 1.0:
            err = np.abs(out[:, :, i:i + 1].numpy().astype(np.float64) - ref)
            bound = 2 * ATTN_REG_ATOL + (0.0 if i >= 63 else ATTN_REG_FEW_TOKENS) + ATTN_REG_RTOL * np.abs(ref)
            assert not (err > bound).any(), f"{what}: max err {err.max():.4g}, {(err > bound).sum()} outside the bound"


def test_prefill_last_row_equals_decode(gpu):
    from custom_kernels import custom_kernels_extension as cke

    B, QH, KVH, T, HD = 2, 32, 8, 96, 64
    q = randn_bf16((B, T, QH, HD), 71).to(gpu).transpose(1, 2)
    k = randn_bf16((B, T, KVH, HD), 72).to(gpu).transpose(1, 2)
    v = randn_bf16((B, T, KVH, HD), 73).to(gpu).transpose(1, 2)
    pre = cke.flash_attention_prefill(q, k, v)
    dec = cke.flash_attention_decode(q[:, :, T - 1:T], k, v)
    torch.cuda.synchronize()
    assert (pre[:, :, T - 1:T].float() - dec.float()).abs().max().item() <= 2.0 ** -7
    with pytest.raises(RuntimeError):
        cke.flash_attention_prefill(q, k[:, :, :10], v[:, :, :10])     # fewer cached tokens than queries
