"""GPU parity of decode attention in its single-launch form: the split kernel's cooperative workgroups
merge a (batch, kv head) themselves (the last one to arrive, out of its XCD's L2) instead of a combine
launch.  Against the float64 oracle, against the two-launch form on the same inputs, and for what the
scheme must leave behind: counters at zero and no head merged across XCDs."""

import math

import numpy as np
import pytest
import torch

from helpers import assert_attn_close, make_qkv, t2bits, t2f32
from oracle import attention_decode_ref

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def l3(gpu):
    from custom_kernels import _l3lib

    lib = _l3lib.load()
    ws = torch.empty(_l3lib.L3_ATTN_COUNTER_BYTES, dtype=torch.uint8, device=gpu)
    assert lib.l3_attn_workspace_init(ws.data_ptr(), ws.numel(), None) == 0
    torch.cuda.synchronize()
    if not lib.l3_attn_merge_in_launch_available():
        pytest.skip("the placement probe did not confirm round-robin XCD placement on this device")
    return _l3lib


class Caller:
    """l3_attn_decode through the C ABI on a workspace this test owns, so that its counters can be read."""

    def __init__(self, l3, gpu, nbytes=64 << 20):
        self.l3, self.lib = l3, l3.load()
        self.ws = torch.empty(nbytes, dtype=torch.uint8, device=gpu)
        assert self.lib.l3_attn_workspace_init(self.ws.data_ptr(), self.ws.numel(), None) == 0
        torch.cuda.synchronize()

    def __call__(self, q, k, v, splits=0, flags=0, kv_len=None):
        l3 = self.l3
        B, QH, _, HD = q.shape
        KVH, S = k.shape[1], k.shape[2]
        flags |= l3.L3_ATTN_FLAG_WS_COUNTERS
        need = self.lib.l3_attn_decode_workspace_bytes(B, QH, KVH, S, HD, splits, flags)
        assert need <= self.ws.numel()
        out = torch.empty_like(q)
        args = [q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), self.ws.data_ptr(), need, B, QH, KVH, S, HD,
                l3.i64_array((q.stride(0), q.stride(1))), l3.i64_array((k.stride(0), k.stride(1), k.stride(2))),
                l3.i64_array((v.stride(0), v.stride(1), v.stride(2))), l3.i64_array((out.stride(0), out.stride(1))),
                1.0 / math.sqrt(HD), splits, flags]
        if kv_len is None:
            rc = self.lib.l3_attn_decode(*args, None)
        else:
            rc = self.lib.l3_attn_decode_devlen(*args, kv_len.data_ptr(), None)
        assert rc == 0, rc
        torch.cuda.synchronize()
        return out

    def counters_are_zero(self):
        words = self.ws[: self.l3.L3_ATTN_COUNTER_BYTES].view(torch.int32)
        return int(words.count_nonzero().item()) == 0

    def placement_errors(self):
        return self.lib.l3_attn_placement_errors(self.ws.data_ptr())


@pytest.fixture(scope="module")
def call(l3, gpu):
    return Caller(l3, gpu)


@pytest.mark.parametrize("HD", [64, 128])
@pytest.mark.parametrize("QH,KVH,B", [(32, 8, 1), (8, 8, 2), (16, 8, 1), (24, 8, 1), (64, 8, 1), (16, 4, 2), (4, 2, 4),
                                       (32, 16, 3), (3, 1, 8)])
@pytest.mark.parametrize("S,splits", [(700, 2), (1000, 3), (1500, 8), (2100, 17), (4096, 32), (5000, 31)])
def test_forced_cooperative_splits_one_launch(l3, call, gpu, HD, QH, KVH, B, S, splits):
    """Every head ratio (1, 2, 3, 4, 8) with 2 ... 32 cooperative splits and ragged lengths; B x KVH is a
    multiple of 8 in every case, so the call must be a single launch.  Oracle, the two-launch form on the
    same plan (same float32 partials, merged by another kernel: at most the last bf16 bit may differ),
    counters back at zero, no head merged across XCDs."""
    COOP, TWO, W = l3.L3_ATTN_FLAG_FORM_COOP, l3.L3_ATTN_FLAG_TWO_LAUNCHES, l3.L3_ATTN_FLAG_WS_COUNTERS
    print(f"one launch: B={B} QH={QH} KVH={KVH} S={S} HD={HD} splits={splits}", flush=True)
    assert call.lib.l3_attn_launches(B, QH, KVH, S, HD, splits, COOP | W) == 1
    assert call.lib.l3_attn_launches(B, QH, KVH, S, HD, splits, COOP | W | TWO) == 2
    q, k, v = make_qkv(B, QH, KVH, S, HD, seed=S + splits)
    qg, kg, vg = make_qkv(B, QH, KVH, S, HD, seed=S + splits, device=gpu)
    one = call(qg, kg, vg, splits, COOP)
    assert call.counters_are_zero()
    two = call(qg, kg, vg, splits, COOP | TWO)
    ref = attention_decode_ref(t2f32(q), t2f32(k), t2f32(v))
    assert_attn_close(one, ref, what="one launch", min_kv_len=S)
    assert_attn_close(two, ref, what="two launches", min_kv_len=S)
    d = np.abs(t2f32(one).astype(np.float64) - t2f32(two).astype(np.float64))
    assert d.max() <= 2.0 ** -8 * max(1e-3, np.abs(ref).max())
    assert call.placement_errors() == 0


@pytest.mark.parametrize("HD", [64, 128])
def test_dominant_key_in_a_late_split_one_launch(l3, call, gpu, HD):
    """The merge inside the launch must weigh every split by its own statistics: one key far above the
    rest in the last of 8 splits takes all the weight (a merge that reused split 0's statistics, as
    custom_kernels.cu:184,201,209 does, would return the mean of the splits)."""
    S = 1500
    q, k, v = make_qkv(1, 32, 8, S, HD, seed=3)
    k[0, 1, S - 10] = q[0, 5, 0] * 4.0
    qg, kg, vg = make_qkv(1, 32, 8, S, HD, seed=3, device=gpu)
    kg[0, 1, S - 10] = qg[0, 5, 0] * 4.0
    out = call(qg, kg, vg, 8, l3.L3_ATTN_FLAG_FORM_COOP)
    assert_attn_close(out, attention_decode_ref(t2f32(q), t2f32(k), t2f32(v)), what="dominant key", min_kv_len=S)
    assert np.abs(t2f32(out)[0, 5, 0] - t2f32(v)[0, 1, S - 10]).max() < 0.05


def test_calls_of_different_shapes_share_one_workspace(l3, call, gpu):
    """The counters belong to the workspace, not to a shape: a sequence of calls with different batch
    sizes, head counts and split counts on one workspace, each checked against the oracle, and the same
    call twice in a row giving the same bits (nothing of the previous call is left in the counters)."""
    shapes = [(1, 32, 8, 4096, 128, 0), (4, 8, 2, 900, 64, 5), (1, 32, 8, 8192, 64, 0), (2, 32, 8, 700, 128, 3),
              (1, 32, 8, 4096, 128, 0), (8, 4, 1, 3000, 64, 9)]
    for i, (B, QH, KVH, S, HD, splits) in enumerate(shapes):
        print(f"shared workspace, call {i}: B={B} QH={QH} KVH={KVH} S={S} HD={HD} splits={splits}", flush=True)
        q, k, v = make_qkv(B, QH, KVH, S, HD, seed=100 + i)
        qg, kg, vg = make_qkv(B, QH, KVH, S, HD, seed=100 + i, device=gpu)
        flags = l3.L3_ATTN_FLAG_FORM_COOP if splits else 0
        a = call(qg, kg, vg, splits, flags)
        b = call(qg, kg, vg, splits, flags)
        np.testing.assert_array_equal(t2bits(a), t2bits(b))
        assert_attn_close(a, attention_decode_ref(t2f32(q), t2f32(k), t2f32(v)), what=f"call {i}", min_kv_len=S)
        assert call.counters_are_zero()
    assert call.placement_errors() == 0


@pytest.mark.parametrize("HD", [64, 128])
@pytest.mark.parametrize("length", [1, 100, 1023, 1024, 1025, 4000, 8192])
def test_device_side_length_one_launch(l3, call, gpu, HD, length):
    """The plan is made for the cache's full length; a shorter device-side length leaves the later splits
    without tokens.  They still count as arrivals (the counters must return to zero) and their rows are
    skipped by the merge."""
    B, QH, KVH, L = 1, 32, 8, 8192
    W = l3.L3_ATTN_FLAG_WS_COUNTERS
    assert call.lib.l3_attn_launches(B, QH, KVH, L, HD, 0, W) == 1
    q, k, v = make_qkv(B, QH, KVH, L, HD, seed=length)
    qg, kg, vg = make_qkv(B, QH, KVH, L, HD, seed=length, device=gpu)
    kv_len = torch.tensor([length], dtype=torch.int32, device=gpu)
    # poison the partial rows first: a merge that read a row of a split without tokens would show it
    call.ws[l3.L3_ATTN_COUNTER_BYTES:].view(torch.float32).fill_(float("nan"))
    out = call(qg, kg, vg, 0, 0, kv_len=kv_len)
    ref = attention_decode_ref(t2f32(q), t2f32(k[:, :, :length]), t2f32(v[:, :, :length]))
    assert_attn_close(out, ref, what=f"device-side length {length} of {L}", min_kv_len=length)
    assert call.counters_are_zero()


def test_grids_that_cannot_keep_a_head_on_one_xcd_take_two_launches(l3, call, gpu):
    """B x KVH not a multiple of 8, more than 32 splits, or a streamed plan: the library must fall back to
    split kernel + combine by itself, with the same flags and workspace."""
    COOP, ST, W = l3.L3_ATTN_FLAG_FORM_COOP, l3.L3_ATTN_FLAG_FORM_STREAM, l3.L3_ATTN_FLAG_WS_COUNTERS
    for (B, QH, KVH, S, HD, splits, form) in [(1, 12, 3, 1500, 64, 6, COOP), (1, 32, 8, 8192, 128, 40, COOP),
                                               (1, 32, 8, 4096, 128, 16, ST), (3, 8, 2, 2000, 128, 4, COOP)]:
        assert call.lib.l3_attn_launches(B, QH, KVH, S, HD, splits, form | W) == 2
        q, k, v = make_qkv(B, QH, KVH, S, HD, seed=S)
        qg, kg, vg = make_qkv(B, QH, KVH, S, HD, seed=S, device=gpu)
        out = call(qg, kg, vg, splits, form)
        assert_attn_close(out, attention_decode_ref(t2f32(q), t2f32(k), t2f32(v)), what="fallback", min_kv_len=S)
        assert call.counters_are_zero()


def test_one_launch_under_graph_replay(l3, call, gpu):
    """The single-launch form is what a captured decode step replays: every replay must leave the counters
    at zero for the next and reproduce the eager result, also with other work between replays."""
    B, QH, KVH, S, HD = 1, 32, 8, 4096, 128
    qg, kg, vg = make_qkv(B, QH, KVH, S, HD, seed=8, device=gpu)
    eager = call(qg, kg, vg)
    lib, W = call.lib, l3.L3_ATTN_FLAG_WS_COUNTERS
    need = lib.l3_attn_decode_workspace_bytes(B, QH, KVH, S, HD, 0, W)
    out = torch.empty_like(qg)
    stream = torch.cuda.Stream()
    args = [qg.data_ptr(), kg.data_ptr(), vg.data_ptr(), out.data_ptr(), call.ws.data_ptr(), need, B, QH, KVH, S, HD,
            l3.i64_array((qg.stride(0), qg.stride(1))), l3.i64_array((kg.stride(0), kg.stride(1), kg.stride(2))),
            l3.i64_array((vg.stride(0), vg.stride(1), vg.stride(2))), l3.i64_array((out.stride(0), out.stride(1))),
            1.0 / math.sqrt(HD), 0, W]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for _ in range(3):
            assert lib.l3_attn_decode(*args, torch.cuda.current_stream().cuda_stream) == 0
    for _ in range(4):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(t2bits(out), t2bits(eager))
        assert call.counters_are_zero()
        call(qg, kg, vg, 5, l3.L3_ATTN_FLAG_FORM_COOP)   # eager work on the same workspace between replays
    assert call.placement_errors() == 0


def test_calls_on_two_streams_at_once(l3, gpu):
    """Two callers with their own workspaces on two streams, long enough kernels (256 workgroups each, 15 and
    25 us) and deep enough queues that their launches overlap on the device, and matrix products on a third
    stream: the placement of a grid's workgroups on the XCDs must not depend on what else is being dispatched.
    Every call must reproduce the bits of the same call made alone, leave its counters at zero and report no
    head whose arrivals came from several XCDs."""
    lib = l3.load()
    W = l3.L3_ATTN_FLAG_WS_COUNTERS

    class StreamCaller:
        def __init__(self, S, seed):
            B, QH, KVH, HD = 1, 32, 8, 128
            self.stream = torch.cuda.Stream()
            self.q, self.k, self.v = make_qkv(B, QH, KVH, S, HD, seed=seed, device=gpu)
            self.ws = torch.empty(32 << 20, dtype=torch.uint8, device=gpu)
            assert lib.l3_attn_workspace_init(self.ws.data_ptr(), self.ws.numel(), self.stream.cuda_stream) == 0
            torch.cuda.synchronize()
            self.out = torch.empty_like(self.q)
            self.bad = torch.zeros(1, dtype=torch.int64, device=gpu)
            q, k, v, out = self.q, self.k, self.v, self.out
            self.args = [q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), self.ws.data_ptr(), self.ws.numel(), B, QH, KVH,
                         S, HD, l3.i64_array((q.stride(0), q.stride(1))), l3.i64_array((k.stride(0), k.stride(1), k.stride(2))),
                         l3.i64_array((v.stride(0), v.stride(1), v.stride(2))), l3.i64_array((out.stride(0), out.stride(1))),
                         1.0 / math.sqrt(HD), 0, W]
            assert lib.l3_attn_launches(B, QH, KVH, S, HD, 0, W) == 1
            self.call()
            torch.cuda.synchronize()
            self.alone = self.out.clone()

        def call(self):
            assert lib.l3_attn_decode(*self.args, self.stream.cuda_stream) == 0

        def check(self):
            with torch.cuda.stream(self.stream):
                self.bad += (self.out.view(torch.int16) != self.alone.view(torch.int16)).sum()
                self.out.zero_()

    a, b = StreamCaller(32768, 31), StreamCaller(16384, 32)
    side = torch.cuda.Stream()
    x = torch.randn(2048, 2048, device=gpu, dtype=torch.bfloat16)
    for it in range(150):
        for c in (a, b):
            for _ in range(4):
                c.call()
            c.check()
        if it % 3 == 0:
            with torch.cuda.stream(side):
                _ = x @ x
    torch.cuda.synchronize()
    for c in (a, b):
        assert int(c.bad.item()) == 0
        assert int(c.ws[: l3.L3_ATTN_COUNTER_BYTES - 128].view(torch.int32).count_nonzero().item()) == 0
        assert lib.l3_attn_placement_errors(c.ws.data_ptr()) == 0
