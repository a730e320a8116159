#!/usr/bin/env python3
"""Benchmark of the custom-kernel hot path on one MI355X.

Default workload (the headline configuration): decode attention at head_dim 128, batch 1,
32 query / 8 KV heads, bf16, KV length swept over every power of two from 512 to 32768.
One step = one pass over the seven lengths (split-KV kernel + combine each).  Inputs are
resident in HBM before the timed region.  Every launch reads K/V from its own region of a 2 GiB
pool, and a region is read again only after at least 512 MB of other regions have been read,
so the 256 MB Infinity Cache cannot serve any of it: every figure is HBM-cold.  The
launches are captured in a HIP graph (launch-bound otherwise) and replayed -- at least 30 ms
untimed, then at least 50 ms timed, whatever --steps says; the clock is wall time around the
replays with a device synchronisation on both sides.

Prints ONE JSON line: value = algorithmic GB/s (K+V+Q read, O written) over the timed steps;
"roofline" prices the split-KV kernel alone against the 8 TB/s HBM peak from HIP-event timing and
carries the read bandwidth a pure stream reaches on the same device; "cpu_baseline" is stock
PyTorch on the host cores for a bounded sample of the same sweep.  The same line carries the rest
of the target ("north_star": head_dim 64, the batched shapes, longer KV lengths, RMSNorm, rotary
embedding, each cold; beside every attention shape torch's own attention on the same GPU and the
time a kernel that only reads takes for the same bytes), the causal prefill kernel on three prompt
shapes against the MFMA peak ("prefill") and the end-to-end tokens/s ("e2e").

Other workloads (--workload c1|c3a|c3b|hd64|rms|rope|prefill|linear|e2e|copy|readstream) report the
remaining configurations in the same format.
"""

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "llama3-custom-inference_amd")
for _p in (ROOT, PKG):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E peak
SEED = 42               # the reference's default seed (benchmark_kernel.py:126)
FORCE_SPLITS = 0        # --splits
ATTN_FLAGS = 0          # --attn-kernel fma sets L3_ATTN_FLAG_KERNEL_FMA
COLD_BYTES = 512 << 20  # distinct input bytes between two reads of the same region (Infinity Cache: 256 MB)
MIN_WARM_S = 0.03       # untimed replays: after an idle spell the first milliseconds run at lower clocks
MIN_TIMED_S = 0.05


# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this file (the summaries, their commands and the copy-kernel calibration are under profiles/).
# An entry is reported only while the split plan it was measured with is the plan of this run.
MEASURED_TRAFFIC = {
    "c2": {"bytes": 39150000, "plan": [8, 16, 32, 32, 32, 32, 32], "flags": 2,
           "profile": "profiles/attn_splitkv_mfma_c2_sweep_hbm_traffic.md"},
    "c3a": {"flags": 2, "bytes": 136660000, "plan": [1], "profile": "profiles/hbm_traffic_batched_attention_rms_norm_rot_embed.md"},
    "c3b": {"flags": 2, "bytes": 135870000, "plan": [11], "profile": "profiles/hbm_traffic_batched_attention_rms_norm_rot_embed.md"},
    "rms": {"flags": 2, "bytes": 67250000, "plan": None, "profile": "profiles/hbm_traffic_batched_attention_rms_norm_rot_embed.md"},
    "rope": {"flags": 2, "bytes": 68200000, "plan": None, "profile": "profiles/hbm_traffic_batched_attention_rms_norm_rot_embed.md"},
}


def measured_traffic(name, plan=None):
    rec = MEASURED_TRAFFIC.get(name)
    if rec is None or (ATTN_FLAGS & ~rec.get("flags", 0)) or FORCE_SPLITS or (rec["plan"] is not None and rec["plan"] != plan):
        return None, None
    return rec["bytes"], rec["profile"]


def attn_kernel_name():
    from custom_kernels import _l3lib as l3
    return "fma" if ATTN_FLAGS & l3.L3_ATTN_FLAG_KERNEL_FMA else "mfma"


def attn_bytes(B, QH, KVH, S, HD):
    """K+V+Q read, O written, bf16 (the reference counts K+V only: benchmark_kernel.py:48)."""
    return 2 * B * KVH * S * HD * 2 + 2 * B * QH * HD * 2


class KVPool:
    """2 GiB of N(0,1) bf16 (1 GiB for K, 1 GiB for V) that every attention shape carves its
    rotating input copies from.  `regions` hands out disjoint (B, L, KVH, HD) caches; a launch that
    walks over them reads each byte once per walk."""

    def __init__(self, torch, dev, elems=1 << 29):
        self.torch = torch
        self.k = torch.empty(elems, dtype=torch.bfloat16, device=dev).normal_()
        self.v = torch.empty(elems, dtype=torch.bfloat16, device=dev).normal_()
        self.next = 0

    def reset(self):
        self.next = 0

    def region(self, B, L, KVH, HD):
        per = B * L * KVH * HD
        if self.next + per > self.k.numel():
            raise RuntimeError("KV pool exhausted")
        k = self.k[self.next:self.next + per].view(B, L, KVH, HD)
        v = self.v[self.next:self.next + per].view(B, L, KVH, HD)
        self.next += per
        return k, v

    def capacity(self, B, L, KVH, HD):
        return (self.k.numel() - self.next) // (B * L * KVH * HD)


class AttnCase:
    """One attention shape with `slots` disjoint copies of its K/V (token-major storage, transposed
    views: the model's cache layout, benchmark_kernel.py:165-173), a pre-allocated output and
    workspace, launched straight through the C ABI (no per-call allocation)."""

    def __init__(self, torch, lib, l3, dev, pool, B, QH, KVH, S, HD, slots, cache_len=0, splits=None, flags=None):
        self.torch, self.lib = torch, lib
        splits = FORCE_SPLITS if splits is None else splits
        flags = ATTN_FLAGS if flags is None else flags
        self.flags = flags
        self.B, self.QH, self.KVH, self.S, self.HD = B, QH, KVH, S, HD
        self.bytes = attn_bytes(B, QH, KVH, S, HD)
        L = max(S, cache_len)
        self.slots = max(1, min(slots, pool.capacity(B, L, KVH, HD)))
        g = torch.Generator().manual_seed(SEED)
        self.q = torch.randn((B, 1, QH, HD), generator=g).to(torch.bfloat16).to(dev).transpose(1, 2)
        self.k, self.v = [], []
        for _ in range(self.slots):
            kc, vc = pool.region(B, L, KVH, HD)
            # the model's layout (model.py:107-111): a (B, L, KVH, HD) cache of which the first S tokens are attended
            self.k.append(kc[:, :S].transpose(1, 2))
            self.v.append(vc[:, :S].transpose(1, 2))
        self.out = torch.empty_like(self.q)
        # 0 = the library plans for the current device (split count and kernel form)
        self.req_splits = splits
        self.num_splits = splits or lib.l3_attn_choose_splits(B, KVH, S, HD, 0, flags)
        self.ws_bytes = lib.l3_attn_decode_workspace_bytes(B, QH, KVH, S, HD, self.req_splits, flags)
        self.ws = torch.empty(max(self.ws_bytes, l3.L3_ATTN_COUNTER_BYTES), dtype=torch.uint8, device=dev)
        if flags & l3.L3_ATTN_FLAG_WS_COUNTERS:
            # the workspace starts with the arrival counters of the single-launch form (zeroed once, here)
            rc = lib.l3_attn_workspace_init(self.ws.data_ptr(), self.ws.numel(), torch.cuda.current_stream().cuda_stream)
            if rc != 0:
                raise RuntimeError(f"l3_attn_workspace_init failed: {rc}")
            torch.cuda.synchronize()
        self.part_o = self.part_ml = None
        qt, ot = self.q, self.out
        self._args = []
        for kt, vt in zip(self.k, self.v):
            self._args.append((
                qt.data_ptr(), kt.data_ptr(), vt.data_ptr(), ot.data_ptr(), self.ws.data_ptr(), self.ws_bytes,
                B, QH, KVH, S, HD,
                l3.i64_array((qt.stride(0), qt.stride(1))), l3.i64_array((kt.stride(0), kt.stride(1), kt.stride(2))),
                l3.i64_array((vt.stride(0), vt.stride(1), vt.stride(2))), l3.i64_array((ot.stride(0), ot.stride(1))),
                1.0 / math.sqrt(HD), self.req_splits, flags))

    def launch(self, slot, stream_ptr):
        rc = self.lib.l3_attn_decode(*self._args[slot % self.slots], stream_ptr)
        if rc != 0:
            raise RuntimeError(f"l3_attn_decode failed: {rc}")

    def launch_split_stage(self, slot, stream_ptr):
        """The split-KV kernel alone (l3_attn_split), for pricing it against the roofline."""
        a = self._args[slot % self.slots]
        if self.part_o is None:
            n = max(self.num_splits, 1)
            self.part_o = self.torch.empty((self.B, self.QH, n, self.HD), dtype=self.torch.float32, device=self.ws.device)
            self.part_ml = self.torch.empty((self.B, self.QH, n, 2), dtype=self.torch.float32, device=self.ws.device)
        rc = self.lib.l3_attn_split(a[0], a[1], a[2], self.part_o.data_ptr(), self.part_ml.data_ptr(),
                                    self.B, self.QH, self.KVH, self.S, self.HD, a[11], a[12], a[13], a[15],
                                    self.req_splits, self.flags, stream_ptr)
        if rc < 0:
            raise RuntimeError(f"l3_attn_split failed: {rc}")


def cold_slots(call_bytes, floor=4, cap=1024):
    """Copies of a shape's inputs needed so that COLD_BYTES of other data pass between two reads of one copy
    (at most `cap`: a call of a few KB is bound by latency, not by where its bytes come from)."""
    return min(cap, max(floor, int(math.ceil(COLD_BYTES / call_bytes)) + 1))


def capture_graph(torch, fn):
    """Capture fn() (which launches on torch's current stream) into a HIP graph."""
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        fn()  # warm-up outside capture (module load, allocator)
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
    return graph


def event_time_ms(torch, run, reps):
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        run()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / reps


def timed_replays(torch, graph, min_replays=1, wall=False):
    """Replays `graph` untimed for MIN_WARM_S, then timed for at least MIN_TIMED_S (and at least
    min_replays times).  Returns (milliseconds per replay, replays timed).  HIP events on the
    stream the graph runs on, or -- wall=True -- the host clock with a device synchronisation on
    both sides."""
    t0 = time.perf_counter()
    n_warm = 0
    while time.perf_counter() - t0 < MIN_WARM_S or n_warm < 2:
        graph.replay()
        torch.cuda.synchronize()
        n_warm += 1
    est = event_time_ms(torch, graph.replay, 2)
    reps = max(min_replays, int(math.ceil(MIN_TIMED_S * 1e3 / max(est, 1e-4))))
    if not wall:
        return event_time_ms(torch, graph.replay, reps), reps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        graph.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / reps, reps


def time_cpu(fn, min_seconds, min_reps=3, max_reps=100000):
    fn()
    t0 = time.perf_counter()
    n = 0
    while True:
        fn()
        n += 1
        el = time.perf_counter() - t0
        if (el >= min_seconds and n >= min_reps) or n >= max_reps:
            return el / n, n


def torch_sdpa_us(torch, case, max_calls=24):
    """torch's own scaled_dot_product_attention (enable_gqa) on the same cold tensors on the same GPU,
    eager calls timed with events: what the reference's benchmark plots beside its kernel
    (benchmark_kernel.py:23-28, 110-115).  A reported baseline only."""
    import torch.nn.functional as F

    try:
        n = min(case.slots, max_calls)
        for i in range(min(2, n)):
            F.scaled_dot_product_attention(case.q, case.k[-1 - i], case.v[-1 - i], enable_gqa=True)
        idx = [0]

        def one():
            i = idx[0] % n
            idx[0] += 1
            F.scaled_dot_product_attention(case.q, case.k[i], case.v[i], enable_gqa=True)
        return round(event_time_ms(torch, one, n) * 1e3, 2)
    except Exception as exc:  # informational only
        print(f"bench.py: torch SDPA failed for B{case.B} S{case.S} HD{case.HD}: {exc}", file=sys.stderr)
        return None


def measure_attention_shape(torch, lib, l3, dev, pool, B, QH, KVH, S, HD, cache_len=0, with_sdpa=True,
                            split_stage=False):
    """One shape alone, HBM-cold: a graph that walks over the shape's copies, replayed."""
    pool.reset()
    c = AttnCase(torch, lib, l3, dev, pool, B, QH, KVH, S, HD, cold_slots(attn_bytes(B, QH, KVH, S, HD)), cache_len)
    launch = c.launch_split_stage if split_stage else c.launch
    launch(0, torch.cuda.current_stream().cuda_stream)
    gph = capture_graph(torch, lambda: [launch(s, torch.cuda.current_stream().cuda_stream) for s in range(c.slots)])
    ms, reps = timed_replays(torch, gph)
    ms /= c.slots
    del gph
    gbps = c.bytes / (ms * 1e-3) / 1e9
    rec = {"B": B, "HD": HD, "kv_len": S, "splits": c.num_splits, "us": round(ms * 1e3, 3), "GBps": round(gbps, 1),
           "frac": round(gbps / HBM_PEAK_GBPS, 4), "bytes": c.bytes, "copies": c.slots,
           "cold": bool(c.bytes * (c.slots - 1) >= COLD_BYTES), "launches_timed": reps * c.slots}
    if not split_stage and c.num_splits > 1:
        # the split-KV kernel of the same calls alone: the difference is what the combine launch costs
        c.launch_split_stage(0, torch.cuda.current_stream().cuda_stream)
        sg = capture_graph(torch, lambda: [c.launch_split_stage(s, torch.cuda.current_stream().cuda_stream)
                                           for s in range(c.slots)])
        rec["split_kernel_us"] = round(timed_replays(torch, sg)[0] / c.slots * 1e3, 3)
        del sg
    if with_sdpa:
        rec["torch_sdpa_us"] = torch_sdpa_us(torch, c)
    if not split_stage:
        # what a kernel that only reads takes for the same number of bytes, cold, launched the same way
        rec["read_stream_us"] = measure_read_stream(torch, lib, dev, pool, (c.bytes + 255) // 256 * 256)["us"]
    return rec


def measure_read_stream(torch, lib, dev, pool, chunk_bytes=128 << 20):
    """The read bandwidth a pure stream reaches: the library's read-only kernel over the K pool in
    chunks of chunk_bytes, each chunk cold, graph-replayed like everything else."""
    src = pool.k
    total = src.numel() * 2
    n = max(1, total // chunk_bytes)
    sink = torch.zeros(16, dtype=torch.int32, device=dev)

    def walk():
        sp = torch.cuda.current_stream().cuda_stream
        for i in range(n):
            rc = lib.l3_hbm_read_stream(src.data_ptr() + i * chunk_bytes, chunk_bytes, sink.data_ptr(), 0, sp)
            if rc != 0:
                raise RuntimeError(f"l3_hbm_read_stream failed: {rc}")
    walk()
    gph = capture_graph(torch, walk)
    ms, reps = timed_replays(torch, gph)
    ms /= n
    gbps = chunk_bytes / (ms * 1e-3) / 1e9
    return {"bytes_per_launch": chunk_bytes, "us": round(ms * 1e3, 3), "GBps": round(gbps, 1),
            "frac": round(gbps / HBM_PEAK_GBPS, 4), "launches_timed": reps * n,
            "kernel": "hbm_read_stream_kernel (16-byte non-temporal loads, no stores, no arithmetic)"}


def weights_read_floor_us(torch, lib, dev):
    """What a decode step of the 1B architecture would take if it did nothing but read its weights: the
    read-only kernel launched once per linear kernel of the step, on that kernel's weight bytes (qkv, output
    projection, gate|up pair, down projection per layer, then the vocabulary projection), each region its own
    part of a 2.5 GB buffer, so that a replay finds every byte as cold as the real step finds its weights."""
    C, FF, V, LAYERS, KV = 2048, 8192, 128256, 16, 512
    sizes = [((C + 2 * KV) * C * 2), C * C * 2, 2 * FF * C * 2, C * FF * 2] * LAYERS + [V * C * 2]
    offsets, total = [], 0
    for n in sizes:
        offsets.append(total)
        total += (n + 4095) // 4096 * 4096
    buf = torch.empty(total, dtype=torch.uint8, device=dev)
    buf.random_(0, 255)
    sink = torch.zeros(16, dtype=torch.int32, device=dev)

    def walk():
        sp = torch.cuda.current_stream().cuda_stream
        for off, n in zip(offsets, sizes):
            rc = lib.l3_hbm_read_stream(buf.data_ptr() + off, n, sink.data_ptr(), 0, sp)
            if rc != 0:
                raise RuntimeError(f"l3_hbm_read_stream failed: {rc}")
    walk()
    gph = capture_graph(torch, walk)
    ms, _ = timed_replays(torch, gph)
    del gph, buf
    torch.cuda.empty_cache()
    return round(ms * 1e3, 1), len(sizes), sum(sizes)


def measure_rw_stream(torch, lib, dev, nbytes):
    """The read + write yardstick: the library's copy-through kernel (16-byte non-temporal loads, plain 16-byte
    stores) over cold source / destination pairs of `nbytes` each, graph-replayed: what a row-wise operator
    that reads and writes every element once can reach."""
    nbytes = (nbytes + 255) // 256 * 256
    copies = cold_slots(2 * nbytes, floor=2)
    src = [torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(i & 0xff) for i in range(copies)]
    dst = [torch.empty(nbytes, dtype=torch.uint8, device=dev) for _ in range(copies)]

    best = None
    for block_kib in (8, 16, 32, 64):   # which is fastest depends on how the buffer divides over the compute units
        def walk():
            sp = torch.cuda.current_stream().cuda_stream
            for a, b in zip(src, dst):
                rc = lib.l3_hbm_rw_stream(a.data_ptr(), b.data_ptr(), nbytes, 0, block_kib, sp)
                if rc != 0:
                    raise RuntimeError(f"l3_hbm_rw_stream failed: {rc}")
        walk()
        gph = capture_graph(torch, walk)
        ms, reps = timed_replays(torch, gph)
        del gph
        if best is None or ms < best[0]:
            best = (ms, reps, block_kib)
    ms, reps, block_kib = best
    ms /= copies
    gbps = 2 * nbytes / (ms * 1e-3) / 1e9
    return {"bytes_read_and_written": 2 * nbytes, "us": round(ms * 1e3, 3), "GBps": round(gbps, 1),
            "frac": round(gbps / HBM_PEAK_GBPS, 4), "launches_timed": reps * copies, "block_KiB": block_kib}


ATTN_WORKLOADS = {
    # name: (B, HD, KV lengths, label)
    "c2": (1, 128, [512, 1024, 2048, 4096, 8192, 16384, 32768],
           "decode attention sweep: B1 QH32 KVH8 HD128 bf16, KV length 512..32768 (x2), split+combine"),
    "c1": (1, 64, [256], "decode attention: B1 QH32 KVH8 HD64 bf16, KV length 256, split+combine"),
    "c3a": (256, 64, [256], "batched decode attention: B256 QH32 KVH8 HD64 bf16, KV length 256"),
    "c3b": (16, 64, [4096], "batched decode attention: B16 QH32 KVH8 HD64 bf16, KV length 4096, split+combine"),
    "hd64": (1, 64, [512, 1024, 2048, 4096, 8192, 16384, 32768],
             "decode attention sweep: B1 QH32 KVH8 HD64 bf16, KV length 512..32768 (x2), split+combine"),
}


# ------------------------------------------------------------------------------ workloads
def run_attention(args, torch, lib, l3, dev, name, pool):
    from oracle.cpu_baseline import attention_cpu

    QH, KVH = 32, 8
    B, HD, lengths, label = ATTN_WORKLOADS[name]
    if args.lengths:
        lengths = [int(x) for x in args.lengths.split(",")]
        label += f" [lengths overridden: {lengths}]"
    if args.cache_len:
        label += f" [K/V are views of (B, {args.cache_len}, KVH, HD) caches]"
    pass_bytes = sum(attn_bytes(B, QH, KVH, S, HD) for S in lengths)
    # a pass reads every length once, each from its own region; enough passes per graph that
    # COLD_BYTES of other regions separate two reads of one region
    passes = cold_slots(pass_bytes)
    pool.reset()
    cases = [AttnCase(torch, lib, l3, dev, pool, B, QH, KVH, S, HD, passes, args.cache_len) for S in lengths]
    passes = min(c.slots for c in cases)

    def one_pass(slot):
        sp = torch.cuda.current_stream().cuda_stream
        for c in cases:
            c.launch(slot, sp)

    if args.single_shot:
        # one eager call per length on cold copies, for use under a profiler (the reference's
        # --use_ncu mode, benchmark_kernel.py:175-176); no graph, no repetition
        one_pass(0)
        torch.cuda.synchronize()
        detail = []
        for c in cases:
            ms = event_time_ms(torch, lambda c=c: c.launch(1, torch.cuda.current_stream().cuda_stream), 1)
            detail.append({"kv_len": c.S, "splits": c.num_splits, "us": round(ms * 1e3, 3),
                           "GBps": round(c.bytes / ms / 1e6, 1)})
        total_ms = sum(d["us"] for d in detail) / 1e3
        return {
            "metric": "decode_attn_hbm_GBps", "value": round(pass_bytes / total_ms / 1e6, 1), "unit": "GB/s",
            "steps": 1, "ms_per_step": round(total_ms, 5), "dtype": "bf16",
            "config": {"workload": label + " [single shot: one eager call per length, launch latency included]",
                       "seed": SEED},
            "roofline": None, "cpu_baseline": None, "per_length": detail,
        }

    one_pass(0)
    # The headline: exactly args.steps passes, wall clock with a device synchronisation on both sides, after at
    # least args.warmup passes and MIN_WARM_S untimed.  The passes are recorded in HIP graphs (launch-bound
    # otherwise): a main graph of a whole number of rotations over the K/V copies, replayed, plus one shorter
    # graph for the remainder, so that the copies keep their order across replays.
    g_passes = passes * max(1, min(args.steps, 512) // passes) if args.steps >= passes else 0
    n_main = args.steps // g_passes if g_passes else 0
    rem = args.steps - n_main * g_passes
    main_graph = capture_graph(torch, lambda: [one_pass(s) for s in range(g_passes)]) if g_passes else None
    rem_graph = capture_graph(torch, lambda: [one_pass(n_main * g_passes + s) for s in range(rem)]) if rem else None

    def timed_region():
        for _ in range(n_main):
            main_graph.replay()
        if rem_graph is not None:
            rem_graph.replay()

    t_warm, warmed = time.perf_counter(), 0
    while time.perf_counter() - t_warm < MIN_WARM_S or warmed < args.warmup:
        timed_region()
        torch.cuda.synchronize()
        warmed += args.steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    timed_region()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    steps = args.steps
    ms_per_step = wall_ms / steps
    value = pass_bytes / (ms_per_step * 1e-3) / 1e9
    # HIP-event timing of the same launches (events on the stream the kernels run on), over at least MIN_TIMED_S
    ev_reps = max(1, int(math.ceil(MIN_TIMED_S * 1e3 / max(wall_ms, 1e-3))))
    ev_ms = event_time_ms(torch, timed_region, ev_reps) / steps
    op_gbps = pass_bytes / (ev_ms * 1e-3) / 1e9
    del main_graph, rem_graph

    # The dominant kernel on its own.  Where every length of the sweep runs as ONE launch (the split kernel
    # merges its partials itself) that kernel is the whole call, timed above; otherwise the split-KV stage of
    # every length (l3_attn_split: the same kernel writing partials only), same regions, graph-replayed.
    plan = [c.num_splits for c in cases]
    single_launch = [bool(lib.l3_attn_launches(B, QH, KVH, c.S, HD, c.req_splits, c.flags) == 1) for c in cases]

    def split_pass(slot):
        sp = torch.cuda.current_stream().cuda_stream
        for c in cases:
            c.launch_split_stage(slot, sp)

    split_pass(0)
    sgraph = capture_graph(torch, lambda: [split_pass(s) for s in range(passes)])
    sms, sreps = timed_replays(torch, sgraph)
    split_ms = sms / passes
    del sgraph
    kernel_ms = ev_ms if all(single_launch) else split_ms
    achieved = pass_bytes / (kernel_ms * 1e-3) / 1e9
    split_kernel = "attn_splitkv_mfma_kernel" if attn_kernel_name() == "mfma" else "attn_splitkv_fma_kernel"
    traffic, traffic_src = measured_traffic(name, plan)
    del cases

    # per-length detail: each length alone over its own cold copies, with torch's attention beside it
    detail = [measure_attention_shape(torch, lib, l3, dev, pool, B, QH, KVH, S, HD, args.cache_len,
                                      with_sdpa=not args.no_sdpa) for S in lengths]

    cpu = None
    if not args.no_cpu_baseline and name in ("c2", "c1"):
        g = torch.Generator().manual_seed(SEED)
        smax = max(lengths)
        q = torch.randn((B, 1, QH, HD), generator=g).to(torch.bfloat16).transpose(1, 2)
        k = torch.randn((B, smax, KVH, HD), generator=g).to(torch.bfloat16)
        v = torch.randn((B, smax, KVH, HD), generator=g).to(torch.bfloat16)

        def cpu_pass():
            for S in lengths:
                attention_cpu(q, k[:, :S].transpose(1, 2), v[:, :S].transpose(1, 2))
        sec, n = time_cpu(cpu_pass, args.cpu_seconds)
        cpu = {"value": round(pass_bytes / sec / 1e9, 2), "unit": "GB/s", "cores": torch.get_num_threads(),
               "kind": "port", "host_cpus": os.cpu_count(),
               "sample": f"{n} passes of the same sweep with torch CPU scaled_dot_product_attention "
                         f"(bf16, enable_gqa) in {sec * n:.1f} s"}

    return {
        "metric": "decode_attn_hbm_GBps", "value": round(value, 1), "unit": "GB/s",
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "steps": steps, "ms_per_step": round(ms_per_step, 5), "dtype": "bf16",
        "config": {"workload": label, "kv_regions_per_length": passes, "cold_bytes_between_reuse": COLD_BYTES,
                   "accumulate": "f32", "launch": "hip graph", "seed": SEED,
                   "timed_region_s": round(wall_ms / 1e3, 5)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_profile": traffic_src,
                     "kernel": split_kernel, "launches_per_pass": len(lengths), "split_plan": plan,
                     "single_launch": single_launch,
                     "timed_as": ("the whole call (one launch per length: the kernel merges its partials itself)"
                                  if all(single_launch) else "the split stage alone (l3_attn_split)"),
                     "avg_launch_us": round(kernel_ms * 1e3 / len(lengths), 3),
                     "launches_timed": (ev_reps * steps if all(single_launch) else sreps * passes) * len(lengths),
                     "algorithmic_bytes_per_launch": pass_bytes // len(lengths),
                     "split_stage_only_avg_us": round(split_ms * 1e3 / len(lengths), 3),
                     # the same quotient for the split stage alone (partials written, nothing merged): what this key
                     # measured while the merge was a launch of its own
                     "split_stage_only_frac": round(pass_bytes / (split_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                     "whole_call_GBps": round(op_gbps, 1),
                     "whole_call_frac": round(op_gbps / HBM_PEAK_GBPS, 4)},
        "cpu_baseline": cpu, "per_length": detail,
    }


def north_star_extras(args, torch, lib, l3, dev, pool):
    """The rest of the target beside the headline sweep, every entry HBM-cold: head_dim 64 at batch 1,
    the batched shapes (split + combine together), RMSNorm and rotary embedding at 4096 rows."""
    QH, KVH = 32, 8
    sdpa = not args.no_sdpa
    out = {"hd64_b1": [measure_attention_shape(torch, lib, l3, dev, pool, 1, QH, KVH, S, 64, with_sdpa=sdpa)
                       for S in (4096, 8192, 16384, 32768)],
           "c1_b1_hd64_s256": measure_attention_shape(torch, lib, l3, dev, pool, 1, QH, KVH, 256, 64, with_sdpa=sdpa),
           "c3a_b256_hd64_s256": measure_attention_shape(torch, lib, l3, dev, pool, 256, QH, KVH, 256, 64, with_sdpa=sdpa),
           "c3b_b16_hd64_s4096": measure_attention_shape(torch, lib, l3, dev, pool, 16, QH, KVH, 4096, 64, with_sdpa=sdpa)}
    # beyond the configured sweep: where batch 1 crosses the target as the stream grows against the fixed
    # cost of two launches
    out["longer_kv_b1"] = [measure_attention_shape(torch, lib, l3, dev, pool, 1, QH, KVH, S, HD, with_sdpa=sdpa)
                           for HD in (128, 64) for S in (65536, 131072)]
    out["rms_norm"] = [rows_record(torch, lib, l3, dev, "rms", 2, 2048, C) for C in (2048, 4096)]
    out["rot_embed"] = [rows_record(torch, lib, l3, dev, "rope", 2, 2048, HD) for HD in (64, 128)]
    return out


def rows_record(torch, lib, l3, dev, name, B, T, width):
    """One RMSNorm (width = C) or rotary-embedding (width = HD, 32 heads of a strided qkv view) shape,
    cold: enough copies of input and output that COLD_BYTES pass between two uses of one copy."""
    from custom_kernels import precompute_freqs_cis

    g = torch.Generator().manual_seed(SEED)
    sp = lambda: torch.cuda.current_stream().cuda_stream  # noqa: E731
    if name == "rms":
        C = width
        nbytes = 2 * B * T * C * 2 + C * 2
        copies = cold_slots(nbytes, floor=2)
        # drawn on the device: the values do not matter, and no large host buffer has to cross the bus
        x0 = torch.empty((B, T, C), dtype=torch.bfloat16, device=dev).normal_()
        xs = [x0] + [torch.empty_like(x0).normal_() for _ in range(copies - 1)]
        w = (torch.randn((C,), generator=g) * 0.02 + 1).to(torch.bfloat16).to(dev)
        ys = [torch.empty_like(x) for x in xs]
        run = lambda: [lib.l3_rms_norm(x.data_ptr(), w.data_ptr(), y.data_ptr(), B * T, C, 1e-5, sp())  # noqa: E731
                       for x, y in zip(xs, ys)]
        rec = {"rows": B * T, "C": C}
        keep = (x0, w)
    else:
        HD, NH = width, 32
        nbytes = 2 * B * T * NH * HD * 2 + T * HD * 4
        copies = cold_slots(nbytes, floor=2)
        tab = precompute_freqs_cis(HD, 4096, 500000.0, True, scale_factor=32.0, device=dev)
        buf0 = torch.empty((B, T, (NH + 16) * HD), dtype=torch.bfloat16, device=dev).normal_()
        bufs = [buf0] + [torch.empty_like(buf0).normal_() for _ in range(copies - 1)]
        xs = [b[..., : NH * HD].view(B, T, NH, HD) for b in bufs]
        ys = [torch.empty((B, T, NH, HD), dtype=torch.bfloat16, device=dev) for _ in xs]
        fr = tab[:T].contiguous()
        st = l3.i64_array((xs[0].stride(0), xs[0].stride(1), xs[0].stride(2)))
        run = lambda: [lib.l3_rot_embed(x.data_ptr(), fr.data_ptr(), y.data_ptr(), B, T, NH, HD, st, sp())  # noqa: E731
                       for x, y in zip(xs, ys)]
        rec = {"tokens": B * T, "NH": NH, "HD": HD}
        keep = (xs[0], fr)
    run()
    gph = capture_graph(torch, run)
    ms, reps = timed_replays(torch, gph)
    ms /= copies
    del gph
    rec.update({"us": round(ms * 1e3, 3), "GBps": round(nbytes / ms / 1e6, 1),
                "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4), "bytes": nbytes, "copies": copies,
                "cold": bool(nbytes * (copies - 1) >= COLD_BYTES), "launches_timed": reps * copies})
    # the read + write yardstick on the same byte count, launched the same way
    del xs, ys
    if name != "rms":
        del bufs
    torch.cuda.empty_cache()
    rec["rw_stream_us"] = measure_rw_stream(torch, lib, dev, nbytes // 2)["us"]
    rec["_keep"] = keep
    rec["_ms"] = ms
    return rec


def public(rec):
    return {k: v for k, v in rec.items() if not k.startswith("_")}


def run_rows(args, torch, lib, l3, dev, name):
    """RMSNorm / rotary embedding at the largest configured shape (4096 rows / tokens), plus the small ones."""
    from oracle.cpu_baseline import rms_norm_cpu, rot_embed_cpu

    detail, head = [], None
    for width in ((2048, 4096) if name == "rms" else (64, 128)):
        for (B, T) in ((1, 1), (1, 64), (1, 256), (2, 2048)):
            rec = rows_record(torch, lib, l3, dev, name, B, T, width)
            if B * T == 4096 and width == (4096 if name == "rms" else 128):
                head = rec
            detail.append(public(rec))
    if name == "rms":
        label = "fused RMSNorm: 4096 rows x C 4096 bf16 (2x2048-token prefill), eps 1e-5"
        metric, kernel = "rms_norm_hbm_GBps", "rms_norm_stream_kernel"
        x, w = (t.cpu() for t in head["_keep"])
        cpu_fn = lambda: rms_norm_cpu(x, w, 1e-5)  # noqa: E731
    else:
        label = "fused rotary embedding: 4096 tokens x 32 heads x HD 128 bf16 from a strided qkv view"
        metric, kernel = "rot_embed_hbm_GBps", "rot_embed_rows_kernel"
        x, f = (t.cpu() for t in head["_keep"])
        cpu_fn = lambda: rot_embed_cpu(x, f)  # noqa: E731
    cpu = None
    if not args.no_cpu_baseline:
        sec, n = time_cpu(cpu_fn, min(args.cpu_seconds, 5.0))
        cpu = {"value": round(head["bytes"] / sec / 1e9, 2), "unit": "GB/s", "cores": torch.get_num_threads(),
               "kind": "port", "host_cpus": os.cpu_count(), "sample": f"{n} runs of the same shape in torch on the CPU"}
    traffic, traffic_src = measured_traffic(name)
    return {
        "metric": metric, "value": head["GBps"], "unit": "GB/s", "frac_of_hbm_peak": head["frac"],
        "steps": head["launches_timed"], "ms_per_step": round(head["_ms"], 5), "dtype": "bf16",
        "config": {"workload": label, "accumulate": "f32", "launch": "hip graph", "seed": SEED},
        "roofline": {"bound": "hbm", "achieved": head["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": head["frac"], "traffic": traffic, "traffic_profile": traffic_src, "kernel": kernel,
                     "algorithmic_bytes_per_launch": head["bytes"]},
        "cpu_baseline": cpu, "per_shape": detail,
    }


def prefill_summary(torch, dev):
    """The causal prefill kernel in short form, for the default line: the library's own choice of form on
    the 1B and 8B prompt shapes and a long prompt, against the dense bf16 MFMA peak with the causal flop
    count; torch's scaled_dot_product_attention on the same tensors beside it (--workload prefill has
    every form)."""
    import torch.nn.functional as F
    from custom_kernels import custom_kernels_extension as cke

    out = []
    for (B, QH, KVH, T, HD) in [(2, 32, 8, 2048, 64), (1, 32, 8, 2048, 128), (1, 32, 8, 8192, 128)]:
        g = torch.Generator().manual_seed(SEED)
        q = torch.randn((B, T, QH, HD), generator=g).to(torch.bfloat16).to(dev).transpose(1, 2)
        k = torch.randn((B, T, KVH, HD), generator=g).to(torch.bfloat16).to(dev).transpose(1, 2)
        v = torch.randn((B, T, KVH, HD), generator=g).to(torch.bfloat16).to(dev).transpose(1, 2)
        flops = 4.0 * B * QH * HD * (T * (T + 1) / 2)
        reps = 8
        cke.flash_attention_prefill(q, k, v)
        gph = capture_graph(torch, lambda: [cke.flash_attention_prefill(q, k, v) for _ in range(reps)])
        t_warm = time.perf_counter()    # untimed: after an idle spell the first milliseconds run at lower clocks
        while time.perf_counter() - t_warm < 0.03:
            gph.replay()
            torch.cuda.synchronize()
        ms = event_time_ms(torch, gph.replay, 5) / reps
        del gph
        try:
            F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
            sd_us = round(1e3 * event_time_ms(torch, lambda: F.scaled_dot_product_attention(q, k, v, is_causal=True,
                                                                                            enable_gqa=True), 10), 2)
        except Exception as exc:  # informational only
            sd_us = None
            print(f"bench.py: torch SDPA failed for {B, QH, KVH, T, HD}: {exc}", file=sys.stderr)
        out.append({"B": B, "QH": QH, "KVH": KVH, "T": T, "HD": HD, "us": round(ms * 1e3, 2),
                    "TFLOPs": round(flops / ms / 1e9, 1), "frac_of_mfma_peak": round(flops / ms / 1e9 / 2500.0, 4),
                    "torch_sdpa_us": sd_us})
    return out


def run_prefill(args, torch, lib, l3, dev):
    """Causal prefill attention (T query tokens against T cached tokens).  Compute-bound: priced
    against the dense bf16 MFMA peak with the causal flop count 4*HD per (query, attended token)
    pair.  torch's own scaled_dot_product_attention on the same tensors is timed beside it."""
    import torch.nn.functional as F
    from custom_kernels import custom_kernels_extension as cke

    MFMA_PEAK_TFLOPS = 2500.0
    shapes = [(1, 32, 8, 128, 64), (1, 32, 8, 2048, 64), (2, 32, 8, 2048, 64), (1, 32, 8, 8192, 64),
              (1, 32, 8, 2048, 128), (1, 32, 8, 4096, 128), (1, 32, 8, 8192, 128)]
    detail, head = [], None
    for (B, QH, KVH, T, HD) in shapes:
        g = torch.Generator().manual_seed(SEED)
        q = torch.randn((B, T, QH, HD), generator=g).to(torch.bfloat16).to(dev).transpose(1, 2)
        k = torch.randn((B, T, KVH, HD), generator=g).to(torch.bfloat16).to(dev).transpose(1, 2)
        v = torch.randn((B, T, KVH, HD), generator=g).to(torch.bfloat16).to(dev).transpose(1, 2)
        flops = 4.0 * B * QH * HD * (T * (T + 1) / 2)
        reps = 8
        forms = {}
        for fname in ("auto", "wave", "tiled"):
            with cke.attention_flags(prefill=fname):
                cke.flash_attention_prefill(q, k, v)
                gph = capture_graph(torch, lambda: [cke.flash_attention_prefill(q, k, v) for _ in range(reps)])
            t_warm = time.perf_counter()    # untimed: after an idle spell the first milliseconds run at lower clocks
            while time.perf_counter() - t_warm < 0.03:
                gph.replay()
                torch.cuda.synchronize()
            forms[fname] = event_time_ms(torch, gph.replay, 5) / reps
            del gph
        ms = forms["auto"]
        try:
            F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
            sd_ms = event_time_ms(torch, lambda: F.scaled_dot_product_attention(q, k, v, is_causal=True,
                                                                                enable_gqa=True), 10)
        except Exception as exc:  # informational only
            sd_ms = None
            print(f"bench.py: torch SDPA failed for {B, QH, KVH, T, HD}: {exc}", file=sys.stderr)
        rec = {"B": B, "QH": QH, "KVH": KVH, "T": T, "HD": HD, "us": round(ms * 1e3, 2),
               "TFLOPs": round(flops / ms / 1e9, 1), "frac": round(flops / ms / 1e9 / MFMA_PEAK_TFLOPS, 4),
               "flops": flops, "wave_form_us": round(forms["wave"] * 1e3, 2),
               "tiled_form_us": round(forms["tiled"] * 1e3, 2),
               "torch_sdpa_us": None if sd_ms is None else round(sd_ms * 1e3, 2)}
        detail.append(rec)
        if (B, T, HD) == (2, 2048, 64):
            head = (rec, ms, q, k, v)
    rec, ms, q, k, v = head
    cpu = None
    if not args.no_cpu_baseline:
        qc, kc, vc = q.cpu(), k.cpu(), v.cpu()
        sec, n = time_cpu(lambda: F.scaled_dot_product_attention(qc, kc, vc, is_causal=True, enable_gqa=True),
                          min(args.cpu_seconds, 10.0))
        cpu = {"value": round(rec["flops"] / sec / 1e12, 3), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
               "kind": "port", "host_cpus": os.cpu_count(),
               "sample": f"{n} runs of the same shape with torch CPU scaled_dot_product_attention (bf16, causal)"}
    return {
        "metric": "prefill_attn_TFLOPs", "value": rec["TFLOPs"], "unit": "TFLOP/s", "steps": args.steps,
        "ms_per_step": round(ms, 5), "dtype": "bf16",
        "config": {"workload": "causal prefill attention: B2 QH32 KVH8 HD64 bf16, 2048 tokens (the 2x2048-token "
                               "prefill of the 1B shape)", "accumulate": "f32", "launch": "hip graph", "seed": SEED},
        "roofline": {"bound": "mfma", "achieved": rec["TFLOPs"], "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": rec["frac"], "traffic": None, "kernel": "attn_prefill_tiled_kernel",
                     "algorithmic_flops_per_launch": rec["flops"]},
        "cpu_baseline": cpu, "per_shape": detail,
    }


def run_linear(args, torch, lib, l3, dev):
    """The nn.Linear calls of one decode step of the 1B architecture (model.py:95,121,134,225) at
    batch 1 (l3_linear_decode / l3_linear_swiglu_decode) and 64 (l3_linear_splitk + finish for the
    three matrices of a few thousand rows, l3_linear_swiglu_decode for the gate|up pair): a stream
    over the weight matrix, priced against HBM.  Each shape owns enough weight copies that the Infinity Cache
    cannot hold them; stock F.linear (hipBLASLt) on the same tensors is timed beside it."""
    import torch.nn.functional as F
    from custom_kernels import custom_kernels_extension as cke

    shapes = [("c_attn", 3072, 2048, False), ("c_proj", 2048, 2048, False), ("mlp gate+up (SwiGLU)", 8192, 2048, True),
              ("mlp c_proj", 2048, 8192, False), ("lm_head", 128256, 2048, False)]
    detail, head = [], None
    for M in (1, 64):
        total_us, total_bytes, torch_us = 0.0, 0, 0.0
        for (name, N, K, swiglu) in shapes:
            wbytes = N * K * 2 * (2 if swiglu else 1)
            copies = max(2, min(48, (1 << 30) // wbytes + 1))
            g = torch.Generator().manual_seed(SEED)
            x = torch.randn((M, K), generator=g).to(torch.bfloat16).to(dev)
            w0 = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16).to(dev)
            ws = [w0] + [w0.clone() for _ in range(copies - 1)]
            ws2 = [w.clone() for w in ws] if swiglu else None
            if swiglu and M > 16:
                # as the end-to-end harness does at these batch sizes: one library GEMM over the stacked
                # gate|up matrix, then the library's SwiGLU product on its two halves
                cats = [torch.cat([a, b], dim=0) for a, b in zip(ws, ws2)]

                def run_l3():
                    for c in cats:
                        gu = F.linear(x, c)
                        cke.silu_mul(gu[..., :N], gu[..., N:])
                run_t = lambda: [F.silu(F.linear(x, a)) * F.linear(x, b) for a, b in zip(ws, ws2)]  # noqa: E731
            elif swiglu:
                run_l3 = lambda: [cke.linear_swiglu_decode(x, a, b) for a, b in zip(ws, ws2)]  # noqa: E731
                run_t = lambda: [F.silu(F.linear(x, a)) * F.linear(x, b) for a, b in zip(ws, ws2)]  # noqa: E731
            else:
                # up to 16 rows: l3_linear_decode; 64 rows: l3_linear_splitk + l3_linear_splitk_finish
                run_l3 = lambda: [cke.linear_decode(x, a) for a in ws]  # noqa: E731
                run_t = lambda: [F.linear(x, a) for a in ws]  # noqa: E731
            # At 64 rows the vocabulary projection stays with the library GEMM (as in the end-to-end harness).
            library = M > 16 and not swiglu and N > 32768
            if library:
                run_l3 = run_t
            run_l3()
            gph = capture_graph(torch, run_l3)
            gph.replay()
            ms = event_time_ms(torch, gph.replay, 5) / copies
            del gph
            run_t()
            gph = capture_graph(torch, run_t)
            gph.replay()
            tms = event_time_ms(torch, gph.replay, 5) / copies
            del gph
            nbytes = wbytes + M * K * 2 + M * N * 2
            detail.append({"M": M, "layer": name, "N": N, "K": K, "us": round(ms * 1e3, 2),
                           "GBps": round(nbytes / ms / 1e6, 1), "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4),
                           "bytes": nbytes, "torch_us": round(tms * 1e3, 2),
                           "path": "F.linear (library GEMM)" if library else
                                   ("F.linear on the stacked matrix + l3_silu_mul_rows" if swiglu and M > 16 else
                                    "l3_linear_swiglu_decode" if swiglu else
                                    ("l3_linear_splitk + l3_linear_splitk_finish" if M > 16 else "l3_linear_decode"))})
            per_token = 1 if name == "lm_head" else 16
            total_us += ms * 1e3 * per_token
            torch_us += tms * 1e3 * per_token
            total_bytes += nbytes * per_token
            del ws, ws2
            torch.cuda.empty_cache()
        detail.append({"M": M, "layer": "all linears of one decode step (16 layers + lm_head)",
                       "us": round(total_us, 1), "GBps": round(total_bytes / total_us / 1e3, 1),
                       "frac": round(total_bytes / total_us / 1e3 / HBM_PEAK_GBPS, 4), "bytes": total_bytes,
                       "torch_us": round(torch_us, 1)})
        if M == 1:
            head = detail[-1]
    return {
        "metric": "decode_linear_hbm_GBps", "value": head["GBps"], "unit": "GB/s", "frac_of_hbm_peak": head["frac"],
        "steps": args.steps, "ms_per_step": round(head["us"] / 1e3, 5), "dtype": "bf16",
        "config": {"workload": "all nn.Linear calls of one batch-1 decode step of the Llama-3.2-1B architecture "
                               "(16 x [c_attn, c_proj, gate+up with SwiGLU, mlp c_proj] + lm_head), weights "
                               "N(0, 0.02)", "accumulate": "f32", "launch": "hip graph", "seed": SEED},
        "roofline": {"bound": "hbm", "achieved": head["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": head["frac"], "traffic": None, "kernel": "linear_skinny_kernel",
                     "algorithmic_bytes_per_launch": head["bytes"] // 65},
        "cpu_baseline": None, "per_shape": detail,
    }


def run_copy(args, torch, dev):
    """A plain device copy of known size (torch's copy kernel): the yardstick that the FETCH_SIZE /
    WRITE_SIZE counters are scaled by, and the practical rate of a read+write stream."""
    nbytes = 256 << 20
    copies = 4
    src = [torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(i) for i in range(copies)]
    dst = [torch.empty(nbytes, dtype=torch.uint8, device=dev) for _ in range(copies)]
    gph = capture_graph(torch, lambda: [d.copy_(s_) for s_, d in zip(src, dst)])
    gph.replay()
    ms = event_time_ms(torch, gph.replay, 10) / copies
    gbps = 2 * nbytes / ms / 1e6
    return {
        "metric": "device_copy_hbm_GBps", "value": round(gbps, 1), "unit": "GB/s",
        "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4), "steps": 10 * copies, "ms_per_step": round(ms, 5),
        "dtype": "u8", "config": {"workload": f"torch device copy, {nbytes} bytes read and {nbytes} bytes written "
                                              "per launch (counter calibration)"},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": None,
                     "algorithmic_bytes_per_launch": 2 * nbytes},
        "cpu_baseline": None,
    }


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3a", "c3b", "hd64", "rms", "rope", "prefill",
                                                         "linear", "e2e", "copy", "readstream"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--single-shot", action="store_true",
                    help="attention workloads: one eager call per length (for profilers), no graph replay")
    ap.add_argument("--no-e2e", action="store_true",
                    help="default workload only: skip the end-to-end tokens/s summary that rides along")
    ap.add_argument("--no-extras", action="store_true",
                    help="default workload only: skip the other shapes of the target (head_dim 64, batched, RMSNorm, rotary)")
    ap.add_argument("--no-sdpa", action="store_true", help="skip torch's scaled_dot_product_attention beside the decode kernel")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="wall time spent on the CPU baseline sample")
    ap.add_argument("--e2e-batch", type=int, default=1)
    ap.add_argument("--attn-kernel", default="default", choices=["default", "mfma", "fma"],
                    help="split-KV kernel to measure (default: the library's choice)")
    ap.add_argument("--two-launches", action="store_true",
                    help="decode attention always as split kernel + combine kernel (no merge inside the split launch)")
    ap.add_argument("--splits", type=int, default=0, help="force the split count (0 = the library's choice)")
    ap.add_argument("--lengths", default="", help="comma-separated KV lengths replacing the workload's own (experiments)")
    ap.add_argument("--cache-len", type=int, default=0,
                    help="attention workloads: K/V as views of caches this many tokens long (the model's batch stride)")
    args = ap.parse_args()

    global FORCE_SPLITS, ATTN_FLAGS
    FORCE_SPLITS = args.splits
    if args.gpus != 1:
        print(f"bench.py: this path runs on one GPU with no sharding; --gpus {args.gpus} is not supported "
              "(every (batch, kv head) pair is independent and could be sharded by batch or kv head)", file=sys.stderr)
        sys.exit(2)

    import torch

    from custom_kernels import _l3lib as l3

    lib = l3.load()  # raises if the HIP library is missing: nothing else can run this path
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the hot path has no CPU implementation to measure", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    # every attention workspace of this file starts with prepared arrival counters (l3_attn_workspace_init)
    ATTN_FLAGS = l3.L3_ATTN_FLAG_WS_COUNTERS
    if args.attn_kernel == "fma":
        ATTN_FLAGS |= l3.L3_ATTN_FLAG_KERNEL_FMA
    if args.two_launches:
        ATTN_FLAGS |= l3.L3_ATTN_FLAG_TWO_LAUNCHES
    attn_opts = {"split_kv_kernel": attn_kernel_name()}
    attention = args.workload in ATTN_WORKLOADS
    default_line = args.workload == "c2" and not args.lengths and not args.single_shot and not args.cache_len

    def cpu_op_table():
        from oracle import cpu_baseline

        class cpu_ops:
            rms_norm = staticmethod(cpu_baseline.rms_norm_cpu)
            rot_embed = staticmethod(cpu_baseline.rot_embed_cpu)
            flash_attention_decode = staticmethod(cpu_baseline.attention_cpu)
        return cpu_ops

    pool = KVPool(torch, dev) if attention or args.workload == "readstream" else None
    if attention:
        res = run_attention(args, torch, lib, l3, dev, args.workload, pool)
    elif args.workload in ("rms", "rope"):
        res = run_rows(args, torch, lib, l3, dev, args.workload)
    elif args.workload == "prefill":
        res = run_prefill(args, torch, lib, l3, dev)
    elif args.workload == "linear":
        res = run_linear(args, torch, lib, l3, dev)
    elif args.workload == "copy":
        res = run_copy(args, torch, dev)
    elif args.workload == "readstream":
        rs = {str(mb): measure_read_stream(torch, lib, dev, pool, mb << 20) for mb in (16, 32, 64, 128, 256, 512)}
        head = rs["128"]
        res = {"metric": "read_stream_hbm_GBps", "value": head["GBps"], "unit": "GB/s", "frac_of_hbm_peak": head["frac"],
               "steps": head["launches_timed"], "ms_per_step": round(head["us"] / 1e3, 5), "dtype": "u8",
               "config": {"workload": "pure read stream over a 1 GiB pool in chunks of 128 MiB (16 ... 512 MiB beside it), "
                                      "each chunk cold", "launch": "hip graph"},
               "roofline": {"bound": "hbm", "achieved": head["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                            "frac": head["frac"], "traffic": None, "kernel": "hbm_read_stream_kernel",
                            "algorithmic_bytes_per_launch": head["bytes_per_launch"]},
               "cpu_baseline": None, "per_chunk_MiB": rs}
    else:
        import llama_arch

        res = llama_arch.bench_e2e(args, torch, dev, None if args.no_cpu_baseline else cpu_op_table())

    head = {"metric": res.pop("metric"), "value": res.pop("value"), "unit": res.pop("unit"), "n_gpus": 1,
            "steps": res.pop("steps"), "warmup": args.warmup, "ms_per_step": res.pop("ms_per_step"),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": res.pop("dtype"),
            "data": "synthetic", "config": res.pop("config")}
    if attention:
        head["config"].update(attn_opts)
    # The line is ordered for a reader who keeps only its end: the bulky per-shape detail first, the contract
    # keys and the summaries ("roofline" with one row per shape of the target, "cpu_baseline") last.
    roofline, cpu = res.pop("roofline", None), res.pop("cpu_baseline", None)
    line = dict(res)
    if default_line:
        # the read bandwidth a pure stream reaches here: the practical ceiling the fractions are read against
        rs = measure_read_stream(torch, lib, dev, pool)
        roofline["practical_read_peak"] = rs
        points = [[f"hd128_b1_s{r['kv_len']}", r["us"], r["frac"], r.get("read_stream_us")] for r in line["per_length"]
                  if r["kv_len"] >= 4096]
        if not args.no_extras:
            ns = north_star_extras(args, torch, lib, l3, dev, pool)
            ns["rms_norm"] = [public(r) for r in ns["rms_norm"]]
            ns["rot_embed"] = [public(r) for r in ns["rot_embed"]]
            ns["hd128_b1"] = [r for r in line["per_length"] if r["kv_len"] >= 4096]
            target = 0.70
            pts = ns["hd128_b1"] + ns["hd64_b1"] + [ns["c3a_b256_hd64_s256"], ns["c3b_b16_hd64_s4096"]]
            ns["target_frac"] = target
            ns["points_at_or_above_target"] = sum(r["frac"] >= target for r in pts)
            ns["points"] = len(pts)
            ns["longer_kv_points_at_or_above_target"] = sum(r["frac"] >= target for r in ns["longer_kv_b1"])
            line["north_star"] = ns
            points += [[f"hd64_b1_s{r['kv_len']}", r["us"], r["frac"], r.get("read_stream_us")] for r in ns["hd64_b1"]]
            points += [[f"hd{r['HD']}_b1_s{r['kv_len']}", r["us"], r["frac"], r.get("read_stream_us")]
                       for r in ns["longer_kv_b1"]]
            points += [[k, ns[k]["us"], ns[k]["frac"], ns[k].get("read_stream_us")]
                       for k in ("c1_b1_hd64_s256", "c3a_b256_hd64_s256", "c3b_b16_hd64_s4096")]
            points += [[f"rms_norm_{r['rows']}x{r['C']}", r["us"], r["frac"], r.get("rw_stream_us")] for r in ns["rms_norm"]]
            points += [[f"rot_embed_{r['tokens']}x{r['NH']}x{r['HD']}", r["us"], r["frac"], r.get("rw_stream_us")]
                       for r in ns["rot_embed"]]
            # the next row after the hot path: causal prefill attention (compute-bound, against the MFMA peak)
            line["prefill"] = prefill_summary(torch, dev)
        # one row per shape of the target: [shape, us per call (split + merge, HBM-cold), fraction of 8 TB/s,
        # us of the yardstick on the same byte count -- the read stream for attention, read + write for the row operators]
        roofline["points"] = points
        roofline["points_columns"] = ["shape", "us", "frac_of_8TBps", "yardstick_us"]
        roofline["points_at_or_above_0.70"] = sum(1 for pt in points if pt[2] >= 0.70)
        del pool
        torch.cuda.empty_cache()
        if not args.no_e2e:
            # the second half of the headline metric: greedy decode tokens/s of the 1B architecture
            # (128 prompt ids + 128 generated tokens; --workload e2e has the detail)
            import llama_arch

            line["e2e"] = llama_arch.e2e_summary(torch, dev, cpu_ops=None if args.no_cpu_baseline else cpu_op_table())
            line["e2e_tokens_per_s"] = {k: v["tok_per_s"] for k, v in line["e2e"].items() if k.startswith("bs")}
            floor_us, launches, wbytes = weights_read_floor_us(torch, lib, dev)
            line["e2e"]["weights_read_stream_floor"] = {
                "us_per_step": floor_us, "launches": launches, "bytes": wbytes,
                "what": "the read-only kernel once per linear kernel of a batch-1 decode step, on that kernel's weight bytes, cold"}
    line.update(head)
    line["roofline"] = roofline
    line["cpu_baseline"] = cpu
    if "e2e_tokens_per_s" in line:
        line["e2e_tokens_per_s"] = line.pop("e2e_tokens_per_s")
    line["device"] = torch.cuda.get_device_name(0)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
