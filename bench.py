#!/usr/bin/env python3
"""Benchmark of the custom-kernel hot path on one MI355X.

Default workload (the headline configuration): decode attention at head_dim 128, batch 1,
32 query / 8 KV heads, bf16, KV length swept over every power of two from 512 to 32768.
One step = one pass over the seven lengths (split-KV kernel + combine each).  Inputs are
resident in HBM before the timed region; each length owns several copies of its K/V and a
pass uses the next copy, so that >1 GB of other traffic separates two reads of the same
bytes and the 256 MB Infinity Cache cannot serve them.  The passes are captured in a HIP
graph (launch-bound otherwise) and replayed; the clock is wall time around the replays with
a device synchronisation on both sides.

Prints ONE JSON line: value = algorithmic GB/s (K+V+Q read, O written) over the timed
steps; "roofline" prices the same bytes against the 8 TB/s HBM peak from HIP-event timing;
"cpu_baseline" is stock PyTorch on the host cores for a bounded sample of the same sweep.

Other workloads (--workload c1|c3a|c3b|hd64|rms|rope|prefill|linear|e2e|copy) report the remaining configurations
in the same format.
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


# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# file (summaries and the copy-kernel calibration are in profiles/); keyed by (workload, kernel).
MEASURED_TRAFFIC = {
    # profiles/attn_splitkv_mfma_c2_sweep_hbm_traffic.md: 38.21 MB fetched + 2.47 MB written per launch
    ("c2", "attn_splitkv_mfma_kernel"): 40680000,
    # profiles/hbm_traffic_batched_attention_rms_norm_rot_embed.md (largest shape of each workload)
    ("c3a", "attn_splitkv_mfma_kernel"): 136660000,   # 135.37 MB fetched + 1.29 MB written
    ("c3b", "attn_splitkv_mfma_kernel"): 135890000,   # 134.39 MB fetched + 1.50 MB written (partials of 11 splits)
    ("rms", "rms_norm_stream_kernel"): 67270000,      # 4096 x 4096: 33.72 MB fetched + 33.55 MB written
    ("rope", "rot_embed_rows_kernel"): 68670000,      # 4096 x 32 x 128: 35.12 MB fetched + 33.55 MB written
}


def attn_kernel_name(lib=None):
    from custom_kernels import _l3lib as l3
    return "fma" if ATTN_FLAGS & l3.L3_ATTN_FLAG_KERNEL_FMA else "mfma"


def attn_bytes(B, QH, KVH, S, HD):
    """K+V+Q read, O written, bf16 (the reference counts K+V only: benchmark_kernel.py:48)."""
    return 2 * B * KVH * S * HD * 2 + 2 * B * QH * HD * 2


class AttnCase:
    """One attention shape with `slots` independent copies of its inputs, pre-allocated outputs
    and workspace, launched straight through the C ABI (no per-call allocation)."""

    def __init__(self, torch, lib, l3, dev, B, QH, KVH, S, HD, slots, src_k=None, src_v=None, src_q=None,
                 cache_len=0):
        self.torch, self.lib = torch, lib
        self.B, self.QH, self.KVH, self.S, self.HD = B, QH, KVH, S, HD
        self.bytes = attn_bytes(B, QH, KVH, S, HD)
        self.slots = slots
        g = torch.Generator().manual_seed(SEED)
        q = src_q if src_q is not None else torch.randn((B, 1, QH, HD), generator=g).to(torch.bfloat16)
        k = src_k if src_k is not None else torch.randn((B, S, KVH, HD), generator=g).to(torch.bfloat16)
        v = src_v if src_v is not None else torch.randn((B, S, KVH, HD), generator=g).to(torch.bfloat16)
        self.cpu = (q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
        # token-major storage, transposed views: the model's cache layout (benchmark_kernel.py:165-173)
        self.q = [q.to(dev).transpose(1, 2) for _ in range(slots)]
        if cache_len > S:
            # the model's layout (model.py:107-111): a (B, L, KVH, HD) cache of which the first S tokens are attended
            def cache_view(t):
                full = torch.zeros((B, cache_len, KVH, HD), dtype=torch.bfloat16, device=dev)
                full[:, :S] = t.to(dev)
                return full[:, :S].transpose(1, 2)
            self.k = [cache_view(k) for _ in range(slots)]
            self.v = [cache_view(v) for _ in range(slots)]
        else:
            self.k = [k.to(dev).transpose(1, 2) for _ in range(slots)]
            self.v = [v.to(dev).transpose(1, 2) for _ in range(slots)]
        self.out = [torch.empty_like(t) for t in self.q]
        # 0 = the library plans for the current device (split count and kernel form)
        self.req_splits = FORCE_SPLITS
        self.num_splits = FORCE_SPLITS or lib.l3_attn_choose_splits(B, KVH, S, HD, 0, ATTN_FLAGS)
        self.ws_bytes = lib.l3_attn_decode_workspace_bytes(B, QH, KVH, S, HD, self.req_splits, ATTN_FLAGS)
        self.ws = torch.empty(max(self.ws_bytes, 256), dtype=torch.uint8, device=dev)
        self.part_o = self.part_ml = None
        self._args = []
        for i in range(slots):
            qt, kt, vt, ot = self.q[i], self.k[i], self.v[i], self.out[i]
            self._args.append((
                qt.data_ptr(), kt.data_ptr(), vt.data_ptr(), ot.data_ptr(), self.ws.data_ptr(), self.ws_bytes,
                B, QH, KVH, S, HD,
                l3.i64_array((qt.stride(0), qt.stride(1))), l3.i64_array((kt.stride(0), kt.stride(1), kt.stride(2))),
                l3.i64_array((vt.stride(0), vt.stride(1), vt.stride(2))), l3.i64_array((ot.stride(0), ot.stride(1))),
                1.0 / math.sqrt(HD), self.req_splits, ATTN_FLAGS))

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
                                    self.req_splits, ATTN_FLAGS, stream_ptr)
        if rc < 0:
            raise RuntimeError(f"l3_attn_split failed: {rc}")


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


# ------------------------------------------------------------------------------ workloads
def run_attention(args, torch, lib, l3, dev, name):
    from oracle.cpu_baseline import attention_cpu

    QH, KVH = 32, 8
    if name == "c2":
        B, HD, lengths = 1, 128, [512, 1024, 2048, 4096, 8192, 16384, 32768]
        label = "decode attention sweep: B1 QH32 KVH8 HD128 bf16, KV length 512..32768 (x2), split+combine"
    elif name == "c1":
        B, HD, lengths = 1, 64, [256]
        label = "decode attention: B1 QH32 KVH8 HD64 bf16, KV length 256, split+combine"
    elif name == "c3a":
        B, HD, lengths = 256, 64, [256]
        label = "batched decode attention: B256 QH32 KVH8 HD64 bf16, KV length 256"
    elif name == "c3b":
        B, HD, lengths = 16, 64, [4096]
        label = "batched decode attention: B16 QH32 KVH8 HD64 bf16, KV length 4096, split+combine"
    elif name == "hd64":
        B, HD, lengths = 1, 64, [512, 1024, 2048, 4096, 8192, 16384, 32768]
        label = "decode attention sweep: B1 QH32 KVH8 HD64 bf16, KV length 512..32768 (x2), split+combine"
    else:
        raise ValueError(name)

    if args.lengths:
        lengths = [int(x) for x in args.lengths.split(",")]
        label += f" [lengths overridden: {lengths}]"
    smax = max(lengths)
    g = torch.Generator().manual_seed(SEED)
    q = torch.randn((B, 1, QH, HD), generator=g).to(torch.bfloat16)
    k = torch.randn((B, smax, KVH, HD), generator=g).to(torch.bfloat16)
    v = torch.randn((B, smax, KVH, HD), generator=g).to(torch.bfloat16)
    pass_bytes = sum(attn_bytes(B, QH, KVH, S, HD) for S in lengths)
    # enough copies that a pass over all of them moves > 1 GiB between two uses of the same bytes
    slots = max(4, int(math.ceil((1 << 30) / pass_bytes)))
    slots = min(slots, 64)
    if args.cache_len:
        label += f" [K/V are views of (B, {args.cache_len}, KVH, HD) caches]"
    cases = [AttnCase(torch, lib, l3, dev, B, QH, KVH, S, HD, slots, src_k=k[:, :S].contiguous(),
                      src_v=v[:, :S].contiguous(), src_q=q, cache_len=args.cache_len) for S in lengths]

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

    passes_per_graph = slots
    graph = capture_graph(torch, lambda: [one_pass(s) for s in range(passes_per_graph)])

    steps = max(passes_per_graph, (args.steps + passes_per_graph - 1) // passes_per_graph * passes_per_graph)
    warm = max(1, (args.warmup + passes_per_graph - 1) // passes_per_graph)
    for _ in range(warm):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps // passes_per_graph):
        graph.replay()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / steps
    value = pass_bytes / (ms_per_step * 1e-3) / 1e9

    # HIP-event timing of the same replays (events on the stream the kernels run on)
    ev_ms = event_time_ms(torch, graph.replay, max(1, steps // passes_per_graph)) / passes_per_graph
    op_gbps = pass_bytes / (ev_ms * 1e-3) / 1e9

    # The dominant kernel on its own: the split-KV stage of every length, same rotation, graph-replayed.
    def split_pass(slot):
        sp = torch.cuda.current_stream().cuda_stream
        for c in cases:
            c.launch_split_stage(slot, sp)

    split_pass(0)
    sgraph = capture_graph(torch, lambda: [split_pass(s) for s in range(passes_per_graph)])
    sgraph.replay()
    split_ms = event_time_ms(torch, sgraph.replay, max(1, steps // passes_per_graph)) / passes_per_graph
    achieved = pass_bytes / (split_ms * 1e-3) / 1e9
    split_kernel = "attn_splitkv_mfma_kernel" if attn_kernel_name(lib) == "mfma" else "attn_splitkv_fma_kernel"
    del sgraph

    # per-length detail: each length alone, rotating over its copies, graph-replayed
    detail = []
    for c in cases:
        reps_in_graph = max(slots, 16)
        gph = capture_graph(torch, lambda c=c: [c.launch(s, torch.cuda.current_stream().cuda_stream)
                                                for s in range(reps_in_graph)])
        gph.replay()
        ms = event_time_ms(torch, gph.replay, 5) / reps_in_graph
        gbps = c.bytes / (ms * 1e-3) / 1e9
        detail.append({"kv_len": c.S, "splits": c.num_splits, "us": round(ms * 1e3, 3), "GBps": round(gbps, 1),
                       "frac": round(gbps / HBM_PEAK_GBPS, 4), "bytes": c.bytes,
                       "cold": bool(c.bytes * slots > (300 << 20))})
        del gph

    cpu = None
    if not args.no_cpu_baseline and name in ("c2", "c1"):
        def cpu_pass():
            for c in cases:
                attention_cpu(*c.cpu)
        sec, n = time_cpu(cpu_pass, args.cpu_seconds)
        cpu = {"value": round(pass_bytes / sec / 1e9, 2), "unit": "GB/s", "cores": torch.get_num_threads(),
               "kind": "port", "host_cpus": os.cpu_count(),
               "sample": f"{n} passes of the same sweep with torch CPU scaled_dot_product_attention "
                         f"(bf16, enable_gqa) in {sec * n:.1f} s"}

    return {
        "metric": "decode_attn_hbm_GBps", "value": round(value, 1), "unit": "GB/s",
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "steps": steps, "ms_per_step": round(ms_per_step, 5), "dtype": "bf16",
        "config": {"workload": label, "kv_copies_per_length": slots, "accumulate": "f32", "launch": "hip graph",
                   "seed": SEED},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": MEASURED_TRAFFIC.get((name, split_kernel)),
                     "kernel": split_kernel, "launches_per_pass": len(cases),
                     "avg_launch_us": round(split_ms * 1e3 / len(cases), 3),
                     "algorithmic_bytes_per_launch": pass_bytes // len(cases),
                     "split_plus_combine_GBps": round(op_gbps, 1),
                     "split_plus_combine_frac": round(op_gbps / HBM_PEAK_GBPS, 4)},
        "cpu_baseline": cpu, "per_length": detail,
    }


def run_rows(args, torch, lib, l3, dev, name):
    """RMSNorm / rotary embedding at the largest configured shape (4096 rows / tokens), plus the small ones."""
    from custom_kernels import custom_kernels_extension as cke
    from custom_kernels import precompute_freqs_cis
    from oracle.cpu_baseline import rms_norm_cpu, rot_embed_cpu

    detail = []
    head = None
    if name == "rms":
        for C in (2048, 4096):
            for (B, T) in ((1, 1), (1, 64), (1, 256), (2, 2048)):
                copies = max(2, min(64, (1 << 30) // max(1, 2 * B * T * C * 2)))
                g = torch.Generator().manual_seed(SEED)
                xs = [torch.randn((B, T, C), generator=g).to(torch.bfloat16).to(dev) for _ in range(min(copies, 4))]
                xs = xs + [xs[0].clone() for _ in range(copies - len(xs))]
                w = (torch.randn((C,), generator=g) * 0.02 + 1).to(torch.bfloat16).to(dev)
                ys = [torch.empty_like(x) for x in xs]
                sp = lambda: torch.cuda.current_stream().cuda_stream  # noqa: E731
                gph = capture_graph(torch, lambda: [lib.l3_rms_norm(x.data_ptr(), w.data_ptr(), y.data_ptr(), B * T, C,
                                                                    1e-5, sp()) for x, y in zip(xs, ys)])
                gph.replay()
                ms = event_time_ms(torch, gph.replay, 10) / copies
                nbytes = 2 * B * T * C * 2 + C * 2
                rec = {"rows": B * T, "C": C, "us": round(ms * 1e3, 3), "GBps": round(nbytes / ms / 1e6, 1),
                       "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4), "bytes": nbytes}
                detail.append(rec)
                if C == 4096 and B * T == 4096:
                    head = (rec, ms, nbytes, lambda x=xs[0].cpu(), w=w.cpu(): rms_norm_cpu(x, w, 1e-5))
        label = "fused RMSNorm: 4096 rows x C 4096 bf16 (2x2048-token prefill), eps 1e-5"
        metric = "rms_norm_hbm_GBps"
    else:
        for HD in (64, 128):
            tab = precompute_freqs_cis(HD, 4096, 500000.0, True, scale_factor=32.0, device=dev)
            for (B, T) in ((1, 1), (1, 64), (1, 256), (2, 2048)):
                NH = 32
                copies = max(2, min(64, (1 << 30) // max(1, 2 * B * T * NH * HD * 2)))
                g = torch.Generator().manual_seed(SEED)
                buf0 = torch.randn((B, T, (NH + 16) * HD), generator=g).to(torch.bfloat16).to(dev)
                bufs = [buf0] + [buf0.clone() for _ in range(copies - 1)]
                xs = [b[..., : NH * HD].view(B, T, NH, HD) for b in bufs]
                ys = [torch.empty((B, T, NH, HD), dtype=torch.bfloat16, device=dev) for _ in xs]
                fr = tab[:T].contiguous()
                st = l3.i64_array((xs[0].stride(0), xs[0].stride(1), xs[0].stride(2)))
                sp = lambda: torch.cuda.current_stream().cuda_stream  # noqa: E731
                gph = capture_graph(torch, lambda: [lib.l3_rot_embed(x.data_ptr(), fr.data_ptr(), y.data_ptr(), B, T,
                                                                     NH, HD, st, sp()) for x, y in zip(xs, ys)])
                gph.replay()
                ms = event_time_ms(torch, gph.replay, 10) / copies
                nbytes = 2 * B * T * NH * HD * 2 + T * HD * 4
                rec = {"tokens": B * T, "NH": NH, "HD": HD, "us": round(ms * 1e3, 3),
                       "GBps": round(nbytes / ms / 1e6, 1), "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4),
                       "bytes": nbytes}
                detail.append(rec)
                if HD == 128 and B * T == 4096:
                    head = (rec, ms, nbytes, lambda x=xs[0].cpu(), f=fr.cpu(): rot_embed_cpu(x, f))
        label = "fused rotary embedding: 4096 tokens x 32 heads x HD 128 bf16 from a strided qkv view"
        metric = "rot_embed_hbm_GBps"

    rec, ms, nbytes, cpu_fn = head
    cpu = None
    if not args.no_cpu_baseline:
        sec, n = time_cpu(cpu_fn, min(args.cpu_seconds, 5.0))
        cpu = {"value": round(nbytes / sec / 1e9, 2), "unit": "GB/s", "cores": torch.get_num_threads(),
               "kind": "port", "host_cpus": os.cpu_count(), "sample": f"{n} runs of the same shape in torch on the CPU"}
    return {
        "metric": metric, "value": rec["GBps"], "unit": "GB/s", "frac_of_hbm_peak": rec["frac"],
        "steps": args.steps, "ms_per_step": round(ms, 5), "dtype": "bf16",
        "config": {"workload": label, "accumulate": "f32", "launch": "hip graph", "seed": SEED},
        "roofline": {"bound": "hbm", "achieved": rec["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": rec["frac"],
                     "traffic": MEASURED_TRAFFIC.get((name, "rms_norm_stream_kernel" if name == "rms"
                                                      else "rot_embed_rows_kernel")),
                     "kernel": "rms_norm_stream_kernel" if name == "rms" else "rot_embed_rows_kernel",
                     "algorithmic_bytes_per_launch": nbytes},
        "cpu_baseline": cpu, "per_shape": detail,
    }


def run_prefill(args, torch, lib, l3, dev):
    """Causal prefill attention (T query tokens against T cached tokens).  Compute-bound: priced
    against the dense bf16 MFMA peak with the causal flop count 4*HD per (query, attended token)
    pair.  torch's own scaled_dot_product_attention on the same tensors is timed beside it."""
    import torch.nn.functional as F
    from custom_kernels import custom_kernels_extension as cke

    MFMA_PEAK_TFLOPS = 2500.0
    shapes = [(1, 32, 8, 128, 64), (2, 32, 8, 2048, 64), (1, 32, 8, 8192, 64), (1, 32, 8, 2048, 128),
              (1, 32, 8, 4096, 128), (1, 32, 8, 8192, 128)]
    detail, head = [], None
    for (B, QH, KVH, T, HD) in shapes:
        g = torch.Generator().manual_seed(SEED)
        q = torch.randn((B, T, QH, HD), generator=g).to(torch.bfloat16).to(dev).transpose(1, 2)
        k = torch.randn((B, T, KVH, HD), generator=g).to(torch.bfloat16).to(dev).transpose(1, 2)
        v = torch.randn((B, T, KVH, HD), generator=g).to(torch.bfloat16).to(dev).transpose(1, 2)
        flops = 4.0 * B * QH * HD * (T * (T + 1) / 2)
        reps = 8
        forms = {}
        for fname in ("auto", "wave", "tiled", "pipelined"):
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
               "pipelined_form_us": round(forms["pipelined"] * 1e3, 2),
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
                     "frac": rec["frac"], "traffic": None, "kernel": "attn_prefill_pipe_kernel",
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
            if swiglu:
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
                                   ("l3_linear_swiglu_decode" if swiglu else
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
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3a", "c3b", "hd64", "rms", "rope", "prefill", "linear", "e2e", "copy"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--single-shot", action="store_true",
                    help="attention workloads: one eager call per length (for profilers), no graph replay")
    ap.add_argument("--no-e2e", action="store_true",
                    help="default workload only: skip the end-to-end tokens/s summary that rides along")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="wall time spent on the CPU baseline sample")
    ap.add_argument("--e2e-batch", type=int, default=1)
    ap.add_argument("--attn-kernel", default="default", choices=["default", "mfma", "fma"],
                    help="split-KV kernel to measure (default: the library's choice)")
    ap.add_argument("--splits", type=int, default=0, help="force the split count (0 = the library's choice)")
    ap.add_argument("--lengths", default="", help="comma-separated KV lengths replacing the workload's own (experiments)")
    ap.add_argument("--cache-len", type=int, default=0,
                    help="attention workloads: K/V as views of caches this many tokens long (the model's batch stride)")
    args = ap.parse_args()

    global FORCE_SPLITS
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
    global ATTN_FLAGS
    if args.attn_kernel == "fma":
        ATTN_FLAGS = l3.L3_ATTN_FLAG_KERNEL_FMA
    attn_opts = {"split_kv_kernel": attn_kernel_name(lib)}

    if args.workload in ("c1", "c2", "c3a", "c3b", "hd64"):
        res = run_attention(args, torch, lib, l3, dev, args.workload)
    elif args.workload in ("rms", "rope"):
        res = run_rows(args, torch, lib, l3, dev, args.workload)
    elif args.workload == "prefill":
        res = run_prefill(args, torch, lib, l3, dev)
    elif args.workload == "linear":
        res = run_linear(args, torch, lib, l3, dev)
    elif args.workload == "copy":
        res = run_copy(args, torch, dev)
    else:
        import llama_arch

        cpu_ops = None
        if not args.no_cpu_baseline:
            from oracle import cpu_baseline

            class cpu_ops:
                rms_norm = staticmethod(cpu_baseline.rms_norm_cpu)
                rot_embed = staticmethod(cpu_baseline.rot_embed_cpu)
                flash_attention_decode = staticmethod(cpu_baseline.attention_cpu)

        res = llama_arch.bench_e2e(args, torch, dev, cpu_ops)

    line = {"metric": res.pop("metric"), "value": res.pop("value"), "unit": res.pop("unit"), "n_gpus": 1,
            "steps": res.pop("steps"), "warmup": args.warmup, "ms_per_step": res.pop("ms_per_step"),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": res.pop("dtype"),
            "data": "synthetic", "config": res.pop("config")}
    line.update(res)
    if args.workload in ("c1", "c2", "c3a", "c3b", "hd64"):
        line["config"].update(attn_opts)
    if args.workload == "c2" and not args.no_e2e and not args.lengths and not args.single_shot:
        # the second half of the headline metric: greedy decode tokens/s of the 1B architecture
        # (128 prompt ids + 128 generated tokens, graph-replayed loop; --workload e2e has the detail)
        import llama_arch

        line["e2e_tokens_per_s"] = llama_arch.e2e_summary(torch, dev)
    line["device"] = torch.cuda.get_device_name(0)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
