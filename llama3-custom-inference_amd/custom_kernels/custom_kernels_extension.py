"""The three operators the reference binds in custom_kernels/main.cpp:5-9, same names and
positional signatures, backed by the gfx950 kernels of libl3kernels.so.

    flash_attention_decode(query, keys, values) -> Tensor    custom_kernels.cu:233-338
    rms_norm(input, weight, eps) -> Tensor                   custom_kernels.cu:369-389
    rot_embed(input, freq) -> Tensor                         custom_kernels.cu:418-442

Outputs are fresh tensors with the reference's shapes, dtypes and strides
(``empty_like(query)``, ``empty_like(input)``, and a contiguous (B, T, NH, HD) tensor for
rot_embed).  Unsupported arguments raise RuntimeError like the reference's TORCH_CHECKs.
Kernels are enqueued on torch's current stream of the input's device and the call does
not synchronise.  There is no fallback path: a missing library or a non-GPU tensor raises.
"""

import contextlib
import contextvars
import math

import torch

from . import _l3lib

__all__ = ["flash_attention_decode", "rms_norm", "rot_embed", "attention_num_splits", "attention_flags",
           "flash_attention_decode_static",
           "flash_attention_split", "flash_attention_combine", "flash_attention_decode_devlen",
           "rot_embed_append", "add_rms_norm", "silu_mul", "argmax", "flash_attention_prefill"]

_cu_count = {}
_workspaces = {}  # (device index, stream handle) -> uint8 tensor


def _fail(code: int, detail: str = ""):
    msg = _l3lib.strerror(code)
    raise RuntimeError(f"{msg}{': ' + detail if detail else ''} (l3 error {code})")


def _require_gpu_bf16(name: str, t: torch.Tensor):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be on the GPU (got {t.device}); there is no CPU path")
    if t.dtype != torch.bfloat16:
        # the reference's data_ptr<at::BFloat16>() raises the same way (custom_kernels.cu:274)
        raise RuntimeError(f"expected scalar type BFloat16 for {name} but found {t.dtype}")


# The raw handle of torch's current stream without building a Stream object (2 us per call saved);
# the public accessor is the fallback where this build of torch does not have the direct one.
_raw_current_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_NO_GUARD = contextlib.nullcontext()


def _stream_ptr(device) -> int:
    if _raw_current_stream is not None:
        idx = device.index
        return _raw_current_stream(idx if idx is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


def _on_device(device):
    """Context in which `device` is the current one: nothing to do (and nothing to pay) when it
    already is, which is every call of a single-GPU process."""
    idx = device.index
    if idx is None or idx == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(idx)


def _cus(device) -> int:
    idx = device.index if device.index is not None else torch.cuda.current_device()
    n = _cu_count.get(idx)
    if n is None:
        n = torch.cuda.get_device_properties(idx).multi_processor_count
        _cu_count[idx] = n
    return n


def _workspace(device, stream_ptr: int, nbytes: int):
    """Scratch for the kernels that need it (attention partials, argmax partials), kept per
    (device, stream) and grown on demand so that a decode step does not allocate.  Calls on one
    stream are ordered and can share it; another stream gets its own.  While a stream is being
    captured into a HIP graph the buffer comes from the graph's own memory pool instead (a plain
    allocation that lives and dies with the graph) and is not cached."""
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_ptr)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


_attn_workspaces = {}  # (device index, stream handle) -> uint8 tensor that starts with prepared arrival counters


def _attn_workspace(lib, device, stream_ptr: int, flags: int, size_of):
    """Workspace and flags for a decode-attention call.  Outside stream capture the workspace is one kept per
    (device, stream) whose head holds the arrival counters of the single-launch form, prepared once by
    l3_attn_workspace_init when the buffer is (re)allocated -- that call synchronises, which a capture
    would not allow, so a call under capture takes a plain buffer from the graph's pool and runs split
    kernel + combine.  ``size_of(flags)`` returns the bytes the call needs with those flags."""
    if torch.cuda.is_current_stream_capturing():
        flags &= ~_l3lib.L3_ATTN_FLAG_WS_COUNTERS
        nbytes = size_of(flags)
        return (_workspace(device, stream_ptr, nbytes) if nbytes else None), nbytes, flags
    flags |= _l3lib.L3_ATTN_FLAG_WS_COUNTERS
    nbytes = size_of(flags)
    if nbytes == 0:
        return None, 0, flags
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_ptr)
    ws = _attn_workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 4 << 20), dtype=torch.uint8, device=device)
        rc = lib.l3_attn_workspace_init(ws.data_ptr(), ws.numel(), stream_ptr)
        if rc != 0:
            _fail(rc, "l3_attn_workspace_init")
        _attn_workspaces[key] = ws
    return ws, nbytes, flags


# Flags the attention operators pass to the library when the caller gives none: a context-local
# value (per thread / per asyncio task), never a process-wide switch.  The library itself keeps no
# option between calls.
_attn_flags = contextvars.ContextVar("l3_attn_flags", default=0)

_KERNEL_BITS = {"mfma": 0, "fma": _l3lib.L3_ATTN_FLAG_KERNEL_FMA}
_PREFILL_BITS = {"auto": 0, "wave": _l3lib.L3_ATTN_FLAG_PREFILL_WAVE, "tiled": _l3lib.L3_ATTN_FLAG_PREFILL_TILED,
                 "tiled-no-max": _l3lib.L3_ATTN_FLAG_PREFILL_TILED_NO_MAX}
_LAUNCH_BITS = {"auto": 0, "two": _l3lib.L3_ATTN_FLAG_TWO_LAUNCHES}


@contextlib.contextmanager
def attention_flags(kernel=None, prefill=None, launches=None):
    """Within the block, attention calls of this thread that pass no ``flags`` use the named
    split-KV kernel ("mfma" / "fma"), prefill form ("auto" / "wave" / "tiled" / "tiled-no-max") and launch scheme
    ("auto" / "two": always split kernel + combine kernel).  An argument that is not given keeps what
    an enclosing block chose, so blocks nest.  For measurements and tests; the defaults are the
    library's own choices."""
    bits = _attn_flags.get()
    for name, table, mask in ((kernel, _KERNEL_BITS, _l3lib.L3_ATTN_FLAG_KERNEL_FMA),
                              (prefill, _PREFILL_BITS, _l3lib.L3_ATTN_FLAG_PREFILL_MASK),
                              (launches, _LAUNCH_BITS, _l3lib.L3_ATTN_FLAG_TWO_LAUNCHES)):
        if name is not None:
            bits = (bits & ~mask) | table[name]
    token = _attn_flags.set(bits)
    try:
        yield
    finally:
        _attn_flags.reset(token)


def _flags(flags):
    return _attn_flags.get() if flags is None else int(flags)


def attention_num_splits(B: int, KVH: int, S: int, HD: int, num_cus: int = 256, flags=None) -> int:
    """Split count the kernel picks for this problem (pure host logic, runs without a GPU)."""
    n = _l3lib.load().l3_attn_choose_splits(B, KVH, S, HD, num_cus, _flags(flags))
    if n < 0:
        _fail(n)
    return n


def _check_out(out, like, what: str):
    """A caller-supplied output is written through its raw pointer with `like`'s shape: it must be
    a bf16 tensor of that shape on the same device whose rows the kernels can address."""
    if not isinstance(out, torch.Tensor) or out.dtype != torch.bfloat16 or out.device != like.device \
            or tuple(out.shape) != tuple(like.shape):
        raise RuntimeError(f"{what}: out must be a bf16 tensor of shape {tuple(like.shape)} on {like.device}")
    if out.stride(-1) != 1 or any(st % 8 for st, n in zip(out.stride()[:-1], out.shape[:-1]) if n > 1):
        raise RuntimeError(f"{what}: out needs a contiguous last dimension and 16-byte aligned rows")


def flash_attention_decode(query, keys, values, num_splits: int = 0, flags=None):
    """query (B, QH, 1, HD); keys/values (B, KVH, S, HD) views of the KV cache (model.py:107-118).

    ``num_splits`` (0 = automatic) and ``flags`` (L3_ATTN_FLAG_* bits, None = attention_flags()'s
    context, normally 0) are extensions for tests and sweeps; the reference signature is the three
    tensors.
    """
    lib = _l3lib.load()
    flags = _flags(flags)
    B, QH, KVH, S, HD = _check_qkv(query, keys, values)
    if keys.device != query.device or values.device != query.device:
        raise RuntimeError("query, keys and values must be on the same device")
    if HD not in (64, 128):
        _fail(_l3lib.L3_ERR_HEAD_SIZE, str(HD))
    if KVH == 0 or QH % KVH != 0 or (QH // KVH) not in (1, 2, 3, 4, 8):
        _fail(_l3lib.L3_ERR_HEAD_RATIO, f"{QH}/{KVH}")

    out = torch.empty_like(query)
    if out.stride(3) != 1:
        out = torch.empty(query.shape, dtype=query.dtype, device=query.device)
    if B == 0 or S == 0:
        raise RuntimeError("flash_attention_decode needs at least one sequence and one cached token")

    with _on_device(query.device):
        # num_splits == 0 lets the library plan for the current device (split count and kernel form)
        stream_ptr = _stream_ptr(query.device)
        ws, ws_bytes, flags = _attn_workspace(
            lib, query.device, stream_ptr, flags,
            lambda f: lib.l3_attn_decode_workspace_bytes(B, QH, KVH, S, HD, num_splits, f))
        rc = lib.l3_attn_decode(
            query.data_ptr(), keys.data_ptr(), values.data_ptr(), out.data_ptr(),
            ws.data_ptr() if ws is not None else None, ws_bytes,
            B, QH, KVH, S, HD,
            _l3lib.i64_array((query.stride(0), query.stride(1))),
            _l3lib.i64_array((keys.stride(0), keys.stride(1), keys.stride(2))),
            _l3lib.i64_array((values.stride(0), values.stride(1), values.stride(2))),
            _l3lib.i64_array((out.stride(0), out.stride(1))),
            1.0 / math.sqrt(HD), num_splits, flags, stream_ptr)
    if rc != 0:
        _fail(rc, f"B={B} QH={QH} KVH={KVH} S={S} HD={HD}")
    return out


def flash_attention_decode_static(query, keys, values, out, num_splits: int = 0, flags=None):
    """flash_attention_decode into the caller's ``out`` with the partials in the library's static
    device scratch: the call allocates nothing (l3_attn_decode_static).  Raises when the problem
    needs more scratch than the static array holds.  Calls that overlap on one GPU race."""
    lib = _l3lib.load()
    flags = _flags(flags)
    B, QH, KVH, S, HD = _check_qkv(query, keys, values)
    if keys.device != query.device or values.device != query.device:
        raise RuntimeError("query, keys and values must be on the same device")
    _check_out(out, query, "flash_attention_decode_static")
    with _on_device(query.device):
        rc = lib.l3_attn_decode_static(
            query.data_ptr(), keys.data_ptr(), values.data_ptr(), out.data_ptr(), B, QH, KVH, S, HD,
            _l3lib.i64_array((query.stride(0), query.stride(1))),
            _l3lib.i64_array((keys.stride(0), keys.stride(1), keys.stride(2))),
            _l3lib.i64_array((values.stride(0), values.stride(1), values.stride(2))),
            _l3lib.i64_array((out.stride(0), out.stride(1))),
            1.0 / math.sqrt(HD), num_splits, flags, _stream_ptr(query.device))
    if rc != 0:
        _fail(rc, f"B={B} QH={QH} KVH={KVH} S={S} HD={HD}")
    return out


def _check_qkv(query, keys, values):
    _require_gpu_bf16("query", query)
    _require_gpu_bf16("keys", keys)
    _require_gpu_bf16("values", values)
    if query.dim() != 4 or keys.dim() != 4 or values.dim() != 4:
        raise RuntimeError("expected 4-D query, keys and values")
    B, KVH, S, HD = keys.shape
    QH = query.size(1)
    if query.size(0) != B or query.size(2) != 1 or query.size(3) != HD or tuple(values.shape) != tuple(keys.shape):
        raise RuntimeError(
            f"shape mismatch: query {tuple(query.shape)}, keys {tuple(keys.shape)}, values {tuple(values.shape)}")
    if query.stride(3) != 1 or keys.stride(3) != 1 or values.stride(3) != 1:
        raise RuntimeError("the head dimension of query, keys and values must be contiguous")
    return B, QH, KVH, S, HD


def flash_attention_prefill(query, keys, values, flags=None):
    """Causal GQA attention for T > 1 query tokens: query (B, QH, T, HD), keys / values
    (B, KVH, S, HD) cache views with S >= T; query i attends to tokens 0 .. S - T + i.  Returns a
    (B, QH, T, HD) view of a contiguous (B, T, QH, HD) tensor, so the model's
    ``y.transpose(1, 2).contiguous()`` (model.py:120) is free.  For S == T it computes what the
    reference asks of torch for this case (model.py:114-116).  An extension of the operator set."""
    lib = _l3lib.load()
    _require_gpu_bf16("query", query)
    _require_gpu_bf16("keys", keys)
    _require_gpu_bf16("values", values)
    if query.dim() != 4 or keys.dim() != 4 or tuple(values.shape) != tuple(keys.shape):
        raise RuntimeError("flash_attention_prefill expects 4-D query, keys and values (keys and values alike)")
    B, QH, T, HD = query.shape
    Bk, KVH, S, HDk = keys.shape
    if Bk != B or HDk != HD or T > S:
        raise RuntimeError(f"shape mismatch: query {tuple(query.shape)}, keys {tuple(keys.shape)}")
    if query.stride(3) != 1 or keys.stride(3) != 1 or values.stride(3) != 1:
        raise RuntimeError("the head dimension of query, keys and values must be contiguous")
    if HD not in (64, 128):
        _fail(_l3lib.L3_ERR_HEAD_SIZE, str(HD))
    if KVH == 0 or QH % KVH != 0 or (QH // KVH) not in (1, 2, 3, 4, 8):
        _fail(_l3lib.L3_ERR_HEAD_RATIO, f"{QH}/{KVH}")
    out = torch.empty((B, T, QH, HD), dtype=query.dtype, device=query.device).transpose(1, 2)
    if out.numel() == 0:
        return out
    with _on_device(query.device):
        rc = lib.l3_attn_prefill(
            query.data_ptr(), keys.data_ptr(), values.data_ptr(), out.data_ptr(), B, QH, KVH, T, S, HD,
            _l3lib.i64_array((query.stride(0), query.stride(1), query.stride(2))),
            _l3lib.i64_array((keys.stride(0), keys.stride(1), keys.stride(2))),
            _l3lib.i64_array((values.stride(0), values.stride(1), values.stride(2))),
            _l3lib.i64_array((out.stride(0), out.stride(1), out.stride(2))),
            1.0 / math.sqrt(HD), _flags(flags), _stream_ptr(query.device))
    if rc != 0:
        _fail(rc, f"B={B} QH={QH} KVH={KVH} T={T} S={S} HD={HD}")
    return out


def flash_attention_split(query, keys, values, num_splits: int = 0, flags=None):
    """First stage of flash_attention_decode on its own (an extension; the reference runs its two
    kernels only together, custom_kernels.cu:274-275).  Returns float32 partials
    ``(part_o (B, QH, n, HD), part_ml (B, QH, n, 2))``: unnormalised outputs and (max, sum) per
    split, scores in log2 units.  Partials of several token ranges of one sequence can be
    concatenated along dim 2 and finished by flash_attention_combine."""
    lib = _l3lib.load()
    flags = _flags(flags)
    B, QH, KVH, S, HD = _check_qkv(query, keys, values)
    with _on_device(query.device):
        n_req = num_splits if num_splits > 0 else lib.l3_attn_choose_splits(B, KVH, S, HD, 0, flags)
        if n_req < 0:
            _fail(n_req)
        part_o = torch.empty((B, QH, n_req, HD), dtype=torch.float32, device=query.device)
        part_ml = torch.empty((B, QH, n_req, 2), dtype=torch.float32, device=query.device)
        n = lib.l3_attn_split(
            query.data_ptr(), keys.data_ptr(), values.data_ptr(), part_o.data_ptr(), part_ml.data_ptr(),
            B, QH, KVH, S, HD,
            _l3lib.i64_array((query.stride(0), query.stride(1))),
            _l3lib.i64_array((keys.stride(0), keys.stride(1), keys.stride(2))),
            _l3lib.i64_array((values.stride(0), values.stride(1), values.stride(2))),
            1.0 / math.sqrt(HD), num_splits, flags, _stream_ptr(query.device))
    if n < 0:
        _fail(n, f"B={B} QH={QH} KVH={KVH} S={S} HD={HD}")
    if n != n_req:  # the kernel laid its rows out for n splits: re-view the front of the buffers
        part_o = part_o.flatten()[: B * QH * n * HD].view(B, QH, n, HD)
        part_ml = part_ml.flatten()[: B * QH * n * 2].view(B, QH, n, 2)
    return part_o, part_ml


def flash_attention_combine(part_o, part_ml, dtype=torch.bfloat16):
    """Second stage on its own: log-sum-exp merge of (B, QH, n, HD) / (B, QH, n, 2) float32
    partials into a (B, QH, 1, HD) bf16 tensor laid out like empty_like of the model's query view."""
    lib = _l3lib.load()
    if not part_o.is_cuda or part_o.dtype != torch.float32 or part_ml.dtype != torch.float32:
        raise RuntimeError("partials must be float32 GPU tensors")
    B, QH, n, HD = part_o.shape
    if tuple(part_ml.shape) != (B, QH, n, 2):
        raise RuntimeError(f"part_ml is {tuple(part_ml.shape)}, expected {(B, QH, n, 2)}")
    po = part_o if part_o.is_contiguous() else part_o.contiguous()
    pm = part_ml if part_ml.is_contiguous() else part_ml.contiguous()
    out = torch.empty((B, 1, QH, HD), dtype=dtype, device=part_o.device).transpose(1, 2)
    with _on_device(part_o.device):
        rc = lib.l3_attn_combine(po.data_ptr(), pm.data_ptr(), out.data_ptr(), B, QH, HD, n,
                                 _l3lib.i64_array((out.stride(0), out.stride(1))), _stream_ptr(part_o.device))
    if rc != 0:
        _fail(rc, f"B={B} QH={QH} HD={HD} n={n}")
    return out


def flash_attention_decode_devlen(query, keys, values, kv_len, num_splits: int = 0, out=None, flags=None):
    """flash_attention_decode whose KV length is the int32 GPU scalar ``kv_len`` instead of the
    tensor shape: ``keys`` / ``values`` are (B, KVH, L, HD) views of the whole cache and only the
    first ``kv_len`` tokens are attended.  The launch does not depend on the length, so it can be
    captured once in a HIP graph and replayed while the cache grows (an extension; the reference
    takes the length from keys.size(2), custom_kernels.cu:246).  ``out`` may be supplied to keep
    the call allocation-free under capture."""
    lib = _l3lib.load()
    flags = _flags(flags)
    B, QH, KVH, L, HD = _check_qkv(query, keys, values)
    if keys.device != query.device or values.device != query.device:
        raise RuntimeError("query, keys and values must be on the same device")
    if not kv_len.is_cuda or kv_len.dtype != torch.int32 or kv_len.numel() != 1 or kv_len.device != query.device:
        raise RuntimeError("kv_len must be a one-element int32 tensor on the query's GPU")
    if out is None:
        out = torch.empty_like(query)
    else:
        _check_out(out, query, "flash_attention_decode_devlen")
    with _on_device(query.device):
        stream_ptr = _stream_ptr(query.device)
        ws, ws_bytes, flags = _attn_workspace(
            lib, query.device, stream_ptr, flags,
            lambda f: lib.l3_attn_decode_workspace_bytes(B, QH, KVH, L, HD, num_splits, f))
        rc = lib.l3_attn_decode_devlen(
            query.data_ptr(), keys.data_ptr(), values.data_ptr(), out.data_ptr(),
            ws.data_ptr() if ws is not None else None, ws_bytes, B, QH, KVH, L, HD,
            _l3lib.i64_array((query.stride(0), query.stride(1))),
            _l3lib.i64_array((keys.stride(0), keys.stride(1), keys.stride(2))),
            _l3lib.i64_array((values.stride(0), values.stride(1), values.stride(2))),
            _l3lib.i64_array((out.stride(0), out.stride(1))),
            1.0 / math.sqrt(HD), num_splits, flags, kv_len.data_ptr(), stream_ptr)
    if rc != 0:
        _fail(rc, f"B={B} QH={QH} KVH={KVH} L={L} HD={HD}")
    return out


def rot_embed_append(qkv, freq_table, cache_k, cache_v, pos, n_head: int, out=None):
    """Decode-step fusion of model.py:100-106 for one new token per sequence: rotates the query
    and key heads of ``qkv`` (B, 1, (n_head + 2*KVH)*HD, the fused projection in q|k|v order) with
    row ``pos`` of ``freq_table`` ((rows, HD) float32), writes the rotated keys and the values
    into ``cache_k`` / ``cache_v`` ((maxB, L, KVH, HD)) at token ``pos`` and returns the rotated
    queries (B, 1, n_head, HD).  ``pos`` is a one-element int32 GPU tensor read by the kernel, so
    the launch can be replayed from a HIP graph.  An extension of the reference's operator set."""
    lib = _l3lib.load()
    _require_gpu_bf16("qkv", qkv)
    _require_gpu_bf16("cache_k", cache_k)
    _require_gpu_bf16("cache_v", cache_v)
    if qkv.dim() != 3 or qkv.size(1) != 1 or qkv.stride(2) != 1:
        raise RuntimeError("qkv must be (B, 1, (n_head + 2*KVH)*HD) with a contiguous last dimension")
    if cache_k.dim() != 4 or cache_k.shape != cache_v.shape or cache_k.stride() != cache_v.stride():
        raise RuntimeError("cache_k and cache_v must be (maxB, L, KVH, HD) tensors of the same layout")
    maxB, L, KVH, HD = cache_k.shape
    B = qkv.size(0)
    if qkv.size(2) != (n_head + 2 * KVH) * HD or B > maxB:
        raise RuntimeError(f"qkv {tuple(qkv.shape)} does not match n_head={n_head}, cache {tuple(cache_k.shape)}")
    if cache_k.stride(3) != 1 or cache_k.stride(2) != HD:
        raise RuntimeError("the (KVH, HD) dimensions of the cache must be contiguous")
    if not freq_table.is_cuda or freq_table.dtype != torch.float32 or freq_table.dim() != 2 \
            or freq_table.size(1) != HD or not freq_table.is_contiguous():
        raise RuntimeError("freq_table must be a contiguous (rows, HD) float32 GPU tensor")
    if not pos.is_cuda or pos.dtype != torch.int32 or pos.numel() != 1 or pos.device != qkv.device:
        raise RuntimeError("pos must be a one-element int32 tensor on qkv's GPU")
    if cache_k.device != qkv.device or cache_v.device != qkv.device or freq_table.device != qkv.device:
        raise RuntimeError("qkv, freq_table and the caches must be on the same device")
    if out is None:
        out = torch.empty((B, 1, n_head, HD), dtype=qkv.dtype, device=qkv.device)
    elif not isinstance(out, torch.Tensor) or out.dtype != torch.bfloat16 or out.device != qkv.device \
            or tuple(out.shape) != (B, 1, n_head, HD) or not out.is_contiguous():
        raise RuntimeError(f"rot_embed_append: out must be a contiguous bf16 tensor of shape {(B, 1, n_head, HD)} "
                           f"on {qkv.device}")
    with _on_device(qkv.device):
        rc = lib.l3_rot_embed_append(qkv.data_ptr(), freq_table.data_ptr(), out.data_ptr(), cache_k.data_ptr(),
                                     cache_v.data_ptr(), pos.data_ptr(), B, n_head, KVH, HD, qkv.stride(0),
                                     _l3lib.i64_array((cache_k.stride(0), cache_k.stride(1))), L,
                                     freq_table.size(0), _stream_ptr(qkv.device))
    if rc != 0:
        _fail(rc, f"B={B} NH={n_head} KVH={KVH} HD={HD}")
    return out


def linear_qkv_rope_append(x, w_qkv, freq_table, cache_k, cache_v, pos, n_head: int, norm_weight=None,
                           eps: float = 1e-5):
    """linear_decode_fused(x, w_qkv, norm_weight) followed by rot_embed_append in one launch: the
    whole of model.py:95-106 for one new token per sequence.  x (B, 1, K); returns the rotated
    queries (B, 1, n_head, HD); keys and values are written into the caches at ``pos``."""
    lib = _l3lib.load()
    x2, rows, N, K = _linear_args(x, (w_qkv,))
    _require_gpu_bf16("cache_k", cache_k)
    _require_gpu_bf16("cache_v", cache_v)
    if cache_k.dim() != 4 or cache_k.shape != cache_v.shape or cache_k.stride() != cache_v.stride():
        raise RuntimeError("cache_k and cache_v must be (maxB, L, KVH, HD) tensors of the same layout")
    maxB, L, KVH, HD = cache_k.shape
    if N != (n_head + 2 * KVH) * HD or rows > maxB:
        raise RuntimeError(f"w_qkv {tuple(w_qkv.shape)} does not match n_head={n_head}, cache {tuple(cache_k.shape)}")
    if cache_k.stride(3) != 1 or cache_k.stride(2) != HD:
        raise RuntimeError("the (KVH, HD) dimensions of the cache must be contiguous")
    if not freq_table.is_cuda or freq_table.dtype != torch.float32 or freq_table.dim() != 2 \
            or freq_table.size(1) != HD or not freq_table.is_contiguous():
        raise RuntimeError("freq_table must be a contiguous (rows, HD) float32 GPU tensor")
    if not pos.is_cuda or pos.dtype != torch.int32 or pos.numel() != 1:
        raise RuntimeError("pos must be a one-element int32 GPU tensor")
    if norm_weight is not None:
        _require_gpu_bf16("norm_weight", norm_weight)
        if tuple(norm_weight.shape) != (K,) or not norm_weight.is_contiguous() \
                or rows > linear_decode_fused_max_rows(K):
            raise RuntimeError(f"linear_qkv_rope_append: norm_weight {tuple(norm_weight.shape)} / {rows} rows "
                               f"do not fit the fused input norm (K={K})")
    out = torch.empty((rows, 1, n_head, HD), dtype=x.dtype, device=x.device)
    with _on_device(x.device):
        rc = lib.l3_linear_qkv_rope_append(x2.data_ptr(), None if norm_weight is None else norm_weight.data_ptr(),
                                           float(eps), w_qkv.data_ptr(), freq_table.data_ptr(), out.data_ptr(),
                                           cache_k.data_ptr(), cache_v.data_ptr(), pos.data_ptr(), rows, n_head, KVH,
                                           HD, K, x2.stride(0), w_qkv.stride(0),
                                           _l3lib.i64_array((cache_k.stride(0), cache_k.stride(1))), L,
                                           freq_table.size(0), _stream_ptr(x.device))
    if rc != 0:
        _fail(rc, f"B={rows} NH={n_head} KVH={KVH} HD={HD} K={K}")
    return out


def rms_norm(input, weight, eps):
    """input (B, T, C) bf16, weight (C,) bf16 -> (B, T, C) bf16 (model.py:70-72)."""
    lib = _l3lib.load()
    _require_gpu_bf16("input", input)
    _require_gpu_bf16("weight", weight)
    if input.dim() != 3:
        raise RuntimeError("rms_norm expects a 3-D (B, T, C) input")
    C = input.size(2)
    if weight.numel() != C:
        raise RuntimeError(f"weight has {weight.numel()} elements, expected {C}")
    x = input if input.is_contiguous() else input.contiguous()
    w = weight if weight.is_contiguous() else weight.contiguous()
    out = torch.empty_like(x)
    rows = x.size(0) * x.size(1)
    if rows == 0:
        return out
    with _on_device(x.device):
        rc = lib.l3_rms_norm(x.data_ptr(), w.data_ptr(), out.data_ptr(), rows, C, float(eps),
                             _stream_ptr(x.device))
    if rc != 0:
        _fail(rc, f"rows={rows} C={C}")
    return out


def add_rms_norm(input, residual, weight, eps):
    """(input + residual, rms_norm(input + residual, weight, eps)) in one launch: the residual
    addition of model.py:147-148 fused with the norm that follows it.  Both outputs carry the same
    bits as ``s = input + residual`` (bf16) followed by ``rms_norm(s, weight, eps)``.  An extension
    of the reference's operator set."""
    lib = _l3lib.load()
    _require_gpu_bf16("input", input)
    _require_gpu_bf16("residual", residual)
    _require_gpu_bf16("weight", weight)
    if input.dim() != 3 or tuple(residual.shape) != tuple(input.shape):
        raise RuntimeError("add_rms_norm expects two (B, T, C) tensors of the same shape")
    C = input.size(2)
    if weight.numel() != C:
        raise RuntimeError(f"weight has {weight.numel()} elements, expected {C}")
    x = input if input.is_contiguous() else input.contiguous()
    r = residual if residual.is_contiguous() else residual.contiguous()
    w = weight if weight.is_contiguous() else weight.contiguous()
    s = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    rows = x.size(0) * x.size(1)
    if rows == 0:
        return s, y
    with _on_device(x.device):
        rc = lib.l3_add_rms_norm(x.data_ptr(), r.data_ptr(), w.data_ptr(), s.data_ptr(), y.data_ptr(), rows, C,
                                 float(eps), _stream_ptr(x.device))
    if rc != 0:
        _fail(rc, f"rows={rows} C={C}")
    return s, y


def silu_mul(a, b):
    """F.silu(a) * b for two bf16 tensors of the same shape in one launch (model.py:134), with the
    two roundings of the two torch kernels, so the bits are the same.  An extension."""
    lib = _l3lib.load()
    _require_gpu_bf16("a", a)
    _require_gpu_bf16("b", b)
    if tuple(a.shape) != tuple(b.shape):
        raise RuntimeError(f"silu_mul: shapes differ: {tuple(a.shape)} vs {tuple(b.shape)}")
    C = a.shape[-1] if a.dim() else 1
    rows = a.numel() // max(C, 1)
    strided = (a.dim() >= 1 and a.numel() > 0 and C % 8 == 0 and a.stride(-1) == 1 and b.stride(-1) == 1
               and not (a.is_contiguous() and b.is_contiguous()))
    if strided:
        # rows with a stride (the two halves of a fused gate|up projection): no copies
        a2, b2 = a.reshape(rows, C), b.reshape(rows, C)
        if a2.stride(1) == 1 and b2.stride(1) == 1 and a2.data_ptr() % 16 == 0 and b2.data_ptr() % 16 == 0 \
                and a2.stride(0) % 8 == 0 and b2.stride(0) % 8 == 0 and a2.data_ptr() == a.data_ptr() \
                and b2.data_ptr() == b.data_ptr():
            y = torch.empty(a.shape, dtype=a.dtype, device=a.device)
            with _on_device(a.device):
                rc = lib.l3_silu_mul_rows(a2.data_ptr(), b2.data_ptr(), y.data_ptr(), rows, C, max(a2.stride(0), C),
                                          max(b2.stride(0), C), _stream_ptr(a.device))
            if rc != 0:
                _fail(rc, f"rows={rows} cols={C}")
            return y
    ac = a if a.is_contiguous() else a.contiguous()
    bc = b if b.is_contiguous() else b.contiguous()
    y = torch.empty(ac.shape, dtype=ac.dtype, device=ac.device)
    if y.numel() == 0:
        return y
    with _on_device(ac.device):
        rc = lib.l3_silu_mul(ac.data_ptr(), bc.data_ptr(), y.data_ptr(), y.numel(), _stream_ptr(ac.device))
    if rc != 0:
        _fail(rc, f"n={y.numel()}")
    return y


def _linear_args(x, weights, max_rows=None):
    _require_gpu_bf16("x", x)
    K = x.shape[-1]
    rows = x.numel() // max(K, 1)
    max_rows = _l3lib.L3_LINEAR_MAX_ROWS if max_rows is None else max_rows
    if x.dim() < 1 or rows < 1 or rows > max_rows:
        raise RuntimeError(f"linear_decode: 1..{max_rows} activation rows expected, got {tuple(x.shape)}")
    w0 = weights[0]
    for w in weights:
        _require_gpu_bf16("weight", w)
        if w.dim() != 2 or w.shape[1] != K or w.stride(1) != 1 or \
                (w is not w0 and (w.shape[0] != w0.shape[0] or w.stride(0) != w0.stride(0))):
            raise RuntimeError(f"linear_decode: weight {tuple(w.shape)} does not fit x {tuple(x.shape)}")
    if x.dim() == 2 and x.stride(1) == 1:
        x2 = x                          # rows as they are (any row stride)
    elif x.is_contiguous():
        x2 = x.view(rows, K)
    else:
        x2 = x.reshape(rows, K)
        if x2.stride(1) != 1:
            x2 = x2.contiguous()
    return x2, rows, w0.shape[0], K


def _rows_out(x, rows: int, N: int):
    """A contiguous output of x's leading shape with N columns, (rows, N) to the kernel."""
    if x.dim() == 2:
        return x.new_empty((rows, N))
    return x.new_empty(x.shape[:-1] + (N,))


def _use_splitk(x, weight) -> bool:
    """17..64 activation rows: the split-K kernel plus its finishing pass (one launch serves up to 16)."""
    K = x.shape[-1]
    if K <= 0 or weight.dim() != 2 or not x.is_cuda:
        return False
    return _l3lib.L3_LINEAR_MAX_ROWS < x.numel() // K <= _l3lib.L3_LINEAR_SPLITK_MAX_ROWS


def linear_decode(x, weight):
    """F.linear(x, weight) for at most 64 activation rows (model.py:95,121,134,225 when T == 1):
    one pass over the weight matrix at HBM speed instead of a GEMM.  x (..., K), weight (N, K)
    -> (..., N).  Up to 16 rows are one launch whatever the matrix; 17..64 rows go through
    linear_splitk and linear_splitk_finish (N % 8 == 0, K % 128 == 0), which suits matrices of a
    few thousand rows -- a vocabulary projection at those batch sizes is a library GEMM's job.
    An extension."""
    lib = _l3lib.load()
    if _use_splitk(x, weight):
        return linear_splitk_finish(linear_splitk(x, weight)).view(*x.shape[:-1], weight.shape[0])
    x2, rows, N, K = _linear_args(x, (weight,))
    y = _rows_out(x, rows, N)
    with _on_device(x.device):
        rc = lib.l3_linear_decode(x2.data_ptr(), weight.data_ptr(), y.data_ptr(), rows, N, K, x2.stride(0),
                                  weight.stride(0), N, _stream_ptr(x.device))
    if rc != 0:
        _fail(rc, f"M={rows} N={N} K={K}")
    return y


def linear_swiglu_decode(x, w_gate, w_up):
    """F.silu(F.linear(x, w_gate)) * F.linear(x, w_up) for at most 16 activation rows in one
    launch (model.py:134 with w_gate = c_fc2, w_up = c_fc), same rounding points.  An extension."""
    lib = _l3lib.load()
    x2, rows, N, K = _linear_args(x, (w_gate, w_up))
    y = _rows_out(x, rows, N)
    with _on_device(x.device):
        rc = lib.l3_linear_swiglu_decode(x2.data_ptr(), w_gate.data_ptr(), w_up.data_ptr(), y.data_ptr(), rows, N, K,
                                         x2.stride(0), w_gate.stride(0), N, _stream_ptr(x.device))
    if rc != 0:
        _fail(rc, f"M={rows} N={N} K={K}")
    return y


def linear_decode_fused_max_rows(K: int) -> int:
    """Most activation rows of width K for which linear_decode_fused accepts a norm_weight."""
    return min(16, _l3lib.L3_LINEAR_STAGE_ELEMS // (K + 8)) if K % 512 == 0 else 0


def linear_decode_fused(x, weight, norm_weight=None, eps: float = 1e-5, w_up=None, residual=None):
    """linear_decode with the operators around it folded into the one launch, each optional:
    rms_norm(x, norm_weight, eps) in front (model.py:70-72), the SwiGLU product with a second
    matrix w_up (weight is then the gate, model.py:134), and `residual + result` behind
    (model.py:147-148) -- all with the rounding points of the separate operators.  An extension."""
    lib = _l3lib.load()
    if norm_weight is None and w_up is None and _use_splitk(x, weight):
        # 17..64 rows, small matrix: split-K, the residual joins when the splits are added up
        return linear_splitk_finish(linear_splitk(x, weight), residual).view(*x.shape[:-1], weight.shape[0])
    x2, rows, N, K = _linear_args(x, (weight,) if w_up is None else (weight, w_up))
    if norm_weight is not None:
        _require_gpu_bf16("norm_weight", norm_weight)
        if tuple(norm_weight.shape) != (K,) or not norm_weight.is_contiguous():
            raise RuntimeError(f"linear_decode_fused: norm_weight {tuple(norm_weight.shape)} does not fit K={K}")
        if rows > linear_decode_fused_max_rows(K):
            raise RuntimeError(f"linear_decode_fused: the input norm takes at most "
                               f"{linear_decode_fused_max_rows(K)} rows of width {K}, got {rows}")
    r2 = None
    if residual is not None:
        _require_gpu_bf16("residual", residual)
        if residual.numel() != rows * N or residual.shape[-1] != N:
            raise RuntimeError(f"linear_decode_fused: residual {tuple(residual.shape)} does not fit ({rows}, {N})")
        r2 = residual if residual.is_contiguous() else residual.reshape(rows, N).contiguous()
    y = _rows_out(x, rows, N)
    with _on_device(x.device):
        rc = lib.l3_linear_decode_fused(x2.data_ptr(), None if norm_weight is None else norm_weight.data_ptr(),
                                        float(eps), weight.data_ptr(), None if w_up is None else w_up.data_ptr(),
                                        None if r2 is None else r2.data_ptr(), y.data_ptr(), rows, N, K,
                                        x2.stride(0), weight.stride(0), N, _stream_ptr(x.device))
    if rc != 0:
        _fail(rc, f"M={rows} N={N} K={K}")
    return y


def linear_splitk(x, weight, ksplit: int = 0):
    """x (..., K) with 17..64 rows times weight (N, K)^T as float32 partial products
    (ksplit, rows, N) -- NOT added up: hand them to add_rms_norm_partials or
    rot_embed_append_partials, which sum the splits on their way (or sum them yourself).
    ksplit 0 lets the library choose.  Stands for nn.Linear at batch sizes where the activations no
    longer fit one matrix-instruction column block (model.py:95,121,134).  An extension."""
    lib = _l3lib.load()
    x2, rows, N, K = _linear_args(x, (weight,), _l3lib.L3_LINEAR_SPLITK_MAX_ROWS)
    with _on_device(x.device):
        if ksplit <= 0:
            ksplit = lib.l3_linear_splitk_plan(N, K, _cus(x.device))
            if ksplit < 0:
                _fail(ksplit, f"N={N} K={K}")
        part = torch.empty((ksplit, rows, N), dtype=torch.float32, device=x.device)
        rc = lib.l3_linear_splitk(x2.data_ptr(), weight.data_ptr(), part.data_ptr(), part.numel() * 4, rows, N, K,
                                  x2.stride(0), weight.stride(0), ksplit, _stream_ptr(x.device))
    if rc != 0:
        _fail(rc, f"M={rows} N={N} K={K} ksplit={ksplit}")
    return part


def linear_splitk_finish(part, residual=None):
    """bf16(part.sum(0)) for linear_splitk's partial products (ksplit, rows, N), summed in split
    order and rounded once -- what the unsplit linear would have returned -- plus ``residual``
    (rows x N, bf16) with the rounding of a separate addition if given.  Returns (rows, N)."""
    lib = _l3lib.load()
    if not part.is_cuda or part.dtype != torch.float32 or part.dim() != 3 or not part.is_contiguous():
        raise RuntimeError("linear_splitk_finish: expected contiguous float32 (ksplit, rows, N) partials")
    ksplit, rows, N = part.shape
    r2 = None
    if residual is not None:
        _require_gpu_bf16("residual", residual)
        if residual.numel() != rows * N or residual.shape[-1] != N:
            raise RuntimeError(f"linear_splitk_finish: residual {tuple(residual.shape)} does not fit ({rows}, {N})")
        r2 = residual.reshape(rows, N)
        if not r2.is_contiguous():
            r2 = r2.contiguous()
    y = torch.empty((rows, N), dtype=torch.bfloat16, device=part.device)
    with _on_device(part.device):
        rc = lib.l3_linear_splitk_finish(part.data_ptr(), ksplit, None if r2 is None else r2.data_ptr(), y.data_ptr(),
                                         rows, N, N, _stream_ptr(part.device))
    if rc != 0:
        _fail(rc, f"rows={rows} N={N} ksplit={ksplit}")
    return y


def add_rms_norm_partials(input, part, weight, eps):
    """add_rms_norm(input, r, weight, eps) with r = bf16(part.sum(0)) formed inside the kernel:
    ``part`` is linear_splitk's output for the linear whose result is the residual branch
    (model.py:147-148).  Returns (input + r, rms_norm(input + r))."""
    lib = _l3lib.load()
    _require_gpu_bf16("input", input)
    _require_gpu_bf16("weight", weight)
    C = input.shape[-1]
    rows = input.numel() // C
    if not part.is_cuda or part.dtype != torch.float32 or part.dim() != 3 or not part.is_contiguous() \
            or tuple(part.shape[1:]) != (rows, C):
        raise RuntimeError(f"add_rms_norm_partials: partials {tuple(part.shape)} do not fit input {tuple(input.shape)}")
    if weight.numel() != C or not weight.is_contiguous():
        raise RuntimeError(f"weight has {weight.numel()} elements, expected {C}")
    x = input if input.is_contiguous() else input.contiguous()
    s = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    with _on_device(x.device):
        rc = lib.l3_add_rms_norm_partials(x.data_ptr(), part.data_ptr(), part.shape[0], weight.data_ptr(),
                                          s.data_ptr(), y.data_ptr(), rows, C, float(eps), _stream_ptr(x.device))
    if rc != 0:
        _fail(rc, f"rows={rows} C={C} ksplit={part.shape[0]}")
    return s, y


def rot_embed_append_partials(part, freq_table, cache_k, cache_v, pos, n_head: int):
    """rot_embed_append on a fused qkv projection that is still in linear_splitk's partial
    products (ksplit, B, (n_head + 2*KVH)*HD): summed, rounded to bf16, rotated, appended."""
    lib = _l3lib.load()
    _require_gpu_bf16("cache_k", cache_k)
    _require_gpu_bf16("cache_v", cache_v)
    if cache_k.dim() != 4 or cache_k.shape != cache_v.shape or cache_k.stride() != cache_v.stride():
        raise RuntimeError("cache_k and cache_v must be (maxB, L, KVH, HD) tensors of the same layout")
    maxB, L, KVH, HD = cache_k.shape
    if not part.is_cuda or part.dtype != torch.float32 or part.dim() != 3 or not part.is_contiguous():
        raise RuntimeError("rot_embed_append_partials: expected contiguous float32 (ksplit, B, N) partials")
    ksplit, B, N = part.shape
    if N != (n_head + 2 * KVH) * HD or B > maxB:
        raise RuntimeError(f"partials {tuple(part.shape)} do not match n_head={n_head}, cache {tuple(cache_k.shape)}")
    if cache_k.stride(3) != 1 or cache_k.stride(2) != HD:
        raise RuntimeError("the (KVH, HD) dimensions of the cache must be contiguous")
    if not freq_table.is_cuda or freq_table.dtype != torch.float32 or freq_table.dim() != 2 \
            or freq_table.size(1) != HD or not freq_table.is_contiguous():
        raise RuntimeError("freq_table must be a contiguous (rows, HD) float32 GPU tensor")
    if not pos.is_cuda or pos.dtype != torch.int32 or pos.numel() != 1:
        raise RuntimeError("pos must be a one-element int32 GPU tensor")
    out = torch.empty((B, 1, n_head, HD), dtype=cache_k.dtype, device=part.device)
    with _on_device(part.device):
        rc = lib.l3_rot_embed_append_partials(part.data_ptr(), ksplit, freq_table.data_ptr(), out.data_ptr(),
                                              cache_k.data_ptr(), cache_v.data_ptr(), pos.data_ptr(), B, n_head, KVH,
                                              HD, _l3lib.i64_array((cache_k.stride(0), cache_k.stride(1))), L,
                                              freq_table.size(0), _stream_ptr(part.device))
    if rc != 0:
        _fail(rc, f"B={B} NH={n_head} KVH={KVH} HD={HD} ksplit={ksplit}")
    return out


def argmax(logits):
    """Index of the first maximum along the last dimension of a 2-D bf16 tensor (rows, V), as
    int64 -- torch.argmax(logits.float(), dim=-1) for the greedy pick of model.py:371 (the float
    conversion of model.py:225 is monotone, so it is skipped).  An extension."""
    lib = _l3lib.load()
    _require_gpu_bf16("logits", logits)
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise RuntimeError("argmax expects a 2-D (rows, V) tensor with a contiguous last dimension")
    rows, V = logits.shape
    out = torch.empty(rows, dtype=torch.int64, device=logits.device)
    if rows == 0:
        return out
    with _on_device(logits.device):
        ws_bytes = lib.l3_argmax_workspace_bytes(rows, V)
        stream_ptr = _stream_ptr(logits.device)
        ws = _workspace(logits.device, stream_ptr, ws_bytes)
        rc = lib.l3_argmax(logits.data_ptr(), logits.stride(0), rows, V, ws.data_ptr(), ws_bytes, out.data_ptr(),
                           stream_ptr)
    if rc != 0:
        _fail(rc, f"rows={rows} V={V}")
    return out


def greedy_step(logits, tokens, text_mask, tok, pos, kv_len, eos, stop_tokens):
    """The tail of one greedy decoding step, in place and on the device (model.py:371-378): pick
    argmax(logits[b]) unless position pos + 1 still belongs to the prompt (text_mask), store the
    token into tokens[:, pos + 1] and tok, mark rows that produced a stop token in eos, and
    advance pos and kv_len by one.  logits (rows, V) bf16; tokens (rows, L) int64; text_mask
    (rows, L) bool; tok (rows, 1) or (rows,) int64; pos, kv_len int32 scalars; eos (rows) bool;
    stop_tokens int64.  An extension."""
    lib = _l3lib.load()
    _require_gpu_bf16("logits", logits)
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise RuntimeError("greedy_step expects (rows, V) logits with a contiguous last dimension")
    rows, V = logits.shape
    L = tokens.shape[1]
    ok = (tokens.dtype == torch.int64 and tokens.is_contiguous() and tokens.shape[0] == rows
          and text_mask.dtype == torch.bool and text_mask.is_contiguous() and tuple(text_mask.shape) == (rows, L)
          and tok.dtype == torch.int64 and tok.is_contiguous() and tok.numel() == rows
          and pos.dtype == torch.int32 and pos.numel() == 1 and kv_len.dtype == torch.int32 and kv_len.numel() == 1
          and eos.dtype == torch.bool and eos.is_contiguous() and eos.numel() == rows
          and stop_tokens.dtype == torch.int64 and stop_tokens.is_contiguous())
    if not ok or any(t.device != logits.device for t in (tokens, text_mask, tok, pos, kv_len, eos, stop_tokens)):
        raise RuntimeError("greedy_step: state tensors have the wrong dtype, shape, layout or device")
    with _on_device(logits.device):
        ws_bytes = lib.l3_argmax_workspace_bytes(rows, V)
        stream_ptr = _stream_ptr(logits.device)
        ws = _workspace(logits.device, stream_ptr, ws_bytes)
        rc = lib.l3_greedy_step(logits.data_ptr(), logits.stride(0), rows, V, ws.data_ptr(), ws_bytes,
                                tokens.data_ptr(), text_mask.data_ptr(), L, tok.data_ptr(), pos.data_ptr(),
                                kv_len.data_ptr(), eos.data_ptr(), stop_tokens.data_ptr(), stop_tokens.numel(),
                                stream_ptr)
    if rc != 0:
        _fail(rc, f"rows={rows} V={V}")


def rot_embed(input, freq):
    """input (B, T, NH, HD) bf16 (any strides on the first three dims), freq (T, HD) float32
    interleaved cos/sin -> contiguous (B, T, NH, HD) bf16 (model.py:100-101)."""
    lib = _l3lib.load()
    _require_gpu_bf16("input", input)
    if not freq.is_cuda or freq.dtype != torch.float32:
        raise RuntimeError(f"expected a GPU float32 freq table but found {freq.dtype} on {freq.device}")
    if input.dim() != 4 or freq.dim() != 2:
        raise RuntimeError("rot_embed expects a 4-D (B, T, NH, HD) input and a 2-D (T, HD) freq table")
    B, T, NH, HD = input.shape
    if freq.size(0) != T or freq.size(1) != HD:
        raise RuntimeError(f"freq is {tuple(freq.shape)}, expected {(T, HD)}")
    if input.stride(3) != 1:
        raise RuntimeError("the head dimension of input must be contiguous")
    f = freq if freq.is_contiguous() else freq.contiguous()
    out = input.new_empty((B, T, NH, HD))
    if out.numel() == 0:
        return out
    with _on_device(input.device):
        rc = lib.l3_rot_embed(input.data_ptr(), f.data_ptr(), out.data_ptr(), B, T, NH, HD,
                              _l3lib.i64_array((input.stride(0), input.stride(1), input.stride(2))),
                              _stream_ptr(input.device))
    if rc != 0:
        _fail(rc, f"B={B} T={T} NH={NH} HD={HD} strides={tuple(input.stride())}")
    return out
