"""The C-ABI library without a GPU: it loads, exports every symbol include/l3_kernels.h
declares, rejects bad arguments before any launch, and plans splits sanely."""

import ctypes
import os
import re
import shutil
import subprocess

import pytest

from custom_kernels import _l3lib
from custom_kernels import custom_kernels_extension as cke

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "l3_kernels.h")
FAKE = 0x7F0000001000  # 4 KiB-aligned non-null address that is never dereferenced on the host


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(l3_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    lib = _l3lib.load()
    names = _declared()
    assert names == sorted(_l3lib.SIGNATURES), "header and ctypes table disagree"
    for n in names:
        assert getattr(lib, n) is not None
    assert lib.l3_version() >= 100


C_CALLER = r"""
#include <stdio.h>
#include "l3_kernels.h"

int main(void) {
    /* host-logic entry points only: nothing here touches a GPU */
    if (l3_version() < 100) return 1;
    if (l3_attn_choose_splits(1, 8, 32768, 128, 256, 0) < 2) return 2;
    if (l3_attn_choose_splits(1, 8, 32768, 96, 256, 0) != L3_ERR_HEAD_SIZE) return 3;
    if (l3_attn_decode_workspace_bytes(1, 32, 8, 32768, 128, 4, L3_ATTN_FLAG_KERNEL_FMA) !=
        (size_t)(4 * 32 * 128 * 4 + 4 * 32 * 8)) return 4;
    if (l3_attn_choose_splits(1, 8, 32768, 128, 256, 0x4000) != L3_ERR_FLAGS) return 6;
    if (l3_rms_norm(0, 0, 0, 1, 2048, 1e-5f, 0) != L3_ERR_NULL_POINTER) return 5;
    printf("%s\n", l3_strerror(L3_ERR_HEAD_RATIO));
    return 0;
}
"""


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs a C compiler")
def test_header_is_plain_c_and_a_c_program_links_against_the_library(tmp_path):
    """What a maintainer binding the library from C (or cgo, JNI ...) relies on: the header compiles as
    C99 with nothing but the standard headers, and a C program linked against the library reaches the
    entry points by their undecorated names."""
    lib_path = _l3lib.library_path()
    src = tmp_path / "caller.c"
    src.write_text(C_CALLER)
    exe = tmp_path / "caller"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.dirname(HEADER), str(src),
                    "-o", str(exe), lib_path, "-Wl,-rpath," + os.path.dirname(lib_path)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    assert "Unsupported QKV head ratio" in out


def test_error_codes_match_header():
    text = open(HEADER).read()
    for name, val in re.findall(r"(L3_(?:OK|ERR_[A-Z_]+))\s*=\s*(-?\d+)", text):
        assert getattr(_l3lib, name) == int(val)
        assert _l3lib.strerror(int(val))
    assert int(re.search(r"#define L3_ATTN_MAX_SPLITS (\d+)", text).group(1)) == _l3lib.L3_ATTN_MAX_SPLITS
    assert int(re.search(r"#define L3_LINEAR_MAX_ROWS (\d+)", text).group(1)) == _l3lib.L3_LINEAR_MAX_ROWS
    for name, val in re.findall(r"#define (L3_ATTN_FLAG_[A-Z_]+) (0x[0-9a-fA-F]+)", text):
        assert getattr(_l3lib, name) == int(val, 16)
    assert int(re.search(r"#define L3_ATTN_STATIC_SCRATCH_BYTES \((\d+)u << (\d+)\)", text).group(1)) << 20 \
        == _l3lib.L3_ATTN_STATIC_SCRATCH_BYTES
    assert "unknown" in _l3lib.strerror(-12345)


def _attn(q=FAKE, k=FAKE, v=FAKE, out=FAKE, ws=None, ws_bytes=0, B=1, QH=32, KVH=8, S=256, HD=64,
          qs=(2048, 64), ks=(131072, 64, 512), vs=(131072, 64, 512), os_=(2048, 64), splits=1, flags=0, scale=0.125):
    return _l3lib.load().l3_attn_decode(q, k, v, out, ws, ws_bytes, B, QH, KVH, S, HD, _l3lib.i64_array(qs),
                                        _l3lib.i64_array(ks), _l3lib.i64_array(vs), _l3lib.i64_array(os_),
                                        scale, splits, flags, None)


def test_attention_argument_checks_run_before_any_launch():
    assert _attn(q=None) == _l3lib.L3_ERR_NULL_POINTER
    assert _attn(out=None) == _l3lib.L3_ERR_NULL_POINTER
    assert _attn(HD=96) == _l3lib.L3_ERR_HEAD_SIZE           # custom_kernels.cu:317-319
    assert _attn(HD=256) == _l3lib.L3_ERR_HEAD_SIZE
    assert _attn(QH=40, KVH=8) == _l3lib.L3_ERR_HEAD_RATIO   # ratio 5: custom_kernels.cu:289-291
    assert _attn(QH=30, KVH=8) == _l3lib.L3_ERR_SHAPE
    assert _attn(S=0) == _l3lib.L3_ERR_SHAPE
    assert _attn(B=-1) == _l3lib.L3_ERR_SHAPE
    assert _attn(splits=-1) == _l3lib.L3_ERR_SPLITS
    assert _attn(splits=_l3lib.L3_ATTN_MAX_SPLITS + 1) == _l3lib.L3_ERR_SPLITS
    assert _attn(ks=(131072, 64, 516)) == _l3lib.L3_ERR_STRIDE      # rows off 16-byte boundaries
    assert _attn(vs=(131072, 60, 512)) == _l3lib.L3_ERR_STRIDE
    assert _attn(qs=(2048, -64)) == _l3lib.L3_ERR_STRIDE
    assert _attn(k=FAKE + 2) == _l3lib.L3_ERR_ALIGNMENT
    assert _attn(flags=0x100) == _l3lib.L3_ERR_FLAGS
    assert _attn(flags=-1) == _l3lib.L3_ERR_FLAGS
    for bad in (0.0, -0.125, float("nan"), float("inf")):     # the kernels scale a maximum of raw scores
        assert _attn(scale=bad) == _l3lib.L3_ERR_SCALE
    assert _attn(S=1024, ks=(524288, 64, 512), vs=(524288, 64, 512), splits=4) == _l3lib.L3_ERR_WORKSPACE
    assert _attn(S=1024, ks=(524288, 64, 512), vs=(524288, 64, 512), splits=4, ws=FAKE, ws_bytes=16) \
        == _l3lib.L3_ERR_WORKSPACE
    need = _l3lib.load().l3_attn_decode_workspace_bytes(1, 32, 8, 1024, 64, 4, 0)
    assert _attn(S=1024, ks=(524288, 64, 512), vs=(524288, 64, 512), splits=4, ws=FAKE + 64, ws_bytes=need) \
        == _l3lib.L3_ERR_ALIGNMENT


def test_rms_norm_and_rot_embed_argument_checks():
    lib = _l3lib.load()
    assert lib.l3_rms_norm(None, FAKE, FAKE, 4, 2048, 1e-5, None) == _l3lib.L3_ERR_NULL_POINTER
    assert lib.l3_rms_norm(FAKE, FAKE, FAKE, 0, 2048, 1e-5, None) == _l3lib.L3_ERR_SHAPE
    assert lib.l3_rms_norm(FAKE, FAKE, FAKE, 4, 0, 1e-5, None) == _l3lib.L3_ERR_SHAPE
    assert lib.l3_rms_norm(FAKE + 1, FAKE, FAKE, 4, 2048, 1e-5, None) == _l3lib.L3_ERR_ALIGNMENT
    st = _l3lib.i64_array((3072 * 5, 3072, 64))
    assert lib.l3_rot_embed(FAKE, None, FAKE, 1, 5, 32, 64, st, None) == _l3lib.L3_ERR_NULL_POINTER
    assert lib.l3_rot_embed(FAKE, FAKE, FAKE, 1, 5, 32, 63, st, None) == _l3lib.L3_ERR_SHAPE
    assert lib.l3_rot_embed(FAKE, FAKE, FAKE, 1, 0, 32, 64, st, None) == _l3lib.L3_ERR_SHAPE
    assert lib.l3_rot_embed(FAKE, FAKE, FAKE, 1, 5, 32, 64, _l3lib.i64_array((15360, 3071, 64)), None) \
        == _l3lib.L3_ERR_STRIDE
    assert lib.l3_rot_embed(FAKE + 2, FAKE, FAKE, 1, 5, 32, 64, st, None) == _l3lib.L3_ERR_ALIGNMENT


def test_split_plan_invariants_over_random_shapes():
    """Whatever the shape, the device size or the kernel: between one split and one per tile, never above the
    limit, the same answer twice, and a workspace that holds exactly the partial rows of that many splits."""
    import random

    lib = _l3lib.load()
    rng = random.Random(7)
    fma = _l3lib.L3_ATTN_FLAG_KERNEL_FMA
    for _ in range(3000):
        HD = rng.choice((64, 128))
        KVH = rng.choice((1, 2, 3, 4, 8, 16, 32))
        R = rng.choice((1, 2, 3, 4, 8))
        B = rng.choice((1, 1, 2, 3, 7, 8, 16, 33, 64, 100, 256, 1000))
        S = rng.choice((1, 31, 64, 100, 256, 257, 448, 512, 1000, 4096, 5000, 16384, 32768, 100000, 131072))
        cus = rng.choice((64, 104, 256, 304))
        flags = rng.choice((0, 0, 0, fma))
        n = lib.l3_attn_choose_splits(B, KVH, S, HD, cus, flags)
        what = f"B={B} KVH={KVH} S={S} HD={HD} cus={cus} flags={flags}: {n}"
        assert 1 <= n <= _l3lib.L3_ATTN_MAX_SPLITS, what
        assert n <= max(1, -(-S // 16)), what                      # no kernel's tile is shorter than 16 tokens
        assert n == lib.l3_attn_choose_splits(B, KVH, S, HD, cus, flags), what
        ws = lib.l3_attn_decode_workspace_bytes(B, KVH * R, KVH, S, HD, n, flags)
        rows = B * KVH * R * n
        assert (ws == 0 if n == 1 else rows * (HD + 2) * 4 <= ws <= rows * (HD + 2) * 4 + 512), what


def test_split_planning():
    lib = _l3lib.load()
    for HD, tile in ((64, 64), (128, 32)):
        prev = 0
        for S in (1, 63, 64, 65, 256, 512, 1000, 4096, 32768, 131072):
            n = lib.l3_attn_choose_splits(1, 8, S, HD, 256, 0)
            assert 1 <= n <= _l3lib.L3_ATTN_MAX_SPLITS
            assert n <= max(1, -(-S // tile)), "no split shorter than one workgroup tile"
            assert n >= prev, "more tokens never means fewer splits at fixed batch"
            prev = n
            ws = lib.l3_attn_decode_workspace_bytes(1, 32, 8, S, HD, 0, 0)
            if n == 1:
                assert ws == 0
            else:
                rows = 32 * n
                assert rows * (HD + 2) * 4 <= ws <= rows * (HD + 2) * 4 + 512
        # enough (batch, kv head) pairs to fill the device: no split, no combine
        assert lib.l3_attn_choose_splits(256, 8, 256, HD, 256, 0) == 1
        # the device size matters
        assert lib.l3_attn_choose_splits(1, 8, 32768, HD, 64, 0) < lib.l3_attn_choose_splits(1, 8, 32768, HD, 256, 0)
    # many sequences (8 kv heads: one workgroup per sequence and split group, 256 units):
    plan = lambda B, S, HD: lib.l3_attn_choose_splits(B, 8, S, HD, 256, 0)  # noqa: E731
    assert plan(3, 32768, 128) == 64            # four fifths of the units (68 groups of 3 workgroups at most), whole tiles: 64 x 512 tokens
    assert plan(1, 32768, 128) == 205 and plan(1, 16384, 128) == 171   # 5 and 3 tiles per wavefront
    assert plan(1, 12288, 128) == 32 and plan(1, 8192, 64) == 32       # cooperative form: one workgroup per unit
    assert plan(1, 256, 64) == 1 and plan(1, 384, 64) == 1 and plan(1, 448, 64) == 4 and plan(1, 512, 64) == 4   # one launch up to six tiles
    assert plan(1, 256, 128) == 1 and plan(1, 512, 128) == 8
    assert plan(4, 4096, 64) == 64              # few sequences: one workgroup per unit
    assert plan(16, 4096, 64) == 11             # from 8 sequences on, three quarters of the units: 12 groups, whole tiles
    assert plan(16, 1024, 64) == 16             # 16 tiles over 12 groups would round to 8 splits, half the units: one tile each instead
    assert plan(8, 2048, 64) == 32
    assert plan(48, 4096, 128) == 4
    assert plan(64, 4096, 128) == 3
    assert plan(96, 2048, 64) == 2
    assert plan(96, 512, 64) == 1               # short streams at a quarter of the units or more: no combine
    assert plan(128, 128, 64) == 1 and plan(192, 1024, 128) == 1
    assert plan(100, 4096, 128) == 2            # a long stream is worth the second group
    assert lib.l3_attn_choose_splits(1, 8, 256, 96, 256, 0) == _l3lib.L3_ERR_HEAD_SIZE
    assert lib.l3_attn_choose_splits(0, 8, 256, 64, 256, 0) == _l3lib.L3_ERR_SHAPE
    assert cke.attention_num_splits(16, 8, 4096, 64) == lib.l3_attn_choose_splits(16, 8, 4096, 64, 256, 0)
    # an explicit request is honoured up to what the length allows
    assert lib.l3_attn_decode_workspace_bytes(1, 32, 8, 4096, 128, 7, 0) == 32 * 7 * 128 * 4 + 32 * 7 * 8
    # the plan belongs to the call: the FMA kernel's differs, and the shim's context carries the flag per thread
    fma = _l3lib.L3_ATTN_FLAG_KERNEL_FMA
    assert lib.l3_attn_choose_splits(16, 8, 4096, 64, 256, fma) != lib.l3_attn_choose_splits(16, 8, 4096, 64, 256, 0)
    with cke.attention_flags(kernel="fma"):
        assert cke.attention_num_splits(16, 8, 4096, 64) == lib.l3_attn_choose_splits(16, 8, 4096, 64, 256, fma)
    assert cke.attention_num_splits(16, 8, 4096, 64) == 11


def test_attention_flag_contexts_nest():
    """A block that names one choice keeps what the enclosing block chose for the others."""
    from custom_kernels.custom_kernels_extension import _attn_flags

    fma, tiled, two = _l3lib.L3_ATTN_FLAG_KERNEL_FMA, _l3lib.L3_ATTN_FLAG_PREFILL_TILED, _l3lib.L3_ATTN_FLAG_TWO_LAUNCHES
    assert _attn_flags.get() == 0
    with cke.attention_flags(kernel="fma"):
        with cke.attention_flags(prefill="tiled"):
            assert _attn_flags.get() == fma | tiled
            with cke.attention_flags(kernel="mfma", launches="two"):
                assert _attn_flags.get() == tiled | two
            assert _attn_flags.get() == fma | tiled
        assert _attn_flags.get() == fma
    with cke.attention_flags(prefill="wave"):
        with cke.attention_flags(kernel="fma"):
            assert _attn_flags.get() == fma | _l3lib.L3_ATTN_FLAG_PREFILL_WAVE
    assert _attn_flags.get() == 0


def test_single_launch_entry_points_argument_checks():
    lib = _l3lib.load()
    W, TWO, COOP = _l3lib.L3_ATTN_FLAG_WS_COUNTERS, _l3lib.L3_ATTN_FLAG_TWO_LAUNCHES, _l3lib.L3_ATTN_FLAG_FORM_COOP
    assert lib.l3_attn_workspace_init(None, 1 << 20, None) == _l3lib.L3_ERR_NULL_POINTER
    assert lib.l3_attn_workspace_init(FAKE, _l3lib.L3_ATTN_COUNTER_BYTES - 1, None) == _l3lib.L3_ERR_WORKSPACE
    assert lib.l3_attn_workspace_init(FAKE + 8, 1 << 20, None) == _l3lib.L3_ERR_ALIGNMENT
    # the counters come on top of the partials, and only when the plan has more than one split
    base = lib.l3_attn_decode_workspace_bytes(1, 32, 8, 4096, 128, 7, 0)
    assert lib.l3_attn_decode_workspace_bytes(1, 32, 8, 4096, 128, 7, W) == base + _l3lib.L3_ATTN_COUNTER_BYTES
    assert lib.l3_attn_decode_workspace_bytes(1, 32, 8, 200, 64, 1, W) == 0
    # with the counters the plan keeps cooperative workgroups (at most 32 splits) where it used to stream
    assert lib.l3_attn_choose_splits(1, 8, 16384, 128, 256, 0) == 171
    assert lib.l3_attn_choose_splits(1, 8, 16384, 128, 256, W) == 32
    assert lib.l3_attn_choose_splits(1, 8, 16384, 128, 256, W | TWO) == 171
    assert lib.l3_attn_choose_splits(1, 3, 16384, 128, 256, W) == lib.l3_attn_choose_splits(1, 3, 16384, 128, 256, 0)
    # no device has been probed in this process: two launches whatever the flags; one split is one launch
    assert lib.l3_attn_launches(1, 32, 8, 4096, 128, 0, W) == 2
    assert lib.l3_attn_launches(1, 32, 8, 200, 64, 0, W) == 1
    assert lib.l3_attn_launches(1, 32, 8, 4096, 128, 600, W) == _l3lib.L3_ERR_SPLITS
    assert lib.l3_attn_launches(1, 32, 8, 4096, 128, 4, COOP | _l3lib.L3_ATTN_FLAG_FORM_STREAM) == _l3lib.L3_ERR_FLAGS
    assert lib.l3_attn_merge_in_launch_available() == 0


def test_shim_rejects_cpu_tensors_and_has_no_fallback():
    import torch

    x = torch.zeros(1, 1, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        cke.rms_norm(x, torch.ones(64, dtype=torch.bfloat16), 1e-5)
    with pytest.raises(RuntimeError, match="GPU"):
        cke.rot_embed(torch.zeros(1, 1, 1, 64, dtype=torch.bfloat16), torch.zeros(1, 64))
    with pytest.raises(RuntimeError, match="GPU"):
        cke.flash_attention_decode(torch.zeros(1, 4, 1, 64, dtype=torch.bfloat16),
                                   torch.zeros(1, 4, 8, 64, dtype=torch.bfloat16),
                                   torch.zeros(1, 4, 8, 64, dtype=torch.bfloat16))


def test_missing_library_raises(monkeypatch, tmp_path):
    monkeypatch.setenv("L3_KERNELS_LIB", str(tmp_path / "nope.so"))
    monkeypatch.setattr(_l3lib, "_lib", None)
    with pytest.raises(ImportError, match="no fallback"):
        _l3lib.load()


def test_stage_entry_points_argument_checks():
    lib = _l3lib.load()
    qs, ks = _l3lib.i64_array((2048, 64)), _l3lib.i64_array((131072, 64, 512))
    assert lib.l3_attn_split(FAKE, FAKE, FAKE, None, FAKE, 1, 32, 8, 256, 64, qs, ks, ks, 0.125, 1, 0, None) \
        == _l3lib.L3_ERR_NULL_POINTER
    assert lib.l3_attn_split(FAKE, FAKE, FAKE, FAKE, FAKE, 1, 32, 8, 256, 80, qs, ks, ks, 0.125, 1, 0, None) \
        == _l3lib.L3_ERR_HEAD_SIZE
    assert lib.l3_attn_split(FAKE, FAKE, FAKE, FAKE + 4, FAKE, 1, 32, 8, 256, 64, qs, ks, ks, 0.125, 1, 0, None) \
        == _l3lib.L3_ERR_ALIGNMENT
    assert lib.l3_attn_split(FAKE, FAKE, FAKE, FAKE, FAKE, 1, 32, 8, 256, 64, qs, ks, ks, 0.125, 1, 0x80, None) \
        == _l3lib.L3_ERR_FLAGS
    assert lib.l3_attn_combine(FAKE, FAKE, None, 1, 32, 64, 4, qs, None) == _l3lib.L3_ERR_NULL_POINTER
    assert lib.l3_attn_combine(FAKE, FAKE, FAKE, 1, 32, 96, 4, qs, None) == _l3lib.L3_ERR_HEAD_SIZE
    assert lib.l3_attn_combine(FAKE, FAKE, FAKE, 1, 32, 64, 0, qs, None) == _l3lib.L3_ERR_SPLITS
    assert lib.l3_attn_combine(FAKE, FAKE, FAKE, 1, 32, 64, 513, qs, None) == _l3lib.L3_ERR_SPLITS
    assert lib.l3_attn_combine(FAKE, FAKE, FAKE, 0, 32, 64, 4, qs, None) == _l3lib.L3_ERR_SHAPE
    assert lib.l3_attn_combine(FAKE, FAKE, FAKE, 2, 32, 64, 4, _l3lib.i64_array((2049, 64)), None) \
        == _l3lib.L3_ERR_STRIDE


def test_prefill_argument_checks():
    lib = _l3lib.load()
    qs, ks = _l3lib.i64_array((131072, 64, 2048)), _l3lib.i64_array((131072, 64, 512))

    def call(q=FAKE, out=FAKE, B=1, QH=32, KVH=8, T=16, S=64, HD=64, q_strides=qs, k_strides=ks, flags=0, scale=0.125):
        return lib.l3_attn_prefill(q, FAKE, FAKE, out, B, QH, KVH, T, S, HD, q_strides, k_strides, k_strides,
                                   q_strides, scale, flags, None)

    assert call(scale=0.0) == _l3lib.L3_ERR_SCALE

    assert call(flags=0x80) == _l3lib.L3_ERR_FLAGS
    assert call(flags=0xc) == _l3lib.L3_ERR_FLAGS           # both form bits
    assert call(out=None) == _l3lib.L3_ERR_NULL_POINTER
    assert call(HD=96) == _l3lib.L3_ERR_HEAD_SIZE
    assert call(QH=40) == _l3lib.L3_ERR_HEAD_RATIO      # ratio 5
    assert call(QH=30) == _l3lib.L3_ERR_SHAPE           # not a multiple of KVH
    assert call(T=0) == _l3lib.L3_ERR_SHAPE
    assert call(T=65) == _l3lib.L3_ERR_SHAPE              # more queries than cached tokens
    assert call(q=FAKE + 8) == _l3lib.L3_ERR_ALIGNMENT
    assert call(q_strides=_l3lib.i64_array((131072, 64, 2052))) == _l3lib.L3_ERR_STRIDE
    assert call(k_strides=_l3lib.i64_array((131072, -64, 512))) == _l3lib.L3_ERR_STRIDE


def test_linear_decode_argument_checks():
    lib = _l3lib.load()

    def call(x=FAKE, w=FAKE, y=FAKE, M=1, N=2048, K=2048, xs=2048, ws=2048, ys=2048):
        return lib.l3_linear_decode(x, w, y, M, N, K, xs, ws, ys, None)

    assert call(w=None) == _l3lib.L3_ERR_NULL_POINTER
    assert call(M=0) == _l3lib.L3_ERR_SHAPE
    assert call(M=_l3lib.L3_LINEAR_MAX_ROWS + 1) == _l3lib.L3_ERR_SHAPE
    assert call(K=2040, xs=2040, ws=2040) == _l3lib.L3_ERR_SHAPE       # K not a multiple of 32
    assert call(M=17) == _l3lib.L3_ERR_SHAPE                           # more than one 16-column block of rows
    assert call(N=2046, ys=2048) == _l3lib.L3_ERR_SHAPE                # N not a multiple of 4
    assert call(xs=1024) == _l3lib.L3_ERR_STRIDE                       # rows would overlap
    assert call(ws=2052) == _l3lib.L3_ERR_STRIDE                       # weight rows not 16-byte aligned
    assert call(ys=2046) == _l3lib.L3_ERR_STRIDE
    assert call(x=FAKE + 8) == _l3lib.L3_ERR_ALIGNMENT
    assert call(y=FAKE + 4) == _l3lib.L3_ERR_ALIGNMENT
    assert lib.l3_linear_swiglu_decode(FAKE, FAKE, None, FAKE, 1, 8192, 2048, 2048, 2048, 8192, None) \
        == _l3lib.L3_ERR_NULL_POINTER
    assert lib.l3_linear_swiglu_decode(FAKE, FAKE, FAKE + 2, FAKE, 1, 8192, 2048, 2048, 2048, 8192, None) \
        == _l3lib.L3_ERR_ALIGNMENT


def test_linear_decode_fused_argument_checks():
    lib = _l3lib.load()

    def call(norm=FAKE, res=FAKE, M=1, K=2048):
        return lib.l3_linear_decode_fused(FAKE, norm, 1e-5, FAKE, None, res, FAKE, M, 2048, K, K, K, 2048, None)

    assert call(M=12) == _l3lib.L3_ERR_SHAPE              # 12 rows of 2048 do not fit the LDS stage
    assert call(M=17, K=512) == _l3lib.L3_ERR_SHAPE       # the input norm is for up to 16 rows
    assert call(M=3, K=8192) == _l3lib.L3_ERR_SHAPE
    assert call(norm=FAKE + 2) == _l3lib.L3_ERR_ALIGNMENT
    assert call(res=FAKE + 4) == _l3lib.L3_ERR_ALIGNMENT


def test_greedy_step_argument_checks():
    lib = _l3lib.load()

    def call(logits=FAKE, ws=FAKE, ws_bytes=1 << 20, rows=4, V=1000, stride=1000, L=16, eos=FAKE, pos=FAKE, n_stop=1):
        return lib.l3_greedy_step(logits, stride, rows, V, ws, ws_bytes, FAKE, FAKE, L, FAKE, pos, FAKE, eos, FAKE,
                                  n_stop, None)

    assert call(eos=None) == _l3lib.L3_ERR_NULL_POINTER
    assert call(rows=0) == _l3lib.L3_ERR_SHAPE
    assert call(L=0) == _l3lib.L3_ERR_SHAPE
    assert call(stride=999) == _l3lib.L3_ERR_STRIDE
    assert call(pos=FAKE + 2) == _l3lib.L3_ERR_ALIGNMENT
    assert call(ws_bytes=8) == _l3lib.L3_ERR_WORKSPACE


def test_linear_qkv_rope_append_argument_checks():
    lib = _l3lib.load()
    cs = _l3lib.i64_array((256 * 512, 512))

    def call(table=FAKE, q_out=FAKE, B=1, HD=64, K=2048, strides=cs, norm=None):
        return lib.l3_linear_qkv_rope_append(FAKE, norm, 1e-5, FAKE, table, q_out, FAKE, FAKE, FAKE, B, 32, 8, HD, K,
                                             K, K, strides, 256, 16384, None)

    assert call(table=None) == _l3lib.L3_ERR_NULL_POINTER
    assert call(HD=60) == _l3lib.L3_ERR_SHAPE
    assert call(B=65) == _l3lib.L3_ERR_SHAPE
    assert call(B=17) == _l3lib.L3_ERR_SHAPE               # the rope epilogue is for up to 16 rows
    assert call(K=2040) == _l3lib.L3_ERR_SHAPE
    assert call(B=12, norm=FAKE) == _l3lib.L3_ERR_SHAPE
    assert call(strides=_l3lib.i64_array((256 * 512, 516))) == _l3lib.L3_ERR_STRIDE
    assert call(q_out=FAKE + 8) == _l3lib.L3_ERR_ALIGNMENT


def test_linear_splitk_plan_and_argument_checks():
    lib = _l3lib.load()
    # 1B-architecture matrices on a 256-CU device: enough workgroups (128 weight rows x one split each)
    for (N, K) in ((3072, 2048), (2048, 2048), (2048, 8192), (16384, 2048), (128256, 2048)):
        ks = lib.l3_linear_splitk_plan(N, K, 256)
        chunks = K // 128
        per = -(-chunks // ks)
        assert 1 <= ks <= chunks and per <= (8 if -(-N // 128) < 64 else 4)
        rows_per_wg = 64 if -(-N // 128) < 64 else 128      # few rows: 64-row groups, k range halved inside
        assert per == (8 if rows_per_wg == 64 else 4) or -(-N // rows_per_wg) * ks >= 192
    assert lib.l3_linear_splitk_plan(2048, 2000, 256) == _l3lib.L3_ERR_SHAPE
    assert lib.l3_linear_splitk_workspace_bytes(64, 2048, 16) == 16 * 64 * 2048 * 4

    def call(M=64, N=2048, K=2048, ks=4, nbytes=1 << 30, part=FAKE):
        return lib.l3_linear_splitk(FAKE, FAKE, part, nbytes, M, N, K, K, K, ks, None)

    assert call(part=None) == _l3lib.L3_ERR_NULL_POINTER
    assert call(M=65) == _l3lib.L3_ERR_SHAPE
    assert call(N=2044) == _l3lib.L3_ERR_SHAPE
    assert call(ks=1) == _l3lib.L3_ERR_SPLITS          # 2048 k per workgroup: more than it stages
    assert call(N=16384, ks=2) == _l3lib.L3_ERR_SPLITS # 128-row groups stage at most 512 k
    assert call(ks=17) == _l3lib.L3_ERR_SPLITS
    assert call(nbytes=1024) == _l3lib.L3_ERR_WORKSPACE
    assert _l3lib.L3_LINEAR_MAX_ROWS == 16 and _l3lib.L3_LINEAR_SPLITK_MAX_ROWS == 64

    def finish(part=FAKE, ks=4, res=None, y=FAKE, M=64, N=2048, stride=2048):
        return lib.l3_linear_splitk_finish(part, ks, res, y, M, N, stride, None)

    assert finish(part=None) == _l3lib.L3_ERR_NULL_POINTER
    assert finish(y=None) == _l3lib.L3_ERR_NULL_POINTER
    assert finish(M=65) == _l3lib.L3_ERR_SHAPE
    assert finish(N=2052) == _l3lib.L3_ERR_SHAPE
    assert finish(ks=0) == _l3lib.L3_ERR_SPLITS
    assert finish(stride=2040) == _l3lib.L3_ERR_STRIDE
    assert finish(res=FAKE + 8) == _l3lib.L3_ERR_ALIGNMENT
    assert lib.l3_add_rms_norm_partials(FAKE, FAKE, 0, FAKE, FAKE, FAKE, 64, 2048, 1e-5, None) == _l3lib.L3_ERR_SPLITS
    assert lib.l3_add_rms_norm_partials(FAKE, FAKE, 4, FAKE, FAKE, FAKE, 64, 2044, 1e-5, None) == _l3lib.L3_ERR_SHAPE
    cs = _l3lib.i64_array((256 * 512, 512))
    assert lib.l3_rot_embed_append_partials(FAKE, 4, FAKE, FAKE, FAKE, None, FAKE, 64, 32, 8, 64, cs, 256, 512, None) \
        == _l3lib.L3_ERR_NULL_POINTER
    assert lib.l3_rot_embed_append_partials(FAKE, 4, FAKE, FAKE, FAKE, FAKE, FAKE, 64, 32, 8, 60, cs, 256, 512, None) \
        == _l3lib.L3_ERR_SHAPE


def test_read_stream_argument_checks():
    lib = _l3lib.load()
    assert lib.l3_hbm_read_stream(None, 1 << 20, FAKE, 0, None) == _l3lib.L3_ERR_NULL_POINTER
    assert lib.l3_hbm_read_stream(FAKE, 0, FAKE, 0, None) == _l3lib.L3_ERR_SHAPE
    assert lib.l3_hbm_read_stream(FAKE, 1000, FAKE, 0, None) == _l3lib.L3_ERR_SHAPE
    assert lib.l3_hbm_read_stream(FAKE + 8, 1 << 20, FAKE, 0, None) == _l3lib.L3_ERR_ALIGNMENT
