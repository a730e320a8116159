"""Builds libl3kernels.so for gfx950 with hipcc (in-tree, next to the Python shim).

Counterpart of the reference's setup.py:1-16, which JIT-builds its CUDA sources through
torch.utils.cpp_extension; here the library has no torch or pybind dependency and is a
plain `hipcc -shared`.  Run as `python build.py` (add `--incremental` to recompile only the
sources that changed) or call build_library().
"""

import concurrent.futures
import glob
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(PKG_DIR, "build")
LIB_PATH = os.path.join(PKG_DIR, "custom_kernels", "libl3kernels.so")
SOURCES = ["l3_api.hip", "attn_decode.hip", "attn_mfma.hip", "attn_prefill.hip", "attn_prefill_tiled.hip",
           "linear_skinny.hip", "linear_splitk.hip", "attn_combine.hip", "rms_norm.hip", "rot_embed.hip",
           "decode_misc.hip", "hbm_stream.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # scalar float code must not be turned into packed-fp32 instructions on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the gfx950 kernels cannot be built")
    return exe


def _newest_header() -> float:
    hdrs = glob.glob(os.path.join(CSRC, "*.hpp")) + glob.glob(os.path.join(PKG_DIR, "..", "include", "*.h"))
    return max(os.path.getmtime(h) for h in hdrs)


def build_library(verbose: bool = True, extra_flags=(), incremental: bool = False, jobs: int = 8) -> str:
    """Compile every source to an object file (in parallel) and link the shared library.  With
    `incremental` an object newer than its source and every header is kept."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    base = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, "-I", os.path.join(PKG_DIR, "..", "include")]
    hdr_time = _newest_header()
    todo, objs = [], []
    for s in SOURCES:
        src = os.path.join(CSRC, s)
        obj = os.path.join(OBJ_DIR, s.replace(".hip", ".o"))
        objs.append(obj)
        if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), hdr_time):
            continue
        todo.append(base + ["-c", src, "-o", obj])

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)

    with concurrent.futures.ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        list(pool.map(run, todo))
    run([hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH])
    return LIB_PATH


if __name__ == "__main__":
    argv = sys.argv[1:]
    inc = "--incremental" in argv
    build_library(extra_flags=[a for a in argv if a != "--incremental"], incremental=inc)
