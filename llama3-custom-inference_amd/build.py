"""Builds libl3kernels.so for gfx950 with hipcc (in-tree, next to the Python shim).

Counterpart of the reference's setup.py:1-16, which JIT-builds its CUDA sources through
torch.utils.cpp_extension; here the library has no torch or pybind dependency and is a
plain `hipcc -shared`.  Run as `python build.py` or call build_library().
"""

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "custom_kernels", "libl3kernels.so")
SOURCES = ["l3_api.hip", "attn_decode.hip", "attn_mfma.hip", "attn_prefill.hip", "attn_prefill_tiled.hip", "linear_skinny.hip", "linear_splitk.hip", "linear_rows64.hip", "attn_combine.hip", "rms_norm.hip", "rot_embed.hip",
           "decode_misc.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
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


def build_library(verbose: bool = True, extra_flags=()) -> str:
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, "-I", os.path.join(PKG_DIR, "..", "include")]
    cmd += [os.path.join(CSRC, s) for s in SOURCES]
    cmd += ["-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


if __name__ == "__main__":
    build_library(extra_flags=sys.argv[1:])
