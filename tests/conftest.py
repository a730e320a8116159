import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "llama3-custom-inference_amd")
for p in (ROOT, PKG, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # Tests load the library that is already built in-tree; only when there is none do
    # they build it (hipcc cross-compiles gfx950 without a GPU).
    lib = os.path.join(PKG, "custom_kernels", "libl3kernels.so")
    if not os.path.exists(lib):
        import build as l3_build

        l3_build.build_library(verbose=False)


@pytest.fixture(scope="session")
def gpu():
    """The device the GPU tests run on; also asserts that the HIP library is the thing loaded."""
    import torch
    from custom_kernels import _l3lib

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    _l3lib.load()  # raises if libl3kernels.so is missing: no fallback is allowed
    return torch.device("cuda:0")


@pytest.fixture(params=["mfma", "fma"])
def attn_kernel(request):
    """Run an attention test once per split-KV kernel (MFMA tiles / FMA dot products): the shim's
    context-local default flags carry the choice into every call of the test."""
    from custom_kernels import custom_kernels_extension as cke

    with cke.attention_flags(kernel=request.param):
        yield request.param


@pytest.fixture(params=["auto", "wave", "tiled", "tiled-no-max"])
def prefill_form(request):
    """Run a prefill test once per form of the kernel (the library's own choice, and each forced)."""
    from custom_kernels import custom_kernels_extension as cke

    with cke.attention_flags(prefill=request.param):
        yield request.param
