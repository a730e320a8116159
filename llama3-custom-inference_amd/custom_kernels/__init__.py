"""Drop-in for the reference's ``custom_kernels`` build directory (setup.py:10-14).

``from custom_kernels import custom_kernels_extension`` (model.py:23,
benchmark_kernel.py:4) resolves to a pure-Python module whose three functions call the
gfx950 kernels in ``libl3kernels.so`` through its C ABI.
"""

from . import custom_kernels_extension  # noqa: F401
from .rope_table import apply_scaling, precompute_freqs_cis  # noqa: F401
