"""MI355X-native TileFusion hot path: Python package.

Mirrors the reference's package (python/__init__.py:19-40): importing it loads
`libtilefusion.so` with ctypes, whose static initialisers register
`torch.ops.tilefusion.*`; `tilefusion_amd.ops` holds the thin wrappers
(python/ops/*.py).  The library wraps hand-written HIP kernels for gfx950 behind the C ABI
of include/tilefusion_c.h (libtilefusion_hip.so).  There is no CPU fallback: a missing
library is an error.
"""

import ctypes
import os
from typing import Any

__version__ = "0.1.0"

_HERE = os.path.dirname(os.path.abspath(__file__))


def _load_library(filename: str) -> Any:
    """Load the binding library (python/__init__.py:19-37 in the reference)."""
    lib_path = os.path.join(_HERE, filename)
    if not os.path.exists(lib_path):
        raise RuntimeError(
            f"{lib_path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C tilefusion_amd/csrc all bind` (there is no CPU fallback)")
    try:
        import torch  # noqa: F401  (libtorch must be resident before the binding loads)
        return ctypes.CDLL(lib_path)
    except OSError as e:
        raise RuntimeError(f"Failed to load library from {lib_path}") from e


_lib = _load_library("libtilefusion.so")

from . import _capi, jit, ops  # noqa: E402

__all__ = ["jit", "ops"]
