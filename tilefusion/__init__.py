"""`import tilefusion` for callers written against the reference package name
(python/__init__.py:19-40): the same modules as `tilefusion_amd`, under the reference's name."""

import sys

import tilefusion_amd
from tilefusion_amd import __version__, jit, ops  # noqa: F401

sys.modules[__name__ + ".ops"] = ops
sys.modules[__name__ + ".jit"] = jit
for _name in ("gemm", "fused_two_gemms", "flash_attention", "flash_decode", "scatter_nd"):
    sys.modules[f"{__name__}.ops.{_name}"] = sys.modules[f"tilefusion_amd.ops.{_name}"]

__all__ = ["jit", "ops"]
