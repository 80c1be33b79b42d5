"""Scatter operation (counterpart of python/ops/scatter_nd.py:15-29 in the reference)."""

import torch

__all__ = ["scatter_nd"]


def scatter_nd(scatter_data: torch.Tensor, scatter_indices: torch.Tensor, scatter_updates: torch.Tensor) -> None:
    """Accumulate `scatter_updates` into `scatter_data` at `scatter_indices`, in place.

    scatter_data is [d0, .., d(r-1)]; scatter_indices is [.., k] int64 with k <= r; row i of it
    selects the slice scatter_data[idx0, .., idx(k-1)], to which row i of scatter_updates
    ([.., d(k), .., d(r-1)]) is added.  Duplicate index rows accumulate, like the reference
    kernel's atomicAdd (src/kernels/scatter_nd.cu:30); rows outside the tensor are skipped.
    """
    torch.ops.tilefusion.scatter_nd(scatter_data, scatter_updates, scatter_indices)
