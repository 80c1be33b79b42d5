"""Split-KV flash-decoding wrapper (no counterpart in the reference)."""

import math
from typing import Optional

import torch

__all__ = ["flash_decode"]


def flash_decode(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    num_splits: int = 64,
    softmax_scale: Optional[float] = None,
) -> torch.Tensor:
    """Single-query attention: query [..., 1, D] or [..., D]; key, value [..., Lkv, D].

    The key/value range is cut into `num_splits` chunks that are reduced independently and
    merged by a log-sum-exp combine kernel.  Returns a tensor shaped like `query`."""
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(query.size(-1))
    out = torch.empty_like(query)
    torch.ops.tilefusion.flash_decode(
        query.contiguous(), key.contiguous(), value.contiguous(), out, num_splits, softmax_scale
    )
    return out
