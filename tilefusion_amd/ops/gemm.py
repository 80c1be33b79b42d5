"""GEMM op wrapper (counterpart of python/ops/gemm.py:15-53)."""

import torch

__all__ = ["gemm"]


def gemm(
    tensor_a: torch.Tensor,
    tensor_b: torch.Tensor,
    tensor_c: torch.Tensor,
    tile_m: int,
    tile_n: int,
    tile_k: int,
    num_stages: int,
    pipeline_level: int,
) -> None:
    """C = A @ B with fp16 inputs and fp32 accumulation, written into `tensor_c`.

    Args:
        tensor_a: [M, K] fp16, row-major.
        tensor_b: [N, K] fp16 - the column-major K x N operand.
        tensor_c: [M, N] output, fp32 (as in the reference op) or fp16.
        tile_m, tile_n, tile_k: the reference's shared-memory tile sizes.  They must divide
            the problem; the MI355X library maps the call onto its own MFMA tilings.
        num_stages: 1..3, pipeline_level: 0..2 - validated, kept for signature parity (LDS
            double buffering is always on).
    """
    torch.ops.tilefusion.gemm(
        tensor_a, tensor_b, tensor_c, tile_m, tile_n, tile_k, num_stages, pipeline_level
    )
