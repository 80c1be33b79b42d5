"""Fused back-to-back GEMM wrapper (counterpart of python/ops/fused_two_gemms.py:15-79)."""

import torch

__all__ = ["fused_two_gemms"]


def _validate_tensor(
    tensor: torch.Tensor,
    name: str,
    expected_dtype: torch.dtype = torch.float16,
    expected_device: str = "cuda",
) -> None:
    """Same contract as the reference: ValueError for a wrong device, TypeError for a wrong
    dtype (python/ops/fused_two_gemms.py:33-38)."""
    if tensor.device.type != expected_device:
        raise ValueError(f"{name} must be a {expected_device} tensor")
    if tensor.dtype != expected_dtype:
        raise TypeError(f"{name} must be of type {expected_dtype}, got {tensor.dtype}")


def fused_two_gemms(
    input_a: torch.Tensor,
    input_b: torch.Tensor,
    input_c: torch.Tensor,
    output: torch.Tensor,
    tm: int = 64,
    tn: int = 64,
    tk: int = 64,
    tp: int = 64,
) -> None:
    """D = (A @ B) @ C without writing A @ B to memory.

    Args:
        input_a: [M, K] row-major.
        input_b: [N, K] buffer (the column-major K x N operand).
        input_c: [P, N] buffer (the column-major N x P operand).
        output: [M, P] row-major, written in place.
        tm, tn, tk, tp: the reference's tile sizes; must divide M, N, K, P.

    All four tensors are float16 (as in the reference) or all bfloat16.
    """
    dtype = torch.bfloat16 if input_a.dtype == torch.bfloat16 else torch.float16
    _validate_tensor(input_a, "input_a", dtype)
    _validate_tensor(input_b, "input_b", dtype)
    _validate_tensor(input_c, "input_c", dtype)
    _validate_tensor(output, "output", dtype)
    torch.ops.tilefusion.fused_two_gemms(input_a, input_b, input_c, output, tm, tn, tk, tp)
