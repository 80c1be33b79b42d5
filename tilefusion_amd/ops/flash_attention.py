"""Flash-attention forward wrapper (counterpart of python/ops/flash_attention.py:15-129)."""

import torch

__all__ = ["FlashAttention", "flash_attention"]


class FlashAttention:
    """Callable with the reference's constructor arguments (python/ops/flash_attention.py:18-43)."""

    def __init__(
        self,
        tile_length_q: int,
        tile_length_kv: int,
        tile_hidden_qk: int,
        tile_hidden_v: int,
        softmax_scale: float,
        causal: bool,
    ) -> None:
        self.tile_length_q = tile_length_q
        self.tile_length_kv = tile_length_kv
        self.tile_hidden_qk = tile_hidden_qk
        self.tile_hidden_v = tile_hidden_v
        self.softmax_scale = softmax_scale
        self.causal = causal

    def __call__(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
        """query [..., Lq, D], key [..., D, Lkv] (as the reference's callers pass it,
        tests/python/test_flash_attn.py:173-175), value [..., Lkv, Dv] -> [..., Lq, Dv].

        The reference transposes both key and value before its op
        (python/ops/flash_attention.py:73-74); here only the key is made [Lkv, D]-contiguous
        and the value is consumed in its natural layout (the kernel transposes it on the way
        from LDS to registers).  Tile sizes are validated against the problem."""
        length_q, hidden_qk = query.size(-2), query.size(-1)
        length_kv, hidden_v = value.size(-2), value.size(-1)
        for what, dim, tile in (("length_q", length_q, self.tile_length_q),
                                ("length_kv", length_kv, self.tile_length_kv),
                                ("hidden_qk", hidden_qk, self.tile_hidden_qk),
                                ("hidden_v", hidden_v, self.tile_hidden_v)):
            if tile <= 0 or dim % tile != 0:
                raise RuntimeError(f"tile size {tile} does not divide {what} = {dim}")
        output = torch.empty(*query.shape[:-1], hidden_v, dtype=query.dtype, device=query.device)
        torch.ops.tilefusion.flash_attention_fwd(
            query.contiguous(),
            key.transpose(-1, -2).contiguous(),
            value.contiguous(),
            output,
            self.softmax_scale,
            self.causal,
        )
        return output


def flash_attention(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    tile_length_q: int,
    tile_length_kv: int,
    tile_hidden_qk: int,
    tile_hidden_v: int,
    softmax_scale: float,
    causal: bool,
) -> torch.Tensor:
    """Functional form, same positional signature as the reference
    (python/ops/flash_attention.py:86-96)."""
    return FlashAttention(
        tile_length_q, tile_length_kv, tile_hidden_qk, tile_hidden_v, softmax_scale, causal
    )(query, key, value)
