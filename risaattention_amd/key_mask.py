"""Tile lists that let broadcast key masks skip fully hidden key tiles.

Counterpart of reference src/risa_attention/_key_mask.py:9-28.
"""

from __future__ import annotations

import torch

from . import native
from .policy import MASK_DTYPE_CODES


def prepare_key_bias(mask, key_block_size):
    """Additive FP32 row of a key-only mask, ``(bias, stride_b, stride_h)`` or ``None``.

    ``mask`` is the expanded ``[B,Hq,Lq,Lk]`` view.  Without a query extent
    (stride 0) every query of a head sees the same row, so the attention kernel
    can stage ``bias[b,h,tile]`` per key tile instead of reading mask elements
    per score: 0 / the float entry times log2(e) / -inf, padded to whole tiles.
    """
    if mask is None or mask.stride(2) != 0:
        return None
    batch = mask.shape[0] if mask.stride(0) != 0 else 1
    heads = mask.shape[1] if mask.stride(1) != 0 else 1
    length = mask.shape[-1]
    padded = -(-length // key_block_size) * key_block_size
    bias = torch.empty((batch, heads, padded), device=mask.device, dtype=torch.float32)
    native.check(
        native.library().risa_prepare_key_bias(
            mask.data_ptr(), bias.data_ptr(), batch, heads, length, padded,
            mask.stride(0), mask.stride(1), mask.stride(3), MASK_DTYPE_CODES[mask.dtype],
            native.current_stream(mask.device),
        )
    )
    return bias, (bias.stride(0) if batch > 1 else 0), (bias.stride(1) if heads > 1 else 0)


def prepare_mask_lanes(mask, key_block_size, head_dim):
    """Lane words of a boolean mask several heads share, ``(words, stride_b, stride_h)`` or ``None``.

    ``mask`` is the expanded ``[B,Hq,Lq,Lk]`` view.  The library decides whether the form
    applies (boolean, query-dependent, unit key stride, 64-key tiles, head dim up to 128,
    at least eight (batch, head) pairs per mask plane) by returning the size of the buffer or 0; the
    attention kernel then takes one 64-lane word per score from scalar registers instead
    of reading mask elements.
    """
    if mask is None or mask.dtype != torch.bool:
        return None
    batch, q_heads, q_len, k_len = mask.shape
    planes_b = batch if mask.stride(0) != 0 else 1
    planes_h = q_heads if mask.stride(1) != 0 else 1
    lib = native.library()
    size = lib.risa_mask_lanes_bytes(MASK_DTYPE_CODES[mask.dtype], head_dim, key_block_size, mask.stride(2),
                                     mask.stride(3), batch, q_heads, planes_b, planes_h, q_len, k_len)
    if size == 0:
        return None
    # the lane words of every plane, then one class per tile (the library carves both)
    words = torch.empty(size // 8, device=mask.device, dtype=torch.int64)
    native.check(
        lib.risa_prepare_mask_lanes(
            mask.data_ptr(), words.data_ptr(), planes_b, planes_h, q_len, k_len,
            mask.stride(0), mask.stride(1), mask.stride(2), native.current_stream(mask.device),
        )
    )
    plane = 4 * -(-q_len // 128) * -(-k_len // 64) * 32  # words of one (batch, head) plane
    return words, (plane * planes_h if planes_b > 1 else 0), (plane if planes_h > 1 else 0)


def prepare_key_mask_tiles(mask, key_block_size, query_length, scale, is_causal):
    """int32 [B,Hq,tiles+1] (active tile ids, then the count) or None.

    Built only for masks without a query extent (stride 0), more than 1024
    keys, at least 256 queries, a positive scale and no causal flag.
    """
    if (
        mask is None
        or mask.stride(-2) != 0
        or mask.shape[-1] <= 1024
        or query_length < 256
        or scale <= 0
        or is_causal
    ):
        return None
    batch, heads, _, length = mask.shape
    tiles = torch.empty((batch, heads, -(-length // key_block_size) + 1), device=mask.device, dtype=torch.int32)
    native.check(
        native.library().risa_prepare_key_mask_tiles(
            mask.data_ptr(), tiles.data_ptr(), batch, heads, length, key_block_size,
            mask.stride(0), mask.stride(1), mask.stride(3), MASK_DTYPE_CODES[mask.dtype],
            native.current_stream(mask.device),
        )
    )
    return tiles
