"""Containers returned by the preparation and pattern-construction calls.

The field names, their order and their defaults are the reference's
(src/risa_attention/_types.py:13-79), because callers build and ``replace()`` these
objects by field name; ``v_tile_sum`` is the one addition (appended, defaulted).  The
shapes and layouts documented per field are this build's.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch


def _ceil_div(value: int, unit: int) -> int:
    return -(-value // unit)


@dataclass(frozen=True, slots=True)
class PrequantizedInt8Attention:
    """Packed operands of one attention problem; no floating-point Q, K or V is kept.

    Produced by :func:`prequantize_int8_attention`, consumed by
    :func:`int8_attention_from_prequantized` and the pattern constructors.
    """

    # int8 [B, Hq, Lq, Dk] and [B, Hkv, Lk, Dk] codes of the rotated Q and K (Dk = 64/128/256)
    q: torch.Tensor
    k: torch.Tensor
    # int8 [B*Hkv*Dk, padded keys], channel-major; every 32-token group in the order of
    # risaattention_amd.layout (the order the 32x32x32 INT8 matrix instruction consumes)
    v: torch.Tensor
    # float32 [B, Hq, ceil(Lq/128) * 32 (64 for Dk = 256)]: one scale per 8 (4) interleaved rows
    q_scale: torch.Tensor
    # float32 [B, Hkv, key tiles * 4]: four interleaved scale groups per key tile
    k_scale: torch.Tensor
    # float32 [B*Hkv*Dk] each: per-channel step and (midpoint_affine) residual-corrected centre
    v_scale: torch.Tensor
    v_center: torch.Tensor
    original_head_dim: int          # head dim of the inputs, before zero padding to Dk
    input_dtype: torch.dtype        # decides the output dtype (float32 inputs give bfloat16 kernels)
    attention_scale: float          # softmax scale, natural-log domain
    cta_k: int                      # keys per tile: 64, or 128 (wide head, > 1024 keys, no query mask)
    attn_mask: torch.Tensor | None  # the caller's mask broadcast to [B, Hq, Lq, Lk] (a view, not a copy)
    v_quantization: str = "absmax"
    is_causal: bool = False
    lse_shift: torch.Tensor | None = None  # float32 [B, Hq, Lq]: scale * q . k_anchor, for merged LSEs
    kv_permuted: bool = False
    # int32 [B*Hkv, key tiles, Dk]: accumulator seeds of the P.V product, 128 * (tile sum of the
    # V codes of the channel) + 0x4B400000; None lets the attention call compute them
    v_tile_sum: torch.Tensor | None = None

    @property
    def key_tiles(self) -> int:
        return self.v.shape[-1] // self.cta_k

    @property
    def packed_bytes(self) -> int:
        tensors = (self.q, self.k, self.v, self.q_scale, self.k_scale, self.v_scale, self.v_center)
        return sum(t.numel() * t.element_size() for t in tensors)


@dataclass(frozen=True, slots=True)
class RetainedMassPattern:
    """Key tiles kept per 128-query block, as CSR over rows ``[batch, query head, query block]``."""

    row_offsets: torch.Tensor    # int32 [rows + 1]
    block_indices: torch.Tensor  # int32 [kept tiles], ascending inside every row
    batch_size: int
    q_heads: int
    q_length: int
    kv_length: int
    query_block_size: int
    key_block_size: int
    attention_scale: float
    retained_mass_target: float      # theta
    measured_retained_mass: float    # kept mass / total mass over all rows
    is_causal: bool = False
    mask_signature: tuple | None = None
    mask_reference: torch.Tensor | None = None

    @property
    def query_blocks(self) -> int:
        return _ceil_div(self.q_length, self.query_block_size)

    @property
    def key_blocks(self) -> int:
        return _ceil_div(self.kv_length, self.key_block_size)

    @property
    def rows(self) -> int:
        return self.batch_size * self.q_heads * self.query_blocks

    @property
    def coverage(self) -> float:
        """Kept tiles over all tiles."""
        return self.block_indices.numel() / (self.rows * self.key_blocks)

    @property
    def sparsity(self) -> float:
        return 1.0 - self.coverage

    @property
    def index_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.row_offsets, self.block_indices))
