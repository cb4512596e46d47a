"""Containers returned by the preparation and pattern-construction calls.

Field names, order and defaults follow reference src/risa_attention/_types.py:13-79
so that code written against the reference keeps working; ``v_tile_sum`` is the
one addition (appended with a default) and carries the accumulator seeds of the
P·V product: 128 x the per-tile sums of the V codes (the zero-point term the
signed-INT8 matrix cores need) + 0x4B400000.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch


@dataclass(frozen=True, slots=True)
class PrequantizedInt8Attention:
    """Packed Q/K/V codes, their scales and the launch metadata of one call.

    Holds no floating-point Q, K or V.  ``v`` is ``[B*Hkv*D, padded_keys]`` with
    every 32-token group in the order given by ``risaattention_amd.layout``.
    Instances come from :func:`prequantize_int8_attention`.
    """

    q: torch.Tensor
    k: torch.Tensor
    v: torch.Tensor
    q_scale: torch.Tensor
    k_scale: torch.Tensor
    v_scale: torch.Tensor
    v_center: torch.Tensor
    original_head_dim: int
    input_dtype: torch.dtype
    attention_scale: float
    cta_k: int
    attn_mask: torch.Tensor | None
    v_quantization: str = "absmax"
    is_causal: bool = False
    lse_shift: torch.Tensor | None = None
    kv_permuted: bool = False
    v_tile_sum: torch.Tensor | None = None


@dataclass(frozen=True, slots=True)
class RetainedMassPattern:
    """Frozen block support in CSR form, rows ordered [batch, query head, query block]."""

    row_offsets: torch.Tensor
    block_indices: torch.Tensor
    batch_size: int
    q_heads: int
    q_length: int
    kv_length: int
    query_block_size: int
    key_block_size: int
    attention_scale: float
    retained_mass_target: float
    measured_retained_mass: float
    is_causal: bool = False
    mask_signature: tuple | None = None
    mask_reference: torch.Tensor | None = None

    @property
    def coverage(self) -> float:
        query_blocks = math.ceil(self.q_length / self.query_block_size)
        key_blocks = math.ceil(self.kv_length / self.key_block_size)
        return self.block_indices.numel() / (self.batch_size * self.q_heads * query_blocks * key_blocks)

    @property
    def sparsity(self) -> float:
        return 1.0 - self.coverage

    @property
    def index_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.row_offsets, self.block_indices))
