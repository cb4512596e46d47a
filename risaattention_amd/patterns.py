"""Retained-mass support construction on the device and sparse reuse.

Counterpart of reference src/risa_attention/sparse.py:18-178.
"""

from __future__ import annotations

import math

import torch

from . import native
from .attend import execute_dense_attention, int8_attention_from_prequantized
from .policy import QUERY_BLOCK_SIZE, mask_signature, uses_centered_values
from .prepare import prequantize_int8_attention
from .types import PrequantizedInt8Attention, RetainedMassPattern


def select_retained_mass_csr(masses: torch.Tensor, theta: float):
    """Shortest descending prefix reaching ``theta`` of each row's mass, as ordered CSR.

    Returns ``(row_offsets, block_indices, measured_mass)``.  Reading the
    summary back is the only host synchronisation of pattern construction.
    """
    rows, tiles = masses.shape
    device = masses.device
    library = native.library()
    # Rows that fit one workgroup are sorted inside the library (one launch; ties by ascending
    # tile id); longer ones with torch.sort, as the reference does (sparse.py:24).
    in_library = tiles <= library.risa_sortable_key_blocks() and masses.is_contiguous()
    if in_library:
        sorted_mass = torch.empty_like(masses)
        order = torch.empty((rows, tiles), dtype=torch.int64, device=device)
    else:
        sorted_mass, order = masses.sort(dim=-1, descending=True)
    counts = torch.empty(rows, dtype=torch.int32, device=device)
    support = torch.empty((rows, tiles), dtype=torch.uint8, device=device)
    row_totals = torch.empty((rows, 2), dtype=torch.float64, device=device)
    row_offsets = torch.empty(rows + 1, dtype=torch.int32, device=device)
    storage = torch.empty(rows * tiles, dtype=torch.int32, device=device)
    summary = torch.empty(3, dtype=torch.float64, device=device)
    outputs = (sorted_mass.data_ptr(), order.data_ptr(), counts.data_ptr(), support.data_ptr(),
               row_totals.data_ptr(), row_offsets.data_ptr(), storage.data_ptr(), summary.data_ptr(),
               rows, tiles, float(theta), native.current_stream(device))
    if in_library:
        native.check(library.risa_sort_select_retained_mass(masses.data_ptr(), *outputs))
    else:
        native.check(library.risa_select_retained_mass(*outputs))
    selected_mass, total_mass, selected_blocks = summary.tolist()
    return row_offsets, storage[: int(selected_blocks)], selected_mass / max(total_mass, 1e-20)


def capture_workspace_elements(batch, q_heads, q_len, key_blocks):
    mass = batch * q_heads * math.ceil(q_len / QUERY_BLOCK_SIZE) * key_blocks
    return mass, mass + batch * q_heads * q_len * (key_blocks * 2 + 2)


@torch.inference_mode()
def construct_sparse_int8_attention_from_prequantized(
    quantized: PrequantizedInt8Attention,
    *,
    theta: float = 0.99,
    output_layout: str = "hnd",
) -> tuple[torch.Tensor, RetainedMassPattern]:
    """Dense attention over packed operands that also returns reusable support.

    The attention kernel stores, per query and key tile, the sum of its U8
    probabilities and the tile maximum; block masses are rebuilt from those and
    the final softmax state without replaying QK.  ``theta`` is the retained
    mass threshold.  Masses follow the quantised probabilities; use
    :func:`measure_pattern_recall` for exact FP32 recall.
    """
    if not 0.0 < theta <= 1.0 or not math.isfinite(theta):
        raise ValueError("theta must be finite and in (0, 1]")
    if not isinstance(quantized, PrequantizedInt8Attention):
        raise TypeError(
            f"quantized must be returned by prequantize_int8_attention, got {type(quantized).__name__}"
        )
    batch, q_heads, q_len, _ = quantized.q.shape
    key_blocks = math.ceil(quantized.k.shape[2] / quantized.cta_k)
    mass_elements, total_elements = capture_workspace_elements(batch, q_heads, q_len, key_blocks)
    workspace = torch.empty(total_elements, dtype=torch.float32, device=quantized.q.device)
    output = int8_attention_from_prequantized(quantized, output_layout=output_layout, _block_mass=workspace)
    masses = workspace[:mass_elements].view(-1, key_blocks)
    row_offsets, block_indices, measured = select_retained_mass_csr(masses, theta)
    pattern = RetainedMassPattern(
        row_offsets=row_offsets,
        block_indices=block_indices,
        batch_size=batch,
        q_heads=q_heads,
        q_length=q_len,
        kv_length=quantized.k.shape[2],
        query_block_size=QUERY_BLOCK_SIZE,
        key_block_size=quantized.cta_k,
        attention_scale=quantized.attention_scale,
        retained_mass_target=float(theta),
        measured_retained_mass=measured,
        is_causal=quantized.is_causal,
        mask_signature=mask_signature(quantized.attn_mask),
        mask_reference=quantized.attn_mask,
    )
    return output, pattern


@torch.inference_mode()
def construct_sparse_int8_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    *,
    theta: float = 0.99,
    scale: float | None = None,
    output_layout: str = "hnd",
    v_quantization: str = "absmax",
    is_causal: bool = False,
    attn_mask: torch.Tensor | None = None,
) -> tuple[torch.Tensor, RetainedMassPattern]:
    """Dense INT8 attention that also builds the retained-mass pattern."""
    packed = prequantize_int8_attention(q, k, v, scale=scale, v_quantization=v_quantization,
                                        is_causal=is_causal, attn_mask=attn_mask)
    return construct_sparse_int8_attention_from_prequantized(packed, theta=theta,
                                                             output_layout=output_layout)


def sparse_int8_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    sparse_pattern: RetainedMassPattern,
    *,
    scale: float | None = None,
    output_layout: str = "hnd",
    v_quantization: str = "absmax",
    is_causal: bool = False,
    attn_mask: torch.Tensor | None = None,
) -> torch.Tensor:
    """INT8 attention over a frozen pattern; Q/K/V are quantised again on every call
    (one native call: preparation and the walk over the pattern's key tiles)."""
    return execute_dense_attention(q, k, v, scale=scale, attn_mask=attn_mask,
                                   use_midpoint_affine=uses_centered_values(v_quantization),
                                   is_causal=is_causal, sparse_pattern=sparse_pattern,
                                   output_layout=output_layout)
