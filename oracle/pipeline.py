"""End-to-end oracle calls shaped like the public API (test infrastructure only).

Mirrors the orchestration of src/risa_attention/_quantization.py:23-198,
_execution.py:137-328 and sparse.py:55-178 on top of ``oracle.prepare``,
``oracle.attention`` and ``oracle.selection``.  Inputs are binary32 numpy
arrays holding the exactly converted fp16/bf16/fp32 values; ``dtype_name``
names the original dtype (it fixes the output rounding).
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from . import attention, prepare, selection
from .ieee import F32


@dataclass
class Prepared:
    q: np.ndarray
    k: np.ndarray
    v: np.ndarray  # [B*Hkv*Dk, Lpad], token order
    q_scale: np.ndarray
    k_scale: np.ndarray
    v_scale: np.ndarray
    v_center: np.ndarray
    anchor: np.ndarray
    original_head_dim: int
    attention_scale: float
    cta_k: int
    mask: np.ndarray | None
    is_causal: bool
    lse_shift: np.ndarray | None
    out_dtype: str


def _expand_mask(mask, batch, heads, q_len, k_len):
    """Broadcast to [B,H,Lq|1,Lk]; the query extent stays 1 for key-only masks."""
    if mask is None:
        return None, False
    mask = np.asarray(mask)
    while mask.ndim < 4:
        mask = mask[None]
    # Callers that hold the broadcast view's strides override this (a contiguous
    # [..., 1, Lk] mask over one query has a non-zero query stride in the reference).
    query_dependent = mask.shape[2] != 1
    target_q = q_len if query_dependent else 1
    return np.broadcast_to(mask, (batch, heads, target_q, k_len)), query_dependent


def prequantize(q, k, v, *, scale=None, mask=None, v_quantization="absmax", is_causal=False,
                return_lse=False, dtype_name="bfloat16", query_dependent_mask=None) -> Prepared:
    q, k, v = (np.asarray(t, dtype=F32) for t in (q, k, v))
    batch, q_heads, q_len, head_dim = q.shape
    k_len = k.shape[2]
    dim = prepare.kernel_head_dim(head_dim)
    qp, kp, vp = (prepare.pad_channels(t, dim) for t in (q, k, v))
    attention_scale = head_dim**-0.5 if scale is None else float(scale)
    mask, dependent = _expand_mask(mask, batch, q_heads, q_len, k_len)
    if query_dependent_mask is not None:
        dependent = query_dependent_mask
    cta_k = prepare.select_key_block_size(dim, k_len, mask is not None and dependent)
    q_codes, q_scale = prepare.quantize_queries(qp, k_len)
    k_codes, k_scale, anchor = prepare.quantize_keys(kp, cta_k)
    v_codes, v_scale, v_center = prepare.quantize_values(vp, cta_k, v_quantization == "midpoint_affine")
    shift = prepare.lse_shift(qp, kp, anchor, attention_scale) if return_lse else None
    out_dtype = "bfloat16" if dtype_name == "float32" else dtype_name
    return Prepared(q_codes, k_codes, v_codes, q_scale, k_scale, v_scale, v_center, anchor,
                    head_dim, attention_scale, cta_k, mask, is_causal, shift, out_dtype)


def key_mask_tile_list(p: Prepared):
    """Condition of src/risa_attention/_key_mask.py:9-18."""
    if (p.mask is None or p.mask.shape[2] != 1 or p.mask.shape[-1] <= 1024 or p.q.shape[2] < 256
            or p.attention_scale <= 0 or p.is_causal):
        return None
    return selection.key_mask_tiles(p.mask, p.cta_k)


def attend(p: Prepared, *, pattern=None, capture=False, return_lse=False, use_key_mask_tiles=True):
    tiles = None
    if pattern is None and not capture and use_key_mask_tiles:
        tiles = key_mask_tile_list(p)
    row_offsets = block_indices = None
    if pattern is not None:
        row_offsets, block_indices = pattern
        rows = p.q.shape[0] * p.q.shape[1] * ((p.q.shape[2] + 127) // 128)
        n_kb = (p.k.shape[2] + p.cta_k - 1) // p.cta_k
        if 1.0 - len(block_indices) / (rows * n_kb) < 0.05:  # _execution.py:227-228
            row_offsets = block_indices = None
    out, lse, cap = attention.attend(
        p.q, p.k, p.v, p.q_scale, p.k_scale, p.v_scale, p.v_center,
        key_block=p.cta_k, sm_scale=p.attention_scale, mask=p.mask, is_causal=p.is_causal,
        row_offsets=row_offsets, block_indices=block_indices, key_mask_tiles=tiles,
        capture=capture, out_dtype=p.out_dtype,
    )
    out = out[..., : p.original_head_dim]
    if return_lse:
        lse = (lse + p.lse_shift).astype(F32)
    return out, lse, cap


def int8_attention(q, k, v, **kwargs):
    return_lse = kwargs.pop("return_lse", False)
    p = prequantize(q, k, v, return_lse=return_lse, **kwargs)
    out, lse, _ = attend(p, return_lse=return_lse)
    return (out, lse) if return_lse else out


def construct_sparse(q, k, v, *, theta=0.99, **kwargs):
    p = prequantize(q, k, v, **kwargs)
    out, _, cap = attend(p, capture=True)
    masses = attention.block_mass(cap, p.q.shape[0], p.q.shape[1], p.q.shape[2])
    row_offsets, block_indices, measured, _ = selection.select_retained_mass(masses, theta)
    return out, (row_offsets, block_indices), measured, masses
