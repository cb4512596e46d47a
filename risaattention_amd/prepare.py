"""Q/K/V preparation: padding, tile policy, buffer allocation and the HIP launches.

Host-side counterpart of reference src/risa_attention/_quantization.py:23-198
(``prequantize_int8_attention``) on top of the C ABI in include/risa_hip.h.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch
from torch.nn import functional

from . import native
from .policy import (
    DTYPE_CODES,
    kernel_head_dim,
    pad_key_length,
    select_key_block_size,
    uses_centered_values,
    validate_inputs,
)
from .types import PrequantizedInt8Attention


@dataclass
class PreparedBuffers:
    """Device buffers written by the preparation kernels for one call."""

    q_codes: torch.Tensor
    k_codes: torch.Tensor
    v_codes: torch.Tensor
    q_scale: torch.Tensor
    k_scale: torch.Tensor
    v_scale: torch.Tensor
    v_center: torch.Tensor
    v_tile_sum: torch.Tensor
    anchors: torch.Tensor
    kernel_dim: int
    cta_k: int
    attention_scale: float
    q_padded: torch.Tensor
    k_padded: torch.Tensor


def pad_head_dim(q, k, v):
    """Zero-pad the channel axis to the kernel's 64/128/256 tile."""
    dim = q.shape[-1]
    kernel_dim = kernel_head_dim(dim)
    if kernel_dim != dim:
        extra = (0, kernel_dim - dim)
        q, k, v = functional.pad(q, extra), functional.pad(k, extra), functional.pad(v, extra)
    return q, k, v, kernel_dim


def resolve_scale(scale: float | None, head_dim: int) -> float:
    value = head_dim**-0.5 if scale is None else float(scale)
    if not math.isfinite(value):
        raise ValueError(f"scale must be finite, got {value}")
    return value


def quantize_inputs(q, k, v, attn_mask, scale, use_midpoint_affine: bool,
                    kv_permutation: torch.Tensor | None = None) -> PreparedBuffers:
    """Allocate the packed buffers and enqueue the Q/K and V preparation kernels.

    ``q``, ``k``, ``v`` are validated; ``attn_mask`` is already broadcast (its
    query stride decides the key tile size).  ``kv_permutation`` (int32
    ``[B,Hkv,Lk]``) makes the K and V kernels read key ``n`` from source token
    ``kv_permutation[b,h,n]``: the gather fused into quantisation.
    """
    lib = native.library()
    original_dim = q.shape[-1]
    input_dtype = q.dtype
    q, k, v, dim = pad_head_dim(q, k, v)
    attention_scale = resolve_scale(scale, original_dim)
    batch, q_heads, q_len, _ = q.shape
    _, kv_heads, k_len, _ = k.shape
    query_mask = attn_mask is not None and attn_mask.stride(-2) != 0
    cta_k = select_key_block_size(dim, k_len, has_mask=query_mask)
    padded = pad_key_length(k_len, cta_k)
    device = q.device
    rows = batch * kv_heads * dim

    def empty(*shape, dtype):
        return torch.empty(shape, dtype=dtype, device=device)

    q_codes = empty(*q.shape, dtype=torch.int8)
    k_codes = empty(*k.shape, dtype=torch.int8)
    q_scale = empty(batch, q_heads, -(-q_len // 128) * (64 if dim == 256 else 32), dtype=torch.float32)
    k_scale = empty(batch, kv_heads, -(-k_len // cta_k) * 4, dtype=torch.float32)
    v_codes = empty(rows, padded, dtype=torch.int8)
    v_scale = empty(rows, dtype=torch.float32)
    v_center = empty(rows, dtype=torch.float32)
    v_tile_sum = empty(batch * kv_heads, padded // cta_k, dim, dtype=torch.int32)
    anchors = empty(batch, kv_heads, dtype=torch.int32)
    workspace = empty(
        max(1, lib.risa_quantize_v_workspace_bytes(batch, kv_heads, k_len, dim, int(use_midpoint_affine))),
        dtype=torch.uint8,
    )
    stream = native.current_stream(device)
    code = DTYPE_CODES[input_dtype]
    native.check(
        lib.risa_sdpa_quantize(
            q.data_ptr(), q_codes.data_ptr(), q_scale.data_ptr(),
            k.data_ptr(), k_codes.data_ptr(), k_scale.data_ptr(),
            v.data_ptr(), v_codes.data_ptr(), v_scale.data_ptr(), v_center.data_ptr(),
            v_tile_sum.data_ptr(), workspace.data_ptr(), workspace.numel(),
            batch, q_heads, q_len, kv_heads, k_len, dim, cta_k,
            q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
            v.stride(0), v.stride(1), v.stride(2), code, int(use_midpoint_affine),
            anchors.data_ptr(), native.pointer(kv_permutation), stream,
        )
    )
    return PreparedBuffers(q_codes, k_codes, v_codes, q_scale, k_scale, v_scale, v_center,
                           v_tile_sum, anchors, dim, cta_k, attention_scale, q, k)


def lse_shift(buffers: PreparedBuffers, dtype: torch.dtype) -> torch.Tensor:
    """Row-wise logit offset removed from K by the anchor shift, times the scale."""
    q, k = buffers.q_padded, buffers.k_padded
    batch, q_heads, q_len, dim = q.shape
    out = torch.empty((batch, q_heads, q_len), device=q.device, dtype=torch.float32)
    native.check(
        native.library().risa_lse_shift(
            q.data_ptr(), k.data_ptr(), buffers.anchors.data_ptr(), out.data_ptr(),
            batch, q_heads, k.shape[1], q_len, dim,
            q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
            buffers.attention_scale, DTYPE_CODES[dtype], native.current_stream(q.device),
        )
    )
    return out


def prequantize_int8_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    *,
    scale: float | None = None,
    attn_mask: torch.Tensor | None = None,
    v_quantization: str = "absmax",
    is_causal: bool = False,
    return_lse: bool = False,
    kv_permutation=None,
    fuse_gather: bool = True,
) -> PrequantizedInt8Attention:
    """Quantize Q, K and V without allocating the attention output.

    The result keeps no floating-point input, so callers may free Q/K/V before
    :func:`int8_attention_from_prequantized`.  Everything is enqueued on the
    current stream without host synchronisation.  ``return_lse=True`` also
    stores the K-anchor logit offset so that LSE values of different key
    windows can be merged.  ``kv_permutation`` reorders the keys and values; with
    ``fuse_gather`` (and no LSE) the quantisation kernels read through it,
    otherwise K and V are gathered eagerly first.  Both give the same tensors.
    """
    attn_mask = validate_inputs(q, k, v, attn_mask)
    fused_permutation = None
    if kv_permutation is not None:
        from .permutation import prepare_inputs

        q, k, v, fused_permutation = prepare_inputs(
            q, k, v, permutation=kv_permutation, mask=attn_mask, causal=is_causal,
            return_lse=return_lse, fuse=fuse_gather)
    use_midpoint_affine = uses_centered_values(v_quantization)
    original_dim, input_dtype = q.shape[-1], q.dtype
    buffers = quantize_inputs(q, k, v, attn_mask, scale, use_midpoint_affine, fused_permutation)
    shift = lse_shift(buffers, input_dtype) if return_lse else None
    return PrequantizedInt8Attention(
        q=buffers.q_codes,
        k=buffers.k_codes,
        v=buffers.v_codes,
        q_scale=buffers.q_scale,
        k_scale=buffers.k_scale,
        v_scale=buffers.v_scale,
        v_center=buffers.v_center,
        original_head_dim=original_dim,
        input_dtype=input_dtype,
        attention_scale=buffers.attention_scale,
        cta_k=buffers.cta_k,
        attn_mask=attn_mask,
        v_quantization=v_quantization,
        is_causal=is_causal,
        lse_shift=shift,
        kv_permuted=kv_permutation is not None,
        v_tile_sum=buffers.v_tile_sum,
    )
