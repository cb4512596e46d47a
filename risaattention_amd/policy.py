"""Input contracts, mask helpers and the key-tile policy.

Same rules, error types and messages as reference
src/risa_attention/_validation.py:11-148; the device requirement reads
"ROCm/gfx950" instead of "CUDA/SM80+".
"""

from __future__ import annotations

import torch

from . import native

DTYPE_CODES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
MASK_DTYPE_CODES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2, torch.bool: 3}
SUPPORTED_DTYPES = (torch.float32, torch.float16, torch.bfloat16)
KEY_BLOCK_SIZE = 64
LARGE_KEY_BLOCK_SIZE = 128
QUERY_BLOCK_SIZE = 128
MIN_PATTERN_SPARSITY = 0.05
OUTPUT_LAYOUTS = ("hnd", "nhd")
VALUE_QUANTIZATION_MODES = ("midpoint_affine", "absmax")

UNAVAILABLE = "INT8 attention requires the risaattention_amd HIP extension and a gfx950 (MI355X) GPU"


def uses_centered_values(v_quantization: str) -> bool:
    if v_quantization not in VALUE_QUANTIZATION_MODES:
        raise ValueError(
            f"v_quantization must be one of {VALUE_QUANTIZATION_MODES}, got {v_quantization!r}"
        )
    return v_quantization == "midpoint_affine"


def mask_signature(mask: torch.Tensor | None) -> tuple | None:
    """Identity of a mask's storage and contents version (None for no mask)."""
    if mask is None:
        return None
    try:
        version = mask._version
    except RuntimeError:  # inference tensors carry no version counter
        version = None
    return (mask.data_ptr(), version, tuple(mask.shape), tuple(mask.stride()), mask.dtype, mask.device)


def apply_score_mask(scores, attn_mask, is_causal, start):
    """FP32 masking of a block of score rows beginning at query ``start``."""
    rows = scores.shape[-2]
    if attn_mask is not None:
        window = attn_mask[..., start : start + rows, :]
        scores = scores.masked_fill(~window, -torch.inf) if window.dtype == torch.bool else scores + window
    if is_causal:
        q_index = torch.arange(start, start + rows, device=scores.device)[:, None]
        k_index = torch.arange(scores.shape[-1], device=scores.device)[None, :]
        scores = scores.masked_fill(k_index > q_index, -torch.inf)
    return scores


def pad_key_length(length: int, key_block_size: int = KEY_BLOCK_SIZE) -> int:
    return -(-length // key_block_size) * key_block_size


def kernel_head_dim(head_dim: int) -> int:
    return 64 if head_dim <= 64 else 128 if head_dim <= 128 else 256


def select_key_block_size(kernel_dim: int, key_length: int, *, has_mask: bool) -> int:
    """128-key tiles need a wide head, a long sequence and no query-dependent mask."""
    wide = not has_mask and kernel_dim >= 128 and key_length > 1024
    return LARGE_KEY_BLOCK_SIZE if wide else KEY_BLOCK_SIZE


def is_available(device: torch.device | int | None = None) -> bool:
    return native.is_available(device)


_CHECKED_DEVICES: set[int] = set()  # CUDA device indices that passed is_available()


def validate_inputs(q, k, v, attn_mask):
    """Check shapes/dtypes/devices and return the mask broadcast to [B,Hq,Lq,Lk]."""
    if q.ndim != 4 or k.ndim != 4 or v.ndim != 4:
        raise ValueError("q, k, and v must have shape [batch, heads, sequence, head_dim]")
    if q.dtype not in SUPPORTED_DTYPES:
        raise TypeError(f"q, k, and v must be float32, float16, or bfloat16, got {q.dtype}")
    if q.dtype != k.dtype or q.dtype != v.dtype:
        raise TypeError(
            f"q, k, and v must have the same dtype, got {q.dtype}, {k.dtype}, and {v.dtype}"
        )
    if not q.is_cuda or q.device != k.device or q.device != v.device:
        raise ValueError("q, k, and v must be on the same CUDA device")
    # the device check costs several microseconds: done once per device
    index = q.device.index
    if index is None or index not in _CHECKED_DEVICES:
        if not is_available(q.device):
            raise RuntimeError(UNAVAILABLE)
        if index is not None:
            _CHECKED_DEVICES.add(index)

    batch, q_heads, q_len, head_dim = q.shape
    k_batch, kv_heads, k_len, k_dim = k.shape
    if v.shape != (batch, kv_heads, k_len, head_dim):
        raise ValueError(
            f"v must have shape [q.batch, k.heads, k.sequence, q.head_dim], got {tuple(v.shape)}"
        )
    if k_batch != batch or k_dim != head_dim:
        raise ValueError(
            f"q and k batch/head dimensions must match, got {tuple(q.shape)} and {tuple(k.shape)}"
        )
    if 0 in (batch, q_heads, kv_heads, q_len, k_len):
        raise ValueError("batch, head counts, and sequence lengths must be positive")
    if q_heads % kv_heads != 0:
        raise ValueError(
            f"q head count ({q_heads}) must be divisible by k/v head count ({kv_heads})"
        )
    if head_dim <= 0 or head_dim > 256:
        raise ValueError(f"head_dim must be in [1, 256], got {head_dim}")
    if q.stride(-1) != 1 or k.stride(-1) != 1 or v.stride(-1) != 1:
        raise ValueError("the last dimension of q, k, and v must be contiguous")
    if attn_mask is None:
        return None
    if attn_mask.device != q.device:
        raise ValueError("attn_mask must be on the same CUDA device as q, k, and v")
    if attn_mask.dtype not in MASK_DTYPE_CODES:
        raise TypeError("attn_mask must be bool, float16, bfloat16, or float32")
    try:
        return torch.broadcast_to(attn_mask, (batch, q_heads, q_len, k_len))
    except RuntimeError as error:
        raise ValueError(
            "attn_mask must be broadcastable to "
            f"[{batch}, {q_heads}, {q_len}, {k_len}], got {tuple(attn_mask.shape)}"
        ) from error
