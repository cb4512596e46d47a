"""Input contracts, mask helpers and the key-tile policy.

The rules, the exception types and the message texts are the contract of reference
src/risa_attention/_validation.py:11-148 (callers and tests match on them); the device
requirement reads "HIP extension / gfx950" instead of "CUDA extension / SM80+".  The
checks are table-driven here: one entry per rule, applied in the reference's order so
that the first violated rule is the one reported.
"""

from __future__ import annotations

import torch

from . import native

DTYPE_CODES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
MASK_DTYPE_CODES = {**DTYPE_CODES, torch.bool: 3}
SUPPORTED_DTYPES = tuple(DTYPE_CODES)
QUERY_BLOCK_SIZE = 128
KEY_BLOCK_SIZE = 64
LARGE_KEY_BLOCK_SIZE = 128
MIN_PATTERN_SPARSITY = 0.05
OUTPUT_LAYOUTS = ("hnd", "nhd")
VALUE_QUANTIZATION_MODES = ("midpoint_affine", "absmax")

UNAVAILABLE = "INT8 attention requires the risaattention_amd HIP extension and a gfx950 (MI355X) GPU"

# rule -> (exception type, message template)
_RULES = {
    "rank": (ValueError, "q, k, and v must have shape [batch, heads, sequence, head_dim]"),
    "dtype": (TypeError, "q, k, and v must be float32, float16, or bfloat16, got {dtype}"),
    "same_dtype": (TypeError, "q, k, and v must have the same dtype, got {q}, {k}, and {v}"),
    "device": (ValueError, "q, k, and v must be on the same CUDA device"),
    "unavailable": (RuntimeError, UNAVAILABLE),
    "v_shape": (ValueError, "v must have shape [q.batch, k.heads, k.sequence, q.head_dim], got {shape}"),
    "qk_shape": (ValueError, "q and k batch/head dimensions must match, got {q} and {k}"),
    "empty": (ValueError, "batch, head counts, and sequence lengths must be positive"),
    "groups": (ValueError, "q head count ({q}) must be divisible by k/v head count ({kv})"),
    "head_dim": (ValueError, "head_dim must be in [1, 256], got {head_dim}"),
    "stride": (ValueError, "the last dimension of q, k, and v must be contiguous"),
    "mask_device": (ValueError, "attn_mask must be on the same CUDA device as q, k, and v"),
    "mask_dtype": (TypeError, "attn_mask must be bool, float16, bfloat16, or float32"),
    "mask_shape": (ValueError, "attn_mask must be broadcastable to [{b}, {h}, {lq}, {lk}], got {shape}"),
    "v_mode": (ValueError, "v_quantization must be one of {modes}, got {mode!r}"),
}


def _violation(rule: str, **values) -> Exception:
    kind, template = _RULES[rule]
    return kind(template.format(**values))


def uses_centered_values(v_quantization: str) -> bool:
    """True for ``midpoint_affine``, False for ``absmax``; anything else is an error."""
    if v_quantization not in VALUE_QUANTIZATION_MODES:
        raise _violation("v_mode", modes=VALUE_QUANTIZATION_MODES, mode=v_quantization)
    return v_quantization == VALUE_QUANTIZATION_MODES[0]


def mask_signature(mask: torch.Tensor | None) -> tuple | None:
    """What identifies a mask for a retained pattern: its storage, layout and contents version.

    Inference tensors have no version counter (reading it raises); their entry is None and
    the caller must leave them unchanged while a pattern built under them is in use.
    """
    if mask is None:
        return None
    try:
        version = mask._version
    except RuntimeError:
        version = None
    layout = (tuple(mask.shape), tuple(mask.stride()), mask.dtype, mask.device)
    return (mask.data_ptr(), version, *layout)


def apply_score_mask(scores, attn_mask, is_causal, start):
    """Mask FP32 score rows ``start .. start + rows`` the way the kernels do: boolean masks
    hide, floating-point masks add, the causal rule hides keys after the query."""
    rows, keys = scores.shape[-2], scores.shape[-1]
    if attn_mask is not None:
        window = attn_mask.narrow(-2, start, rows)
        scores = scores + window if window.dtype != torch.bool else scores.masked_fill(window.logical_not(), -torch.inf)
    if is_causal:
        query_index = torch.arange(start, start + rows, device=scores.device).unsqueeze(1)
        future = torch.arange(keys, device=scores.device).unsqueeze(0) > query_index
        scores = scores.masked_fill(future, -torch.inf)
    return scores


def pad_key_length(length: int, key_block_size: int = KEY_BLOCK_SIZE) -> int:
    return -(-length // key_block_size) * key_block_size


def kernel_head_dim(head_dim: int) -> int:
    """Head dim the kernels run with: the next of 64, 128, 256."""
    return next(width for width in (64, 128, 256) if head_dim <= width)


def select_key_block_size(kernel_dim: int, key_length: int, *, has_mask: bool) -> int:
    """128-key tiles need a wide head, a long sequence and no query-dependent mask."""
    wide = not has_mask and kernel_dim >= 128 and key_length > 1024
    return LARGE_KEY_BLOCK_SIZE if wide else KEY_BLOCK_SIZE


def is_available(device: torch.device | int | None = None) -> bool:
    return native.is_available(device)


_CHECKED_DEVICES: set[int] = set()  # device indices that passed is_available(): it costs microseconds per call


def _require_device(device: torch.device) -> None:
    index = device.index
    if index is not None and index in _CHECKED_DEVICES:
        return
    if not is_available(device):
        raise _violation("unavailable")
    if index is not None:
        _CHECKED_DEVICES.add(index)


def validate_inputs(q, k, v, attn_mask):
    """Check Q, K, V and the mask; return the mask as a ``[B, Hq, Lq, Lk]`` broadcast view."""
    if q.ndim != 4 or k.ndim != 4 or v.ndim != 4:
        raise _violation("rank")
    dtype, device = q.dtype, q.device
    if dtype not in DTYPE_CODES:
        raise _violation("dtype", dtype=dtype)
    if k.dtype != dtype or v.dtype != dtype:
        raise _violation("same_dtype", q=dtype, k=k.dtype, v=v.dtype)
    if not q.is_cuda or k.device != device or v.device != device:
        raise _violation("device")
    _require_device(device)

    batch, q_heads, q_len, head_dim = q.shape
    kv_heads, k_len = k.shape[1], k.shape[2]
    if tuple(v.shape) != (batch, kv_heads, k_len, head_dim):
        raise _violation("v_shape", shape=tuple(v.shape))
    if (k.shape[0], k.shape[3]) != (batch, head_dim):
        raise _violation("qk_shape", q=tuple(q.shape), k=tuple(k.shape))
    if min(batch, q_heads, kv_heads, q_len, k_len) == 0:
        raise _violation("empty")
    if q_heads % kv_heads:
        raise _violation("groups", q=q_heads, kv=kv_heads)
    if not 1 <= head_dim <= 256:
        raise _violation("head_dim", head_dim=head_dim)
    if q.stride(-1) != 1 or k.stride(-1) != 1 or v.stride(-1) != 1:
        raise _violation("stride")

    if attn_mask is None:
        return None
    if attn_mask.device != q.device:
        raise _violation("mask_device")
    if attn_mask.dtype not in MASK_DTYPE_CODES:
        raise _violation("mask_dtype")
    try:
        return attn_mask.broadcast_to((batch, q_heads, q_len, k_len))
    except RuntimeError as error:
        raise _violation("mask_shape", b=batch, h=q_heads, lq=q_len, lk=k_len,
                         shape=tuple(attn_mask.shape)) from error
