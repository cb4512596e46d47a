"""FP32 retained-mass pattern builder and recall metric (evaluation helpers).

Same results as reference src/risa_attention/reference.py:27-246 — exact FP32
block masses per 128-query chunk, shortest descending prefix reaching theta —
computed with tensor operations on whatever device holds q and k (the
reference restricts them to CUDA; CPU tensors are accepted here so the helpers
also serve as a test oracle for the selector).
"""

from __future__ import annotations

import math

import torch
from torch.nn import functional

from .policy import (
    QUERY_BLOCK_SIZE,
    SUPPORTED_DTYPES,
    apply_score_mask,
    kernel_head_dim,
    mask_signature,
    select_key_block_size,
)
from .types import RetainedMassPattern


def _broadcast_mask(attn_mask, batch, heads, q_len, k_len):
    if attn_mask is None:
        return None
    if attn_mask.dtype not in (torch.bool, torch.float16, torch.bfloat16, torch.float32):
        raise TypeError("attn_mask must be bool, float16, bfloat16, or float32")
    try:
        return torch.broadcast_to(attn_mask, (batch, heads, q_len, k_len))
    except RuntimeError as error:
        raise ValueError(
            f"attn_mask must be broadcastable to [{batch}, {heads}, {q_len}, {k_len}], "
            f"got {tuple(attn_mask.shape)}"
        ) from error


def _check_pair(q, k):
    if q.ndim != 4 or k.ndim != 4:
        raise ValueError("q and k must have shape [batch, heads, sequence, head_dim]")
    if q.dtype not in SUPPORTED_DTYPES or q.dtype != k.dtype:
        raise TypeError("q and k must have the same float32, float16, or bfloat16 dtype")
    if q.device != k.device:
        raise ValueError("q and k must be on the same device")
    batch, q_heads, q_len, dim = q.shape
    if k.shape[0] != batch or k.shape[3] != dim:
        raise ValueError("sparse attention requires self-attention with equal Q/K lengths")
    kv_heads = k.shape[1]
    if 0 in (batch, q_heads, kv_heads, q_len, k.shape[2]):
        raise ValueError("batch, head counts, and sequence length must be positive")
    if q_heads % kv_heads:
        raise ValueError("q head count must be divisible by k head count")
    if dim <= 0 or dim > 256:
        raise ValueError("head_dim must be in [1, 256]")


def _chunk_block_masses(q, k_t, start, end, scale, attn_mask, is_causal, key_block, key_blocks):
    """Block masses [B,Hq,key_blocks] of query rows start..end and their total mass."""
    batch, q_heads, _, dim = q.shape
    kv_heads = k_t.shape[1]
    group = q_heads // kv_heads
    rows = end - start
    chunk = q[:, :, start:end].reshape(batch, kv_heads, group, rows, dim).float()
    scores = torch.matmul(chunk, k_t).mul_(scale).reshape(batch, q_heads, rows, -1)
    scores = apply_score_mask(scores, attn_mask, is_causal, start)
    probabilities = torch.softmax(scores, dim=-1).nan_to_num_(nan=0.0)
    total = float(probabilities.sum())
    k_len = probabilities.shape[-1]
    if k_len % key_block:
        probabilities = functional.pad(probabilities, (0, key_block - k_len % key_block))
    masses = probabilities.reshape(batch, kv_heads, group, rows, key_blocks, key_block)
    return masses.sum(dim=(3, 5)).reshape(batch, q_heads, key_blocks), total


@torch.inference_mode()
def build_retained_mass_pattern(
    q: torch.Tensor,
    k: torch.Tensor,
    *,
    theta: float = 0.99,
    scale: float | None = None,
    attn_mask: torch.Tensor | None = None,
    is_causal: bool = False,
) -> RetainedMassPattern:
    """Frozen retained-mass support from exact FP32 block masses.

    Works in chunks of 128 queries, so the attention matrix is never
    materialised.  Key blocks follow the kernel's tile (64 or 128 keys).
    """
    if not 0.0 < theta <= 1.0 or not math.isfinite(theta):
        raise ValueError("theta must be finite and in (0, 1]")
    _check_pair(q, k)
    batch, q_heads, q_len, dim = q.shape
    k_len = k.shape[2]
    attn_mask = _broadcast_mask(attn_mask, batch, q_heads, q_len, k_len)
    attention_scale = dim**-0.5 if scale is None else float(scale)
    if not math.isfinite(attention_scale):
        raise ValueError("scale must be finite")
    key_block = select_key_block_size(
        kernel_head_dim(dim), k_len, has_mask=attn_mask is not None and attn_mask.stride(-2) != 0
    )
    query_blocks = math.ceil(q_len / QUERY_BLOCK_SIZE)
    key_blocks = math.ceil(k_len / key_block)
    k_t = k.float().transpose(-1, -2).unsqueeze(2)

    support = torch.zeros(batch, q_heads, query_blocks, key_blocks, dtype=torch.bool, device=q.device)
    retained = 0.0
    total = 0.0
    for block in range(query_blocks):
        start = block * QUERY_BLOCK_SIZE
        end = min(start + QUERY_BLOCK_SIZE, q_len)
        masses, _ = _chunk_block_masses(q, k_t, start, end, attention_scale, attn_mask, is_causal,
                                        key_block, key_blocks)
        ordered, order = masses.sort(dim=-1, descending=True)
        target = theta * masses.sum(dim=-1, keepdim=True)
        counts = ((ordered.cumsum(dim=-1) < target).sum(dim=-1) + 1).clamp_(max=key_blocks)
        chosen = torch.arange(key_blocks, device=q.device) < counts[..., None]
        block_support = torch.zeros_like(chosen).scatter_(-1, order, chosen)
        support[:, :, block] = block_support
        retained += float(masses.masked_fill(~block_support, 0.0).double().sum())
        total += float(masses.double().sum())

    flat = support.reshape(-1, key_blocks)
    counts = flat.sum(dim=-1)
    if bool((counts == 0).any()):
        raise RuntimeError("retained-mass construction produced an empty support row")
    row_offsets = torch.zeros(flat.shape[0] + 1, dtype=torch.int32, device=q.device)
    row_offsets[1:] = counts.cumsum(0)
    block_indices = flat.nonzero()[:, 1].to(torch.int32)
    return RetainedMassPattern(
        row_offsets=row_offsets,
        block_indices=block_indices,
        batch_size=batch,
        q_heads=q_heads,
        q_length=q_len,
        kv_length=k_len,
        query_block_size=QUERY_BLOCK_SIZE,
        key_block_size=key_block,
        attention_scale=attention_scale,
        retained_mass_target=float(theta),
        measured_retained_mass=retained / max(total, 1e-20),
        is_causal=is_causal,
        mask_signature=mask_signature(attn_mask),
        mask_reference=attn_mask,
    )


@torch.inference_mode()
def measure_pattern_recall(
    q: torch.Tensor,
    k: torch.Tensor,
    sparse_pattern: RetainedMassPattern,
    *,
    attn_mask: torch.Tensor | None = None,
) -> float:
    """Exact FP32 attention mass kept by a frozen pattern."""
    if not isinstance(sparse_pattern, RetainedMassPattern):
        raise TypeError("sparse_pattern must be returned by build_retained_mass_pattern")
    _check_pair(q, k)
    batch, q_heads, q_len, _ = q.shape
    k_len = k.shape[2]
    attn_mask = _broadcast_mask(attn_mask, batch, q_heads, q_len, k_len)
    if mask_signature(attn_mask) != sparse_pattern.mask_signature:
        raise ValueError("pattern mask has changed")
    if (batch, q_heads, q_len, k_len) != (
        sparse_pattern.batch_size, sparse_pattern.q_heads, sparse_pattern.q_length, sparse_pattern.kv_length
    ):
        raise ValueError("q and k do not match the frozen retained-mass pattern")
    if sparse_pattern.row_offsets.device != q.device:
        raise ValueError("pattern and q/k must be on the same device")
    key_block = sparse_pattern.key_block_size
    query_block = sparse_pattern.query_block_size
    query_blocks = math.ceil(q_len / query_block)
    key_blocks = math.ceil(k_len / key_block)
    rows = batch * q_heads * query_blocks
    counts = (sparse_pattern.row_offsets[1:] - sparse_pattern.row_offsets[:-1]).long()
    row_of_entry = torch.repeat_interleave(torch.arange(rows, device=q.device), counts)
    support = torch.zeros(rows, key_blocks, dtype=torch.bool, device=q.device)
    support[row_of_entry, sparse_pattern.block_indices.long()] = True
    support = support.view(batch, q_heads, query_blocks, key_blocks)
    k_t = k.float().transpose(-1, -2).unsqueeze(2)
    retained = 0.0
    total = 0.0
    for block in range(query_blocks):
        start = block * query_block
        end = min(start + query_block, q_len)
        masses, chunk_total = _chunk_block_masses(q, k_t, start, end, sparse_pattern.attention_scale,
                                                  attn_mask, sparse_pattern.is_causal, key_block, key_blocks)
        retained += float(masses.masked_fill(~support[:, :, block], 0.0).double().sum())
        total += chunk_total
    return retained / max(total, 1e-20)
