"""``int8_attention`` and its ``torch.compile``-visible operator registration.

Counterpart of reference src/risa_attention/dense.py:14-146: the same two
operators (``risa_attention::int8_attention`` and ``::int8_attention_masked``)
with fake implementations that only propagate the query shape.
"""

from __future__ import annotations

import torch

from .attend import execute_dense_attention, int8_attention_from_prequantized
from .policy import uses_centered_values
from .prepare import prequantize_int8_attention

OP_NAMESPACE = "risa_attention"


@torch.library.custom_op(f"{OP_NAMESPACE}::int8_attention", mutates_args=())
def _dense_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float | None,
              use_midpoint_affine: bool, is_causal: bool) -> torch.Tensor:
    return execute_dense_attention(q, k, v, scale=scale, attn_mask=None,
                                   use_midpoint_affine=use_midpoint_affine, is_causal=is_causal)


@_dense_op.register_fake
def _(q, k, v, scale, use_midpoint_affine, is_causal):
    return q.new_empty(q.shape)


@torch.library.custom_op(f"{OP_NAMESPACE}::int8_attention_masked", mutates_args=())
def _masked_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, attn_mask: torch.Tensor,
               scale: float | None, use_midpoint_affine: bool, is_causal: bool) -> torch.Tensor:
    return execute_dense_attention(q, k, v, scale=scale, attn_mask=attn_mask,
                                   use_midpoint_affine=use_midpoint_affine, is_causal=is_causal)


@_masked_op.register_fake
def _(q, k, v, attn_mask, scale, use_midpoint_affine, is_causal):
    return q.new_empty(q.shape)


def int8_attention(
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
) -> torch.Tensor | tuple[torch.Tensor, torch.Tensor]:
    """Inference SDPA with signed INT8 Q/K/V and unsigned 8-bit probabilities.

    Layout is ``[batch, heads, sequence, head_dim]``; grouped-query attention
    and unequal (non-causal) Q/K lengths are allowed.  The head dim is padded to
    64, 128 or 256 and sliced back.  Q and K get the same block-Hadamard
    rotation before per-group INT8 quantisation (H4 blocks up to 256 keys, H64
    for 64 channels, a signed H128 for 128, plain H128 halves for 256), which
    leaves their dot products unchanged; a sampled key is subtracted from K
    when that narrows its range (softmax invariant).  V is quantised per
    channel, symmetric ``absmax`` by default or ``midpoint_affine`` with a
    residual-corrected centre.  Scores, maxima, exponentials, the denominator
    (taken from the same rounded U8 probabilities as P·V) and V dequantisation
    are FP32.  ``return_lse=True`` also returns natural-log normalisers.
    """
    if return_lse or kv_permutation is not None:
        packed = prequantize_int8_attention(
            q, k, v, scale=scale, attn_mask=attn_mask, v_quantization=v_quantization,
            is_causal=is_causal, return_lse=return_lse, kv_permutation=kv_permutation,
            fuse_gather=fuse_gather,
        )
        return int8_attention_from_prequantized(packed, return_lse=return_lse)
    use_midpoint_affine = uses_centered_values(v_quantization)
    # Plain eager tensors skip the operator dispatch (about 10 us per call, a third of a
    # short sequence's whole step); tracing, fake and wrapped tensors go through the
    # registered operators so that torch.compile sees them.
    if (type(q) is torch.Tensor and type(k) is torch.Tensor and type(v) is torch.Tensor
            and (attn_mask is None or type(attn_mask) is torch.Tensor)
            and not torch.compiler.is_compiling()):
        return execute_dense_attention(q, k, v, scale=scale, attn_mask=attn_mask,
                                       use_midpoint_affine=use_midpoint_affine, is_causal=is_causal)
    ops = getattr(torch.ops, OP_NAMESPACE)
    if attn_mask is None:
        return ops.int8_attention(q, k, v, scale, use_midpoint_affine, is_causal)
    return ops.int8_attention_masked(q, k, v, attn_mask, scale, use_midpoint_affine, is_causal)
