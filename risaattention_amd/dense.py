"""``int8_attention`` and the two operators ``torch.compile`` sees.

Operator names and schemas follow reference src/risa_attention/dense.py:14-77
(``risa_attention::int8_attention`` and ``::int8_attention_masked``, fake
implementations that only propagate the query shape), so graphs traced against the
reference keep working.  Eager calls on plain tensors do not go through them.
"""

from __future__ import annotations

import torch

from .attend import execute_dense_attention, int8_attention_from_prequantized
from .policy import uses_centered_values
from .prepare import prequantize_int8_attention

OP_NAMESPACE = "risa_attention"


def _run(q, k, v, attn_mask, scale, use_midpoint_affine, is_causal):
    return execute_dense_attention(q, k, v, scale=scale, attn_mask=attn_mask,
                                   use_midpoint_affine=use_midpoint_affine, is_causal=is_causal)


def _same_shape_as_query(q, *unused):
    return q.new_empty(q.shape)


@torch.library.custom_op(f"{OP_NAMESPACE}::int8_attention", mutates_args=())
def _dense_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float | None,
              use_midpoint_affine: bool, is_causal: bool) -> torch.Tensor:
    return _run(q, k, v, None, scale, use_midpoint_affine, is_causal)


@torch.library.custom_op(f"{OP_NAMESPACE}::int8_attention_masked", mutates_args=())
def _masked_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, attn_mask: torch.Tensor,
               scale: float | None, use_midpoint_affine: bool, is_causal: bool) -> torch.Tensor:
    return _run(q, k, v, attn_mask, scale, use_midpoint_affine, is_causal)


_dense_op.register_fake(_same_shape_as_query)
_masked_op.register_fake(_same_shape_as_query)


def _plain_eager(*tensors) -> bool:
    """Ordinary tensors with nobody watching the dispatcher: no operator boundary is needed.

    A compile in progress, an active ``TorchDispatchMode`` (``make_fx``, fake or
    functional modes, user modes) and a ``torch.jit.trace`` all record what goes through
    the dispatcher; the native call is invisible to them, so they must see the operator.
    """
    if torch.compiler.is_compiling():
        return False
    if torch._C._len_torch_dispatch_stack() != 0 or torch._C._get_tracing_state() is not None:
        return False
    return all(t is None or type(t) is torch.Tensor for t in tensors)


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
    needs_packed_route = return_lse or kv_permutation is not None
    if needs_packed_route:
        # the LSE and the permuted order live in the packed container
        packed = prequantize_int8_attention(
            q, k, v, scale=scale, attn_mask=attn_mask, v_quantization=v_quantization,
            is_causal=is_causal, return_lse=return_lse, kv_permutation=kv_permutation,
            fuse_gather=fuse_gather,
        )
        return int8_attention_from_prequantized(packed, return_lse=return_lse)
    centered = uses_centered_values(v_quantization)
    # Plain eager tensors skip the operator dispatch (about 10 us per call, a third of a
    # short sequence's whole step); tracing, fake and wrapped tensors go through the
    # registered operators so that torch.compile sees them.
    if _plain_eager(q, k, v, attn_mask):
        return _run(q, k, v, attn_mask, scale, centered, is_causal)
    operators = getattr(torch.ops, OP_NAMESPACE)
    if attn_mask is None:
        return operators.int8_attention(q, k, v, scale, centered, is_causal)
    return operators.int8_attention_masked(q, k, v, attn_mask, scale, centered, is_causal)
