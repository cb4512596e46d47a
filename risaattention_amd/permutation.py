"""Reordering of the key/value tokens, read inside the quantisation kernels.

Public surface of reference src/risa_attention/permutation.py (``KVPermutation``,
``prepare_kv_permutation``); the routing is this build's: the K, anchor and V kernels
read token ``n`` from source row ``perm[n]`` for every dtype and head dim (the
reference fuses BF16 / D=128 only).  A request for the LSE (whose anchor correction
reads K rows itself) or ``fuse_gather=False`` gathers K and V up front instead; both
routes produce the same packed tensors.
"""

from __future__ import annotations

import torch

_INT32_MAX = 2**31 - 1


def _owned_copy(indices: torch.Tensor) -> torch.Tensor:
    """Check that every row of ``indices`` is a permutation and return a private int32 copy.

    The check compares sorted rows with 0..N-1 on the device and reads the verdict back,
    so it synchronises once; it must therefore happen outside graph capture.
    """
    if not isinstance(indices, torch.Tensor) or indices.ndim != 3:
        raise ValueError("permutation must be [B,Hkv,Nkv] int32/int64")
    if indices.dtype not in (torch.int32, torch.int64):
        raise ValueError("permutation must be [B,Hkv,Nkv] int32/int64")
    if indices.numel() == 0 or not indices.is_cuda:
        raise ValueError("permutation must be a nonempty CUDA tensor")
    tokens = indices.shape[2]
    if tokens > _INT32_MAX:
        raise ValueError("permutation is too long for INT32")
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError("prepare the permutation before CUDA graph capture")
    in_order = torch.arange(tokens, device=indices.device, dtype=indices.dtype)
    rows_sorted = torch.sort(indices, dim=2).values
    if not bool((rows_sorted == in_order).all()):
        raise ValueError("each permutation row must contain each token exactly once")
    # A normal (non-inference) tensor, so that later in-place edits bump its version.
    with torch.inference_mode(False):
        return indices.detach().to(dtype=torch.int32, copy=True).contiguous()


class KVPermutation:
    """A validated ``[B, Hkv, Nkv]`` token order, owned by this object.

    Built by :func:`prepare_kv_permutation`.  The copy taken at construction is what the
    kernels read; editing it afterwards is detected through the tensor's version counter.
    """

    __slots__ = ("_indices", "_version")

    def __init__(self, indices: torch.Tensor):
        owned = _owned_copy(indices)
        object.__setattr__(self, "_indices", owned)
        object.__setattr__(self, "_version", owned._version)

    def __setattr__(self, name, value):
        raise AttributeError("KVPermutation is immutable")

    def __repr__(self) -> str:
        return f"KVPermutation(shape={tuple(self._indices.shape)}, device={self._indices.device})"

    def indices_for(self, keys: torch.Tensor) -> torch.Tensor:
        """The int32 index tensor, after checking it still is what was validated and fits ``keys``."""
        stored = self._indices
        if stored._version != self._version:
            raise ValueError("validated permutation was modified")
        if stored.device != keys.device or tuple(stored.shape) != tuple(keys.shape[:3]):
            raise ValueError("permutation must match K batch, heads, length, and device")
        return stored

    def gather(self, tensor: torch.Tensor) -> torch.Tensor:
        """``tensor[b, h, perm[b, h, n], :]`` materialised (the eager route)."""
        rows = self._indices.to(torch.int64).unsqueeze(-1).expand(tensor.shape)
        return torch.gather(tensor, 2, rows)


def prepare_kv_permutation(indices: torch.Tensor) -> KVPermutation:
    """Validate a caller-supplied permutation (one host synchronisation) and take a copy."""
    return KVPermutation(indices)


def prepare_inputs(q, k, v, *, permutation, mask, causal, return_lse, fuse):
    """Decide how a permuted call runs.

    Returns ``(q, k, v, fused_indices)``: either the inputs untouched plus the index
    tensor the kernels read through, or gathered K/V and ``None``.
    """
    if not isinstance(permutation, KVPermutation):
        raise TypeError("use prepare_kv_permutation to validate a permutation first")
    indices = permutation.indices_for(k)
    if causal or mask is not None:
        raise ValueError("K/V permutation requires dense, unmasked, noncausal attention")
    if return_lse or not fuse:
        return q, permutation.gather(k), permutation.gather(v), None
    return q, k, v, indices
