"""Validated K/V token permutation, fused into quantisation or applied eagerly.

Counterpart of reference src/risa_attention/permutation.py:1-52.  The
reference fuses the gather into its BF16/D128 quantisers only; here the K, anchor
and V kernels read through the permutation for every dtype and head dim.  As in
the reference, ``return_lse`` (whose anchor correction reads K rows itself) and
``fuse_gather=False`` take the eager gather; both routes give the same tensors.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True, init=False)
class KVPermutation:
    """An owned int32 ``[B,Hkv,Nkv]`` permutation, checked once at construction."""

    _indices: torch.Tensor
    _version: int

    def __init__(self, indices: torch.Tensor):
        if indices.ndim != 3 or indices.dtype not in (torch.int32, torch.int64):
            raise ValueError("permutation must be [B,Hkv,Nkv] int32/int64")
        if not indices.is_cuda or indices.numel() == 0:
            raise ValueError("permutation must be a nonempty CUDA tensor")
        if indices.shape[-1] > 2**31 - 1:
            raise ValueError("permutation is too long for INT32")
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("prepare the permutation before CUDA graph capture")
        identity = torch.arange(indices.shape[-1], device=indices.device).expand_as(indices)
        if not torch.equal(indices.sort(-1).values, identity):
            raise ValueError("each permutation row must contain each token exactly once")
        with torch.inference_mode(False):
            owned = indices.to(torch.int32).clone().contiguous()
        object.__setattr__(self, "_indices", owned)
        object.__setattr__(self, "_version", owned._version)


def prepare_kv_permutation(indices: torch.Tensor) -> KVPermutation:
    """Validate (synchronises) and copy a caller-supplied permutation."""
    return KVPermutation(indices)


def prepare_inputs(q, k, v, *, permutation, mask, causal, return_lse, fuse):
    if not isinstance(permutation, KVPermutation):
        raise TypeError("use prepare_kv_permutation to validate a permutation first")
    perm = permutation._indices
    if perm._version != permutation._version:
        raise ValueError("validated permutation was modified")
    if perm.device != k.device or perm.shape != k.shape[:3]:
        raise ValueError("permutation must match K batch, heads, length, and device")
    if mask is not None or causal:
        raise ValueError("K/V permutation requires dense, unmasked, noncausal attention")
    if fuse and not return_lse:
        return q, k, v, perm
    index = perm.long()[..., None].expand_as(k)
    return q, k.gather(2, index), v.gather(2, index), None
